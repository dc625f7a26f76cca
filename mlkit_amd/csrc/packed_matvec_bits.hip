// One code width of the chunked packed matvec: compiled once per width with
// -DMK_MATVEC_BITS=<2..8> so the widths build in parallel.
#include "packed_matvec_impl.h"

#ifndef MK_MATVEC_BITS
#error "compile with -DMK_MATVEC_BITS=<2..8>"
#endif

#define MK_CONCAT_(a, b) a##b
#define MK_CONCAT(a, b) MK_CONCAT_(a, b)

bool MK_CONCAT(mk_matvec_launch_b, MK_MATVEC_BITS)(const mk_matvec::MatvecArgs &args,
                                                   const mk_matvec::Plan &plan, int x_dtype,
                                                   bool uniform, hipStream_t stream) {
    return mk_matvec::dispatch_bits<MK_MATVEC_BITS>(args, plan, x_dtype, uniform, stream);
}
