/* C ABI of libmlkit_amd.so: the gfx950 kernels behind mlkit's packed-inference and
 * fused-quantization path.
 *
 * Conventions
 *   - every pointer is a device pointer owned by the caller unless it says "host";
 *     the library allocates nothing and retains nothing;
 *   - `stream` is a hipStream_t (NULL = the default stream); every entry point only
 *     enqueues work on it and returns without synchronising;
 *   - return value 0 = enqueued; nonzero = nothing was launched (MK_ERR_*), and
 *     mk_last_error() describes why (per host thread);
 *   - dtype codes: MK_F32 = 0, MK_F16 = 1, MK_BF16 = 2.
 *
 * Each declaration names the reference interface (path under /root/reference/src/mlkit)
 * whose launch it replaces.
 */
#ifndef MLKIT_AMD_H
#define MLKIT_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MK_F32 0
#define MK_F16 1
#define MK_BF16 2

#define MK_OK 0
#define MK_ERR_INVALID 1     /* shape / dtype / alignment the entry point does not accept */
#define MK_ERR_UNSUPPORTED 2 /* valid request with no kernel (e.g. a layout that splits a word) */
#define MK_ERR_HIP 3         /* the HIP runtime reported an error at launch */

/* Library version, "major.minor.patch". */
const char *mk_version(void);

/* Message of the last nonzero status returned to this host thread ("" if none). */
const char *mk_last_error(void);

/* 1 when (bits, input_width, group) has a fused layout, i.e. rows and scale groups hold
 * whole packing words and a tile has at least 16 codes; 0 otherwise.
 * Replaces: kernels/packed_linear.py:63-79 (layout_for is None / not None). */
int mk_packed_layout_supported(int bits, int input_width, int group);

/* y[m, n] = sum_k dequant(code[n, k]) * x[m, k] (+ bias[n]), fp32 accumulate, y in x's dtype.
 * dequant(c) = (uniform ? grid_min + c*grid_step : values[c]) * scales[n, k/group] (+ zeros[n, k/group]).
 *   x       [samples, input_width]   x_dtype, contiguous
 *   packed  little-endian bit stream of [output_width, input_width] codes of `bits` bits
 *   scales  [output_width, groups] scale_dtype, groups = ceil(input_width / group)
 *   values  [n_values] fp32 (n_values <= 2^bits); read only when uniform == 0
 *   zeros   NULL or same shape/dtype as scales
 *   bias    NULL or [output_width] bias_dtype
 *   y       [samples, output_width] x_dtype
 * Any samples >= 1 is accepted (the caller applies its own fused-row limit).
 * Replaces: kernels/packed_linear.py:181-226 (matrix_vector) and the direct launch of
 * packed_matrix_vector in inference/packed_linear.py:181-245. */
int mk_packed_matvec(const void *x, int x_dtype, const uint8_t *packed, const void *scales,
                     int scale_dtype, const float *values, int n_values, const void *zeros,
                     const void *bias, int bias_dtype, void *y, int samples, int output_width,
                     int input_width, int group, int bits, int uniform, float grid_min,
                     float grid_step, void *stream);

/* out[n, k] = dequant(code[n, k]) in out_dtype, same dequantisation as mk_packed_matvec
 * with multiply and add kept separate (no fused multiply-add).
 * Replaces: kernels/packed_linear.py:279-313 (decode / decode_rows). */
int mk_packed_decode(const uint8_t *packed, const void *scales, int scale_dtype,
                     const float *values, int n_values, const void *zeros, void *out,
                     int out_dtype, int output_width, int input_width, int group, int bits,
                     int uniform, float grid_min, float grid_step, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MLKIT_AMD_H */
