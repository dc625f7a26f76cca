// Online input rotation followed by the packed matvec, enqueued from one call.
//
// A rotated layer (the reference's `rotate_inputs` forward pre-hook,
// conversion/model_transforms.py:116-128 in /root/reference/src/mlkit, in front of
// PackedLinear.forward, inference/packed_linear.py:148-245) multiplies its packed weight with
// T(x * signs), T = (basis (x) H_power) / sqrt(power) along the input width.  The rotated
// activations are at most 8 x 16384 values: they are written to a small buffer by the
// row-rotation kernel (mk_rotate_rows: order * samples short workgroups) and read back, from
// L2, by the matvec kernel enqueued right behind it on the same stream.  One library call replaces a Python hook, an
// allocation and two calls.  One fp16 or bf16 sample of an INT4 layer whose transform has no
// basis (a power-of-two row of 2048 to 16384 codes, or separate power-of-two blocks of a row of
// whole 2048-code slices) needs neither the buffer nor the second launch: the matvec kernel
// transforms the activations itself (rotate_inside_the_matvec).

#include <mutex>

#include "packed_matvec_impl.h"

namespace {

// One fp16 or bf16 sample, INT4 codes on a uniform grid with 16-bit scales, a row of whole
// 2048-code slices transformed in blocks of `block` values (the whole row: one block) and whole
// tiles of rows: the matvec kernel rotates the activations itself while its first codes are on
// their way (no second launch, no buffer).  Returns 1 when it took the
// call, 0 when the shape is not one of these, a negative status on errors.
int rotate_inside_the_matvec(const void *x, int x_dtype, int block, const float *signs, float scale, const uint8_t *packed,
                             const void *scales, int scale_dtype, const void *zeros, const void *bias, int bias_dtype,
                             void *y, int samples, int output_width, int input_width, int group, int bits, int uniform,
                             float grid_min, float grid_step, hipStream_t stream) {
    if (samples != 1 || (x_dtype != MK_F16 && x_dtype != MK_BF16) || (scale_dtype != MK_F16 && scale_dtype != MK_BF16) || !packed ||
        !scales || !y || group < 1 || output_width < 1)
        return 0;
    if (!mk_matvec::stream4_accepts(samples, input_width, group, bits, x_dtype, scale_dtype, uniform != 0)) return 0;
    const auto misaligned = [](const void *pointer, uintptr_t mask) { return (reinterpret_cast<uintptr_t>(pointer) & mask) != 0; };
    if (misaligned(packed, 3) || misaligned(scales, 3) || misaligned(zeros, 3) || misaligned(bias, 3) || misaligned(x, 15))
        return 0;
    if (bias && !mk_dtype_valid(bias_dtype)) return 0;
    mk_matvec::Stream4Args a;
    a.x = x; a.packed = packed; a.scales = scales; a.zeros = zeros; a.bias = bias; a.y = y;
    a.samples = samples; a.rows = output_width; a.width = input_width; a.group = group;
    a.groups = mk_cdiv(input_width, group); a.bias_dtype = bias_dtype; a.grid_min = grid_min; a.grid_step = grid_step;
    a.values = nullptr; a.n_values = 0; a.uniform = uniform; a.bits = bits;
    a.x_dtype = x_dtype; a.scale_dtype = scale_dtype;
    a.rotate_signs = signs; a.rotate_scale = scale;
    while ((1 << a.rotate_log_block) < block) ++a.rotate_log_block;
    const int launched = mk_matvec::stream4_launch_rotating(a, stream);
    if (launched == -2) return 0;
    if (launched) return -mk_fail(MK_ERR_HIP, "mk_rotated_packed_matvec: the runtime refused the kernel's LDS size");
    return 1;
}

int rotate_then_multiply(const void *x, int x_dtype, void *rotated, int order, int power, const float *basis,
                         const float *signs, float scale, const uint8_t *packed, const void *scales, int scale_dtype,
                         const float *values, int n_values, const void *zeros, const void *bias, int bias_dtype, void *y,
                         int samples, int output_width, int input_width, int group, int bits, int uniform,
                         float grid_min, float grid_step, void *stream) {
    MK_REQUIRE(x && rotated && x != rotated, MK_ERR_INVALID,
               "mk_rotated_packed_matvec: activations and their rotated copy must be two buffers");
    MK_REQUIRE(order >= 1 && power >= 1 && static_cast<long long>(order) * power == input_width, MK_ERR_INVALID,
               "mk_rotated_packed_matvec: order * power must equal the input width (%d * %d != %d)", order, power,
               input_width);
    // Without a basis: Walsh-Hadamard transforms of the row's `order` blocks, each for itself.
    const bool block_diagonal = order > 1 && !basis;
    MK_REQUIRE(!block_diagonal || (power >= 32 && (power & (power - 1)) == 0), MK_ERR_UNSUPPORTED,
               "mk_rotated_packed_matvec: blocks transformed one by one need a power-of-two length of at least 32 (got %d)",
               power);
    // The rotation runs on order * samples short workgroups (mk_rotate_rows); a plain
    // power-of-two width is split as H_width = H_blocks (x) H_points with about sqrt(width)
    // points per block.
    int status;
    if (order == 1 || block_diagonal) {
        MK_REQUIRE(block_diagonal || ((input_width & (input_width - 1)) == 0 && input_width >= 32), MK_ERR_UNSUPPORTED,
                   "mk_rotated_packed_matvec: a Walsh-Hadamard rotation needs a power-of-two width of at least 32");
        const int inside = rotate_inside_the_matvec(x, x_dtype, power, signs, scale, packed, scales, scale_dtype, zeros, bias,
                                                    bias_dtype, y, samples, output_width, input_width, group, bits, uniform,
                                                    grid_min, grid_step, static_cast<hipStream_t>(stream));
        if (inside < 0) return -inside;
        if (inside > 0) {
            MK_LAUNCH_CHECK("mk_rotated_packed_matvec");
            return MK_OK;
        }
    }
    if (block_diagonal) {
        status = mk_fwht(x, x_dtype, rotated, x_dtype, static_cast<long long>(samples) * order, power, signs, nullptr,
                         input_width, scale, stream);
    } else if (order == 1) {
        int points = 32;
        while (points * points < input_width && points < 1024) points *= 2;
        status = mk_rotate_rows(x, x_dtype, rotated, x_dtype, samples, input_width / points, points, nullptr, signs, scale,
                                stream);
    } else {
        status = mk_rotate_rows(x, x_dtype, rotated, x_dtype, samples, order, power, basis, signs, scale, stream);
    }
    if (status) return status;
    return mk_packed_matvec(rotated, x_dtype, packed, scales, scale_dtype, values, n_values, zeros, bias, bias_dtype, y,
                            samples, output_width, input_width, group, bits, uniform, grid_min, grid_step, stream);
}

}  // namespace

extern "C" int mk_rotated_packed_matvec(const void *x, int x_dtype, void *rotated, int order, int power,
                                        const float *basis, const float *signs, float scale, const uint8_t *packed,
                                        const void *scales, int scale_dtype, const float *values, int n_values,
                                        const void *zeros, const void *bias, int bias_dtype, void *y, int samples,
                                        int output_width, int input_width, int group, int bits, int uniform,
                                        float grid_min, float grid_step, void *stream) {
    return rotate_then_multiply(x, x_dtype, rotated, order, power, basis, signs, scale, packed, scales, scale_dtype, values,
                                n_values, zeros, bias, bias_dtype, y, samples, output_width, input_width, group, bits,
                                uniform, grid_min, grid_step, stream);
}

// ---- the same without a buffer from the caller ---------------------------------------------
//
// For callers that cannot allocate (code under HIP graph capture, serving loops that own no
// allocator): the rotated activations go to a fixed array in the library's own device
// memory.  Every GPU the library runs on holds one copy of the array until the process ends;
// all calls on a GPU share it, so calls that overlap on one GPU (two streams) race.

namespace {

constexpr size_t kStaticRotatedBytes = 512 * 1024;  // 8 rows x 16384 values x 4 bytes
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kStaticRotatedBytes];

// The device address of `scratch` on the current device, looked up once per device.  (In host
// code the array's name is only a handle for this lookup, not an address a kernel can use.)
int static_rotated_buffer(void **buffer) {
    static std::mutex guard;
    static void *address[kMaxDevices];
    int device = 0;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess || device < 0 || device >= kMaxDevices)
        return mk_fail(MK_ERR_HIP, "mk_rotated_packed_matvec_static: no current device (%s)", hipGetErrorString(status));
    std::lock_guard<std::mutex> lock(guard);
    if (!address[device]) {
        void *found = nullptr;
        status = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
        if (status != hipSuccess || !found)
            return mk_fail(MK_ERR_HIP, "mk_rotated_packed_matvec_static: the library's buffer has no address on device %d (%s)",
                           device, hipGetErrorString(status));
        address[device] = found;
    }
    *buffer = address[device];
    return MK_OK;
}

}  // namespace

extern "C" int mk_rotated_packed_matvec_static(const void *x, int x_dtype, int order, int power, const float *basis,
                                               const float *signs, float scale, const uint8_t *packed,
                                               const void *scales, int scale_dtype, const float *values,
                                               int n_values, const void *zeros, const void *bias, int bias_dtype,
                                               void *y, int samples, int output_width, int input_width, int group,
                                               int bits, int uniform, float grid_min, float grid_step, void *stream) {
    MK_REQUIRE(mk_dtype_valid(x_dtype) && samples >= 1 && input_width >= 1, MK_ERR_INVALID,
               "mk_rotated_packed_matvec_static: unknown dtype code or empty input");
    const unsigned long long needed = static_cast<unsigned long long>(samples) * input_width * mk_dtype_bytes(x_dtype);
    MK_REQUIRE(needed <= kStaticRotatedBytes, MK_ERR_INVALID,
               "mk_rotated_packed_matvec_static: %d x %d activations of %d bytes need %llu bytes, the library's buffer "
               "holds %llu; use mk_rotated_packed_matvec with a buffer of the caller's",
               samples, input_width, mk_dtype_bytes(x_dtype), needed, static_cast<unsigned long long>(kStaticRotatedBytes));
    void *rotated = nullptr;
    if (int status = static_rotated_buffer(&rotated)) return status;
    return rotate_then_multiply(x, x_dtype, rotated, order, power, basis, signs, scale, packed, scales, scale_dtype, values,
                                n_values, zeros, bias, bias_dtype, y, samples, output_width, input_width, group, bits,
                                uniform, grid_min, grid_step, stream);
}
