// Rotation of a few activation rows, spread over many workgroups.
//
// T = (basis (x) H_power) along a row of order * power values.  For activations (one to a
// few rows) the transform is latency: a row handled by one workgroup keeps one compute unit
// busy for many microseconds.  By linearity
//     out[f', :] = sum_f basis[f', f] * H(x[f, :]) = H( sum_f basis[f', f] * x[f, :] ),
// so the workgroup of output block f' first mixes the `order` input blocks (order multiply-adds
// per thread, every input value read once per workgroup, from L2) and then runs ONE
// Walsh-Hadamard transform of `power` points: order * rows independent workgroups, each
// short.  A plain power-of-two width W is the same with basis = the +-1 Hadamard matrix of
// order W / power (H_W = H_order (x) H_power in natural order).
//
// The sums are the transform's own sums in another order than transform-then-mix, so results
// agree with mk_fwht / mk_rotate_blocks to fp32 rounding, not bit for bit.
//
// Replaces: the rotate_inputs forward pre-hook of conversion/model_transforms.py:116-128
// (randomized_transform, quantization/operations/orthogonal_transforms.py:101-122) for
// activations, in /root/reference/src/mlkit.

#include "mk_common.h"

namespace {

struct RowsArgs {
    const void *source;
    void *target;
    const float *basis;   // [order, order] row-major, or null: +-1 Hadamard matrix of size `order`
    const float *signs;   // [order * power] or null
    int order, power, log_power;
    int splits;           // threads per point of a block
    int source_dtype, target_dtype;
    float scale;
};

// One workgroup of power * splits threads per (output block, row).  Thread (s, p) mixes the
// inputs f = s, s + splits, s + 2 splits, ... of point p: at most sixteen independent loads
// from L2 (or HBM), all requested before any is used, so the workgroup waits for memory about
// once.  The partial sums of a point meet in LDS and are added in the order of s; the threads
// of s = 0 then run the Walsh-Hadamard stages.
template <int SOURCE>
__global__ void __launch_bounds__(1024) rotate_rows_kernel(const RowsArgs a) {
    __shared__ float exchange[1024];   // the partial sums of a point's splits
    __shared__ float across[1024];     // the block between its wavefronts
    constexpr int kBatch = 16;
    const int p = threadIdx.x % a.power;
    const int split = threadIdx.x / a.power;
    const int block = blockIdx.x;
    const size_t row_start = static_cast<size_t>(blockIdx.y) * a.order * a.power;
    const float *coefficients = a.basis ? a.basis + static_cast<size_t>(block) * a.order : nullptr;  // uniform
    float mixed = 0.0f;
    for (int first = split; first < a.order; first += kBatch * a.splits) {
        float value[kBatch], sign[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int wanted = first + j * a.splits;
            const int f = wanted < a.order ? wanted : a.order - 1;  // past the end: a repeat, weighted zero below
            const size_t column = static_cast<size_t>(f) * a.power + p;
            if constexpr (SOURCE == MK_F32) {
                value[j] = static_cast<const float *>(a.source)[row_start + column];
            } else {
                const uint16_t raw = static_cast<const uint16_t *>(a.source)[row_start + column];
                value[j] = SOURCE == MK_F16 ? static_cast<float>(__builtin_bit_cast(_Float16, raw)) : mk_bf16_to_float(raw);
            }
            sign[j] = a.signs ? a.signs[column] : 1.0f;
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int f = first + j * a.splits;
            float weight = 0.0f;
            if (f < a.order) {
                if (coefficients) weight = coefficients[f];
                else weight = (__builtin_popcount(block & f) & 1) ? -1.0f : 1.0f;  // entry (block, f) of the Hadamard matrix
            }
            mixed = __builtin_fmaf(weight, value[j] * sign[j], mixed);
        }
    }
    if (a.splits > 1) {
        exchange[threadIdx.x] = mixed;
        __syncthreads();
        if (split == 0)
            for (int s = 1; s < a.splits; ++s) mixed += exchange[s * a.power + p];
    }
    // Walsh-Hadamard over the block's `power` values, strides ascending: those below 64 inside the wavefront;
    // for the rest every thread reads the value of its lane in each of the block's wavefronts (at most sixteen)
    // after ONE barrier and runs their stages in registers, the same additions as stage by stage through LDS.
    for (int stage = 0; stage < a.log_power && stage < 6; ++stage) {
        const int stride = 1 << stage;
        const float partner = __shfl_xor(mixed, stride, 64);
        mixed = (p & stride) ? partner - mixed : mixed + partner;
    }
    if (a.log_power > 6) {  // uniform
        if (split == 0) across[p] = mixed;
        __syncthreads();
        const int slices = a.power >> 6, own = p >> 6, lane = p & 63;
        float v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = across[(j < slices ? j : 0) * 64 + lane];
#pragma unroll
        for (int bit = 1; bit < 16; bit <<= 1) {
            if (bit < slices) {  // uniform
                float next[16];
#pragma unroll
                for (int j = 0; j < 16; ++j) next[j] = (j & bit) ? v[j ^ bit] - v[j] : v[j] + v[j ^ bit];
#pragma unroll
                for (int j = 0; j < 16; ++j) v[j] = next[j];
            }
        }
#pragma unroll
        for (int j = 0; j < 16; ++j)
            if (j == own) mixed = v[j];
    }
    if (split == 0)
        mk_store_from_float(a.target, row_start + static_cast<size_t>(block) * a.power + p, a.target_dtype, mixed * a.scale);
}

}  // namespace

extern "C" int mk_rotate_rows(const void *source, int source_dtype, void *target, int target_dtype, int rows,
                              int order, int power, const float *basis, const float *signs, float scale,
                              void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(rows >= 0 && rows <= 65535 && order >= 1 && order <= 65535, MK_ERR_INVALID,
               "mk_rotate_rows: at most 65535 rows and blocks per row");
    MK_REQUIRE(power >= 1 && (power & (power - 1)) == 0, MK_ERR_INVALID,
               "mk_rotate_rows: the block width must be a power of two (got %d)", power);
    MK_REQUIRE(power >= 32 && power <= 1024, MK_ERR_UNSUPPORTED,
               "mk_rotate_rows: blocks of 32 to 1024 values (got %d)", power);
    MK_REQUIRE(basis || (order & (order - 1)) == 0, MK_ERR_INVALID,
               "mk_rotate_rows: without a basis the number of blocks must be a power of two (got %d)", order);
    if (rows == 0) return MK_OK;
    MK_REQUIRE(source && target && source != target, MK_ERR_INVALID,
               "mk_rotate_rows: source and target must be two buffers");
    MK_REQUIRE(mk_dtype_valid(source_dtype) && mk_dtype_valid(target_dtype), MK_ERR_INVALID,
               "mk_rotate_rows: unknown dtype code");
    RowsArgs a{};
    a.source = source; a.target = target; a.basis = basis; a.signs = signs; a.order = order; a.power = power;
    a.source_dtype = source_dtype; a.target_dtype = target_dtype; a.scale = scale;
    while ((1 << a.log_power) < power) ++a.log_power;
    a.splits = mk_cdiv(order, 16);
    if (a.splits * power > 1024) a.splits = 1024 / power;
    const dim3 grid(order, rows), block(power * a.splits);
    if (source_dtype == MK_F32) hipLaunchKernelGGL(rotate_rows_kernel<MK_F32>, grid, block, 0, stream, a);
    else if (source_dtype == MK_F16) hipLaunchKernelGGL(rotate_rows_kernel<MK_F16>, grid, block, 0, stream, a);
    else hipLaunchKernelGGL(rotate_rows_kernel<MK_BF16>, grid, block, 0, stream, a);
    MK_LAUNCH_CHECK("mk_rotate_rows");
    return MK_OK;
}
