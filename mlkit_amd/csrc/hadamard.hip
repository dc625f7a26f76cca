// Fast Walsh-Hadamard transform along rows on gfx950, one launch per tensor.
//
// A row of n = 2^S values goes through S radix-2 butterfly stages in ascending stride
// (1, 2, 4, ...): out[i] = a + b, out[i + stride] = a - b.  Every output of a stage depends
// on exactly two outputs of the stage before it, so grouping stages (several in registers,
// exchanges through LDS between groups) changes no bit of the result as long as the stage
// order is kept.  The last step multiplies by `scale` (fp32(1)/fp32(sqrt n) to normalise).
//
// One workgroup owns whole rows: a row is read from HBM once (coalesced, cast to fp32,
// optionally multiplied by a +-1 sign vector), lives in LDS between stage groups, and is
// written once (optionally multiplied by the sign vector, cast to the output type).
// Rows shorter than a workgroup's worth of elements share a workgroup.
//
// The blocked transform of a width that is not a power of two (order x power, e.g.
// 14336 = 28 x 512) runs this kernel on rows * order rows of `power` values and then
// `mk_basis_mix`, which multiplies the `order` blocks of every row by a dense orthonormal
// basis.
//
// Replaces, in /root/reference/src/mlkit:
//   kernels/hadamard.py:21-136                            hadamard_pass / transform -> mk_fwht
//   quantization/operations/orthogonal_transforms.py:101-109  basis product of
//                                                         structured_transform      -> mk_basis_mix

#include "mk_common.h"

#include <atomic>

namespace {

constexpr int kMaxThreads = 1024;
constexpr long long kLeanRotationRows = 256;  // above this many outer rows mk_rotate_blocks streams with rotate_matrix_kernel

struct FwhtArgs {
    const void *source;
    void *target;
    const float *signs_before;  // multiplied into the input, or null
    const float *signs_after;   // multiplied into the output, or null
    long long rows;
    int width, log_width;
    int source_dtype, target_dtype;
    int sign_period;  // signs repeat every sign_period elements of the flattened tensor
    int rows_per_block, threads_per_row;
    float scale;
    // Blocked transform in one launch: `rows` counts blocks of `width` values, every `order`
    // of them form one outer row, which a workgroup transforms and then mixes with `basis`.
    const float *basis;  // [order, order] row-major, or null
    int order, transpose;
};

typedef float mk_mix16 __attribute__((ext_vector_type(16)));

__host__ __device__ __forceinline__ int padded(int index) { return index + (index >> 4); }

// E values per thread; stage group `g` covers index bits [base, base + log2 E).
// TILES > 0: the workgroup's rows are the `order` blocks of one outer row; after the last
// stage they stay in LDS and are multiplied by the basis (padded to TILES x 32 rows) on the
// fp32 matrix cores, exactly as basis_mix_mfma_kernel does from global memory.  The
// workgroup is then a whole number of wavefronts; threads beyond the rows' share only take
// part in that product.
template <int E, bool VEC, int TILES>
__global__ void __launch_bounds__(kMaxThreads) fwht_kernel(const FwhtArgs a) {
    extern __shared__ float tile[];
    constexpr int kLogE = E == 1 ? 0 : E == 2 ? 1 : E == 4 ? 2 : E == 8 ? 3 : E == 16 ? 4 : 5;
    const int threads_per_row = a.threads_per_row;
    const int wanted_row = threadIdx.x / threads_per_row;
    const bool working = wanted_row < a.rows_per_block;
    const int local_row = working ? wanted_row : 0;
    const int t = threadIdx.x - wanted_row * threads_per_row;
    const long long row = static_cast<long long>(blockIdx.x) * a.rows_per_block + local_row;
    const bool active = working && row < a.rows;
    float *mine = tile + local_row * padded(a.width);
    const size_t row_base = static_cast<size_t>(active ? row : 0) * a.width;
    const int sign_base = a.sign_period ? static_cast<int>(row_base % static_cast<size_t>(a.sign_period)) : 0;

    // The basis goes to LDS behind the rows (read back as the left MFMA operand).
    float *basis_tile = tile + a.rows_per_block * padded(a.width);
    if constexpr (TILES > 0) {
        for (int i = threadIdx.x; i < a.order * a.order; i += blockDim.x) basis_tile[i] = a.basis[i];
    }

    // HBM -> LDS.  All loads of a thread are issued before any is used; with VEC a thread
    // reads groups of four adjacent elements (16 bytes of fp32, 8 of fp16 / bf16).
    if (active) {
        float staged[E];
        if constexpr (VEC) {
            constexpr int kQuads = E / 4;
            if (a.source_dtype == MK_F32) {
                const float4 *source = reinterpret_cast<const float4 *>(static_cast<const float *>(a.source) + row_base);
                float4 loaded[kQuads];
#pragma unroll
                for (int q = 0; q < kQuads; ++q) loaded[q] = source[q * threads_per_row + t];
#pragma unroll
                for (int q = 0; q < kQuads; ++q) {
                    staged[4 * q] = loaded[q].x; staged[4 * q + 1] = loaded[q].y;
                    staged[4 * q + 2] = loaded[q].z; staged[4 * q + 3] = loaded[q].w;
                }
            } else {
                const mk_u32x2 *source = reinterpret_cast<const mk_u32x2 *>(static_cast<const uint16_t *>(a.source) + row_base);
                mk_u32x2 loaded[kQuads];
#pragma unroll
                for (int q = 0; q < kQuads; ++q) loaded[q] = source[q * threads_per_row + t];
#pragma unroll
                for (int q = 0; q < kQuads; ++q)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint32_t word = i < 2 ? loaded[q].x : loaded[q].y;
                        const uint16_t raw = static_cast<uint16_t>((i & 1) ? word >> 16 : word);
                        staged[4 * q + i] = a.source_dtype == MK_F16 ? static_cast<float>(__builtin_bit_cast(_Float16, raw))
                                                                     : mk_bf16_to_float(raw);
                    }
            }
            if (a.signs_before) {
                const float4 *signs = reinterpret_cast<const float4 *>(a.signs_before + sign_base);
#pragma unroll
                for (int q = 0; q < kQuads; ++q) {
                    const float4 sign = signs[q * threads_per_row + t];
                    staged[4 * q] *= sign.x; staged[4 * q + 1] *= sign.y;
                    staged[4 * q + 2] *= sign.z; staged[4 * q + 3] *= sign.w;
                }
            }
#pragma unroll
            for (int q = 0; q < kQuads; ++q)
#pragma unroll
                for (int i = 0; i < 4; ++i) mine[padded((q * threads_per_row + t) * 4 + i)] = staged[4 * q + i];
        } else {
#pragma unroll
            for (int j = 0; j < E; ++j) {
                const int index = j * threads_per_row + t;
                float value = mk_load_as_float(a.source, row_base + index, a.source_dtype);
                if (a.signs_before) value *= a.signs_before[sign_base + index];
                mine[padded(index)] = value;
            }
        }
    }
    __syncthreads();

    float v[E];
    int done = 0;
    while (true) {
        // This group holds index bits [base, base + kLogE) in registers; the last group is
        // shifted down to stay inside the row and skips the stages already done.
        int base = done;
        if (base + kLogE > a.log_width) base = a.log_width - kLogE;
        const int low = t & ((1 << base) - 1);
        const int high = t >> base;
        const int origin = (high << (base + kLogE)) | low;
#pragma unroll
        for (int j = 0; j < E; ++j) v[j] = mine[padded(origin | (j << base))];
#pragma unroll
        for (int bit = 0; bit < kLogE; ++bit) {
            if (base + bit >= done) {
#pragma unroll
                for (int j = 0; j < E; ++j) {
                    if ((j >> bit) & 1) continue;
                    const float first = v[j], second = v[j | (1 << bit)];
                    v[j] = first + second;
                    v[j | (1 << bit)] = first - second;
                }
            }
        }
        done = base + kLogE;
        if (done >= a.log_width) {
            if constexpr (TILES > 0) {
                if (working) {
#pragma unroll
                    for (int j = 0; j < E; ++j) mine[padded(origin | (j << base))] = v[j] * a.scale;
                }
            } else if (active) {
#pragma unroll
                for (int j = 0; j < E; ++j) {
                    const int index = origin | (j << base);
                    float value = v[j] * a.scale;
                    if (a.signs_after) value *= a.signs_after[sign_base + index];
                    mk_store_from_float(a.target, row_base + index, a.target_dtype, value);
                }
            }
            break;
        }
        if (working) {
#pragma unroll
            for (int j = 0; j < E; ++j) mine[padded(origin | (j << base))] = v[j];
        }
        __syncthreads();
    }

    if constexpr (TILES > 0) {
        // target[f', p] = sum_f mix[f', f] * block f [p] over ascending f from zero; a wavefront
        // owns 32 adjacent p at a time, lanes 0..31 reading block f and lanes 32..63 block f + 1.
        __syncthreads();
        constexpr int kMaxPairs = TILES * 16;
        const int lane = threadIdx.x & 63;
        const int half = lane >> 5, within = lane & 31;
        const int pairs = (a.order + 1) >> 1;
        float left[TILES][kMaxPairs];  // left[tile][q]: mix[32 tile + within][2 q + half]
#pragma unroll
        for (int o = 0; o < TILES; ++o)
#pragma unroll
            for (int q = 0; q < kMaxPairs; ++q) {
                const int out = 32 * o + within, in = 2 * q + half;
                const bool inside = out < a.order && in < a.order;
                const int index = a.transpose ? in * a.order + out : out * a.order + in;
                const float held = basis_tile[inside ? index : 0];
                left[o][q] = inside ? held : 0.0f;
            }
        const int row_words = padded(a.width);
        const size_t outer_base = static_cast<size_t>(blockIdx.x) * a.order * a.width;
        for (int first = (threadIdx.x >> 6) * 32; first < a.width; first += (blockDim.x >> 6) * 32) {
            const int p = first + within;
            float right[kMaxPairs];
#pragma unroll
            for (int q = 0; q < kMaxPairs; ++q) {
                const int in = 2 * q + half;
                const bool inside = q < pairs && in < a.order;
                const float held = tile[(inside ? in : 0) * row_words + padded(p)];
                right[q] = inside ? held : 0.0f;
            }
#pragma unroll
            for (int o = 0; o < TILES; ++o) {
                mk_mix16 sums;
#pragma unroll
                for (int r = 0; r < 16; ++r) sums[r] = 0.0f;
#pragma unroll
                for (int q = 0; q < kMaxPairs; ++q)
                    if (q < pairs) sums = __builtin_amdgcn_mfma_f32_32x32x2f32(left[o][q], right[q], sums, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int out = 32 * o + (r >> 2) * 8 + half * 4 + (r & 3);
                    if (out < a.order) {
                        float value = sums[r];
                        if (a.signs_after) value *= a.signs_after[out * a.width + p];
                        mk_store_from_float(a.target, outer_base + static_cast<size_t>(out) * a.width + p, a.target_dtype, value);
                    }
                }
            }
        }
    }
}

template <int E, bool VEC, int TILES = 0>
int launch_fwht_as(const FwhtArgs &a, int threads, size_t lds, hipStream_t stream) {
    static size_t allowed = 48 * 1024;  // raised once per instantiation when a row needs more
    if (lds > allowed) {
        hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(&fwht_kernel<E, VEC, TILES>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (status != hipSuccess)
            return mk_fail(MK_ERR_HIP, "mk_fwht: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(status));
        allowed = 160 * 1024;
    }
    const long long blocks = (a.rows + a.rows_per_block - 1) / a.rows_per_block;
    hipLaunchKernelGGL((fwht_kernel<E, VEC, TILES>), dim3(static_cast<unsigned>(blocks)), dim3(threads), lds, stream, a);
    return MK_OK;
}

// The blocked transform in one launch: a workgroup per outer row.  Returns MK_OK after a
// launch, -1 when the shape does not fit one workgroup (the caller then uses two launches).
template <int E, int TILES>
int launch_blocked(FwhtArgs a, hipStream_t stream) {
    a.threads_per_row = a.width / E;
    a.rows_per_block = a.order;
    const int threads = (a.order * a.threads_per_row + 63) / 64 * 64;
    const size_t lds = (static_cast<size_t>(a.order) * padded(a.width) + static_cast<size_t>(a.order) * a.order) * sizeof(float);
    if (threads > kMaxThreads || lds > 160 * 1024) return -1;
    const auto aligned = [](const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15u) == 0; };
    if (aligned(a.source) && aligned(a.signs_before)) return launch_fwht_as<E, true, TILES>(a, threads, lds, stream);
    return launch_fwht_as<E, false, TILES>(a, threads, lds, stream);
}

template <int E>
int launch_fwht(FwhtArgs a, hipStream_t stream) {
    a.threads_per_row = a.width / E;
    a.rows_per_block = a.threads_per_row >= 256 ? 1 : 256 / a.threads_per_row;
    if (a.rows_per_block > a.rows) a.rows_per_block = static_cast<int>(a.rows);
    const int threads = a.rows_per_block * a.threads_per_row;
    const size_t lds = static_cast<size_t>(a.rows_per_block) * padded(a.width) * sizeof(float);
    if constexpr (E % 4 == 0) {
        const auto aligned = [](const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15u) == 0; };
        if (aligned(a.source) && aligned(a.signs_before)) return launch_fwht_as<E, true>(a, threads, lds, stream);
    }
    return launch_fwht_as<E, false>(a, threads, lds, stream);
}

// ---- Blocked rotation of weight-sized tensors: one pass, transform in registers -------------
//
// A workgroup owns one outer row of `order` blocks of `power` = 32 E values (E = 8 or 16) at a time
// (two workgroups per CU, each taking every 512th row, the next row's values already on their
// way into registers while the current one is mixed).  Half a wavefront holds a block: lane t of the half has elements (32 q + t) 4 + i of it (E / 4 coalesced
// 16-byte loads), so index bits 0-1 and 7+ live in registers and bits 2-6 in the lane number.
// The butterfly stages run in ascending stride as everywhere else: bits 0-1 between registers,
// bits 2-6 between lanes (vector-ALU lane moves; the lane whose bit is set computes
// partner - own, the other own + partner, both as one exactly rounded fma with +-1), the rest
// between registers.  The transformed blocks are written to LDS once (16 bytes per lane, no
// bank conflicts), and after one barrier every wavefront multiplies 32-column slices of them
// by the basis on the fp32 matrix cores, exactly as fwht_kernel<.., TILES> does.  Per element:
// about 20 vector instructions and 8 bytes of LDS traffic.

struct MatrixArgs {
    const float *source;
    float *target;
    const float *basis;
    const float *signs_before, *signs_after;  // [order * power] or null
    long long rows;  // outer rows
    int order, power, transpose;
    float scale;
};

// The value lane `lane ^ (1 << STAGE)` holds, STAGE 0 ... 4 (inside a half wavefront): one DPP
// move where a row permutation exists (lanes ^ 1, ^ 2, ^ 8), one swizzle through the LDS
// crossbar (no memory access, no vector-ALU slot) for lanes ^ 4 and ^ 16.
template <int STAGE>
__device__ __forceinline__ float half_wave_partner(float value) {
    const int bits = __builtin_bit_cast(int, value);
    int moved;
    if constexpr (STAGE == 0) moved = __builtin_amdgcn_mov_dpp(bits, 0xB1, 0xf, 0xf, true);        // quad_perm [1,0,3,2]
    else if constexpr (STAGE == 1) moved = __builtin_amdgcn_mov_dpp(bits, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    else if constexpr (STAGE == 3) moved = __builtin_amdgcn_mov_dpp(bits, 0x128, 0xf, 0xf, true);  // row_ror:8
    else moved = __builtin_amdgcn_ds_swizzle(bits, 0x1F | ((1 << STAGE) << 10));  // bit mode: and 31, or 0, xor 1 << STAGE
    return __builtin_bit_cast(float, moved);
}

template <int E, int STAGE>
__device__ __forceinline__ void lane_stage(float (&v)[E], int t) {
    const float sign = (t >> STAGE) & 1 ? -1.0f : 1.0f;
#pragma unroll
    for (int j = 0; j < E; ++j) v[j] = __builtin_fmaf(v[j], sign, half_wave_partner<STAGE>(v[j]));
}

constexpr int kRotationWaves = 8;   // wavefronts per workgroup: two workgroups share a CU
constexpr int kRotationUnits = 2;   // pairs of blocks per wavefront: up to 32 blocks per outer row

template <int E>
__global__ void __launch_bounds__(64 * kRotationWaves) rotate_matrix_kernel(const MatrixArgs a) {
    extern __shared__ __attribute__((aligned(16))) float tile[];  // [order][power], then the basis
    constexpr int kQuads = E / 4;
    constexpr int kPower = 32 * E;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int half = lane >> 5, t = lane & 31;
    const size_t outer_floats = static_cast<size_t>(a.order) * kPower;

    // In LDS behind the row: the basis as the left operand of the products, mix[out][in] at
    // basis_tile[in * 32 + out], zero outside the basis.
    float *basis_tile = tile + outer_floats;
    for (int i = threadIdx.x; i < 32 * 32; i += blockDim.x) {
        const int in = i >> 5, out = i & 31;
        const bool inside = in < a.order && out < a.order;
        const float held = a.basis[inside ? (a.transpose ? in * a.order + out : out * a.order + in) : 0];
        basis_tile[i] = inside ? held : 0.0f;
    }
    const int pairs = (a.order + 1) >> 1;

    // Wavefront w transforms the pairs of blocks w and w + 8 of every outer row the workgroup
    // takes; their values are requested one row ahead.
    float4 loaded[kRotationUnits][kQuads];
    const int rows = static_cast<int>(a.rows), stride = gridDim.x;  // (rows * order < 2^31: checked by the caller)
    auto request = [&](int u, int row) __attribute__((always_inline)) {
        const int block = 2 * (wave + kRotationWaves * u) + half;
        if (row >= rows || 2 * (wave + kRotationWaves * u) >= a.order) return;  // uniform
        const float4 *source = reinterpret_cast<const float4 *>(a.source + static_cast<size_t>(row) * outer_floats);
        const uint32_t first = static_cast<uint32_t>(block < a.order ? block : 0) * (kPower / 4) + t;
#pragma unroll
        for (int q = 0; q < kQuads; ++q) loaded[u][q] = source[q * 32 + first];
    };
#pragma unroll
    for (int u = 0; u < kRotationUnits; ++u) request(u, blockIdx.x);
    for (int row = blockIdx.x; row < rows; row += stride) {
#pragma unroll
        for (int u = 0; u < kRotationUnits; ++u) {
            const int block = 2 * (wave + kRotationWaves * u) + half;
            if (2 * (wave + kRotationWaves * u) >= a.order) continue;  // uniform
            const bool present = block < a.order;
            const int offset = (present ? block : 0) * kPower;
            // (the signs are requested before the next row's values: loads complete in order, and
            // the butterflies must not wait for that row)
            float4 sign[kQuads];
            if (a.signs_before) {
                const float4 *signs = reinterpret_cast<const float4 *>(a.signs_before + offset);
#pragma unroll
                for (int q = 0; q < kQuads; ++q) sign[q] = signs[q * 32 + t];
            }
            float v[E];
#pragma unroll
            for (int q = 0; q < kQuads; ++q) {
                v[4 * q] = loaded[u][q].x; v[4 * q + 1] = loaded[u][q].y;
                v[4 * q + 2] = loaded[u][q].z; v[4 * q + 3] = loaded[u][q].w;
            }
            request(u, row + stride);  // the same blocks of the workgroup's next row, a whole turn ahead
            if (a.signs_before) {
#pragma unroll
                for (int q = 0; q < kQuads; ++q) {
                    v[4 * q] *= sign[q].x; v[4 * q + 1] *= sign[q].y; v[4 * q + 2] *= sign[q].z; v[4 * q + 3] *= sign[q].w;
                }
            }
            // index bits 0 and 1: inside each group of four
#pragma unroll
            for (int bit = 0; bit < 2; ++bit)
#pragma unroll
                for (int j = 0; j < E; ++j) {
                    if ((j >> bit) & 1) continue;
                    const float first = v[j], second = v[j | (1 << bit)];
                    v[j] = first + second;
                    v[j | (1 << bit)] = first - second;
                }
            // bits 2 ... 6: between the lanes of the half wavefront
            lane_stage<E, 0>(v, t);
            lane_stage<E, 1>(v, t);
            lane_stage<E, 2>(v, t);
            lane_stage<E, 3>(v, t);
            lane_stage<E, 4>(v, t);
            // bits 7 and up: between the groups of four
#pragma unroll
            for (int bit = 2; (1 << bit) < E; ++bit)
#pragma unroll
                for (int j = 0; j < E; ++j) {
                    if ((j >> bit) & 1) continue;
                    const float first = v[j], second = v[j | (1 << bit)];
                    v[j] = first + second;
                    v[j | (1 << bit)] = first - second;
                }
            if (present) {
                float4 *rows = reinterpret_cast<float4 *>(tile + offset);
#pragma unroll
                for (int q = 0; q < kQuads; ++q)
                    rows[q * 32 + t] = make_float4(v[4 * q] * a.scale, v[4 * q + 1] * a.scale, v[4 * q + 2] * a.scale,
                                                   v[4 * q + 3] * a.scale);
            }
        }
        __syncthreads();

        // target[f', p] = sum_f mix[f', f] * block f [p] over ascending f from zero (f in pairs on
        // the matrix cores); lanes 0..31 read block f, lanes 32..63 block f + 1, at 32 adjacent p.
        float *row_target = a.target + static_cast<size_t>(row) * outer_floats;
        const float *mine = tile + half * kPower + t;          // + 2 q kPower + first
        const float *basis_mine = basis_tile + half * 32 + t;  // + 64 q
        for (int first = wave * 32; first < kPower; first += kRotationWaves * 32) {
            // (byte offsets in 32 bits, so that a store takes a scalar base and one offset register)
            const uint32_t store_bytes = static_cast<uint32_t>(half * 4 * kPower + first + t) * 4u;
            mk_mix16 sums;
#pragma unroll
            for (int r = 0; r < 16; ++r) sums[r] = 0.0f;
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                if (q < pairs) {  // uniform
                    // (an odd order's last pair reads one block beyond the row: the basis tile, finite
                    // values that meet the zeros of the basis' padding)
                    const float right = mine[2 * q * kPower + first];
                    sums = __builtin_amdgcn_mfma_f32_32x32x2f32(basis_mine[64 * q], right, sums, 0, 0, 0);
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int out_uniform = (r >> 2) * 8 + (r & 3);   // + 4 for the upper half of the lanes
                const bool both = out_uniform + 4 < a.order, lower = out_uniform < a.order;  // uniform
                if (both || (lower && half == 0)) {
                    float value = sums[r];
                    if (a.signs_after)
                        value *= *reinterpret_cast<const float *>(
                            reinterpret_cast<const char *>(a.signs_after + out_uniform * kPower) + store_bytes);
                    *reinterpret_cast<float *>(reinterpret_cast<char *>(row_target + out_uniform * kPower) + store_bytes) = value;
                }
            }
        }
        __syncthreads();  // the next row's blocks go into the same LDS
    }
}

// Launches rotate_matrix_kernel when the shape fits it: fp32 in and out, 16-byte aligned,
// power = 32 E with E in {8, 16} (blocks of 256 or 512 values), at most 32 blocks that fit
// 76 KB of LDS together (two workgroups per CU).
// Returns -1 when it does not apply.
int launch_rotate_matrix(const FwhtArgs &f, long long outer_rows, hipStream_t stream) {
    const auto aligned = [](const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15u) == 0; };
    const int elements = f.width / 32;
    const size_t lds = (static_cast<size_t>(f.order) * f.width + 32 * 32) * sizeof(float);
    if (f.source_dtype != MK_F32 || f.target_dtype != MK_F32 || f.order > 32 ||
        (elements != 8 && elements != 16) || lds > 80 * 1024 || !aligned(f.source) ||
        !aligned(f.target) || !aligned(f.signs_before))
        return -1;
    MatrixArgs a{static_cast<const float *>(f.source), static_cast<float *>(f.target), f.basis, f.signs_before,
                 f.signs_after, outer_rows, f.order, f.width, f.transpose, f.scale};
    // Two workgroups of eight wavefronts per CU (registers and LDS allow no more), so that one's
    // matrix-core phase overlaps the other's butterflies; each takes every 512th outer row.
    const dim3 grid(static_cast<unsigned>(outer_rows < 512 ? outer_rows : 512)), block(64 * kRotationWaves);
    static std::atomic<bool> raised{false};
    if (lds > 48 * 1024 && !raised.load()) {
        for (const void *kernel : {reinterpret_cast<const void *>(&rotate_matrix_kernel<8>),
                                   reinterpret_cast<const void *>(&rotate_matrix_kernel<16>)}) {
            const hipError_t status = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
            if (status != hipSuccess)
                return mk_fail(MK_ERR_HIP, "mk_rotate_blocks: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(status));
        }
        raised.store(true);
    }
    if (elements == 8) hipLaunchKernelGGL(rotate_matrix_kernel<8>, grid, block, lds, stream, a);
    else hipLaunchKernelGGL(rotate_matrix_kernel<16>, grid, block, lds, stream, a);
    return MK_OK;
}

// ---- Plain transform of weight-sized fp32 tensors: one wavefront per row, registers only -----
//
// A row of 64 E values (E = 4 ... 64: 256 to 4096 values) lives in the registers of one
// wavefront, lane t holding elements (64 q + t) 4 + i: index bits 0-1 and 8+ in registers, bits
// 2-7 in the lane number.  Same stages in the same order as fwht_kernel, same sums, no LDS
// memory and no barrier; lane exchanges are DPP moves (lanes ^ 1, ^ 2, ^ 8), swizzles through
// the LDS crossbar (^ 4, ^ 16) and a crossbar permute (^ 32).

// The value lane `lane ^ 32` holds.
__device__ __forceinline__ float other_half_partner(float value, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, value)));
}

template <int E>
__global__ void __launch_bounds__(256) fwht_rows_kernel(const FwhtArgs a) {
    constexpr int kQuads = E / 4;
    const int lane = threadIdx.x & 63;
    const long long row = static_cast<long long>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= a.rows) return;  // whole wavefronts leave; nothing below synchronises the workgroup
    const size_t row_base = static_cast<size_t>(row) * a.width;
    const int sign_base = a.sign_period ? static_cast<int>(row_base % static_cast<size_t>(a.sign_period)) : 0;
    const float4 *source = reinterpret_cast<const float4 *>(static_cast<const float *>(a.source) + row_base);
    float4 loaded[kQuads];
#pragma unroll
    for (int q = 0; q < kQuads; ++q) loaded[q] = source[q * 64 + lane];
    float v[E];
#pragma unroll
    for (int q = 0; q < kQuads; ++q) {
        v[4 * q] = loaded[q].x; v[4 * q + 1] = loaded[q].y; v[4 * q + 2] = loaded[q].z; v[4 * q + 3] = loaded[q].w;
    }
    if (a.signs_before) {
        const float4 *signs = reinterpret_cast<const float4 *>(a.signs_before + sign_base);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) {
            const float4 sign = signs[q * 64 + lane];
            v[4 * q] *= sign.x; v[4 * q + 1] *= sign.y; v[4 * q + 2] *= sign.z; v[4 * q + 3] *= sign.w;
        }
    }
#pragma unroll
    for (int bit = 0; bit < 2; ++bit)
#pragma unroll
        for (int j = 0; j < E; ++j) {
            if ((j >> bit) & 1) continue;
            const float first = v[j], second = v[j | (1 << bit)];
            v[j] = first + second;
            v[j | (1 << bit)] = first - second;
        }
    lane_stage<E, 0>(v, lane);
    lane_stage<E, 1>(v, lane);
    lane_stage<E, 2>(v, lane);
    lane_stage<E, 3>(v, lane);
    lane_stage<E, 4>(v, lane);
    {
        const float sign = lane & 32 ? -1.0f : 1.0f;
#pragma unroll
        for (int j = 0; j < E; ++j) v[j] = __builtin_fmaf(v[j], sign, other_half_partner(v[j], lane));
    }
#pragma unroll
    for (int bit = 2; (1 << bit) < E; ++bit)
#pragma unroll
        for (int j = 0; j < E; ++j) {
            if ((j >> bit) & 1) continue;
            const float first = v[j], second = v[j | (1 << bit)];
            v[j] = first + second;
            v[j | (1 << bit)] = first - second;
        }
    float4 *target = reinterpret_cast<float4 *>(static_cast<float *>(a.target) + row_base);
    const float4 *signs_after = reinterpret_cast<const float4 *>(a.signs_after ? a.signs_after + sign_base : nullptr);
#pragma unroll
    for (int q = 0; q < kQuads; ++q) {
        float4 out = make_float4(v[4 * q] * a.scale, v[4 * q + 1] * a.scale, v[4 * q + 2] * a.scale, v[4 * q + 3] * a.scale);
        if (signs_after) {
            const float4 sign = signs_after[q * 64 + lane];
            out.x *= sign.x; out.y *= sign.y; out.z *= sign.z; out.w *= sign.w;
        }
        target[q * 64 + lane] = out;
    }
}

// Launches fwht_rows_kernel when it applies (fp32 in and out, rows of 256 ... 4096 values,
// 16-byte aligned, enough rows to fill the GPU with wavefronts); -1 otherwise.
constexpr long long kRegisterTransformRows = 4096;

int launch_fwht_rows(const FwhtArgs &a, hipStream_t stream) {
    const auto aligned = [](const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15u) == 0; };
    if (a.source_dtype != MK_F32 || a.target_dtype != MK_F32 || a.width < 256 || a.width > 4096 ||
        a.rows < kRegisterTransformRows || !aligned(a.source) || !aligned(a.target) || !aligned(a.signs_before) ||
        !aligned(a.signs_after))
        return -1;
    const dim3 grid(static_cast<unsigned>((a.rows + 3) / 4)), block(256);
    switch (a.width / 64) {
        case 4: hipLaunchKernelGGL(fwht_rows_kernel<4>, grid, block, 0, stream, a); break;
        case 8: hipLaunchKernelGGL(fwht_rows_kernel<8>, grid, block, 0, stream, a); break;
        case 16: hipLaunchKernelGGL(fwht_rows_kernel<16>, grid, block, 0, stream, a); break;
        case 32: hipLaunchKernelGGL(fwht_rows_kernel<32>, grid, block, 0, stream, a); break;
        default: hipLaunchKernelGGL(fwht_rows_kernel<64>, grid, block, 0, stream, a); break;
    }
    return MK_OK;
}

struct MixArgs {
    const float *source;
    float *target;
    const float *basis;  // [order, order] row-major
    const float *signs_after;
    long long rows;
    int order, power, transpose;
};

// target[r, f', p] = sum_f mix[f', f] * source[r, f, p], mix = basis or its transpose;
// the sum runs over ascending f with fused multiply-adds starting from zero.
// One thread owns one (r, p) column of `order` values, kept in a private column of LDS
// (dynamically indexed registers would live in scratch memory); consecutive lanes take
// consecutive p, and the basis entries are wavefront-uniform scalar loads.
constexpr int kMaxOrder = 256;

__global__ void __launch_bounds__(256) basis_mix_kernel(const MixArgs a) {
    extern __shared__ float columns_tile[];  // [order][blockDim.x]
    float *mine = columns_tile + threadIdx.x;
    const long long columns = a.rows * a.power;
    const int row_stride = a.transpose ? 1 : a.order;
    const int column_stride = a.transpose ? a.order : 1;
    for (long long column = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; column < columns;
         column += static_cast<long long>(gridDim.x) * blockDim.x) {
        const long long row = column / a.power;
        const int p = static_cast<int>(column - row * a.power);
        const size_t base = static_cast<size_t>(row) * a.order * a.power + p;
        for (int f = 0; f < a.order; ++f) mine[f * blockDim.x] = a.source[base + static_cast<size_t>(f) * a.power];
        for (int out = 0; out < a.order; ++out) {
            const float *mix_row = a.basis + out * row_stride;
            float sum = 0.0f;
            for (int f = 0; f < a.order; ++f) sum = __builtin_fmaf(mix_row[f * column_stride], mine[f * blockDim.x], sum);
            if (a.signs_after) sum *= a.signs_after[out * a.power + p];
            a.target[base + static_cast<size_t>(out) * a.power] = sum;
        }
    }
}

// The same product on the fp32 matrix cores for bases of up to 96 rows.  One wavefront
// owns 32 adjacent columns p of one row r: the basis (zero-padded to TILES x 32 rows) is
// the left operand, kept in registers; the right operand comes straight from global memory,
// lanes 0..31 reading 32 adjacent p of block f and lanes 32..63 of block f + 1, so no LDS is
// involved.  v_mfma_f32_32x32x2_f32 accumulates over ascending f from zero, which equals
// the fused multiply-add chain of basis_mix_kernel bit for bit.
template <int TILES>
__global__ void __launch_bounds__(256) basis_mix_mfma_kernel(const MixArgs a) {
    constexpr int kMaxPairs = TILES * 16;  // k-pairs of a basis padded to TILES * 32
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5, within = lane & 31;
    const int pairs = (a.order + 1) >> 1;
    // left[t][q]: mix[32 t + within][2 q + half]
    float left[TILES][kMaxPairs];
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int q = 0; q < kMaxPairs; ++q) {
            const int out = 32 * t + within, in = 2 * q + half;
            const bool inside = out < a.order && in < a.order;
            const int index = a.transpose ? in * a.order + out : out * a.order + in;
            left[t][q] = inside ? a.basis[inside ? index : 0] : 0.0f;
        }
    const int tiles_per_row = (a.power + 31) >> 5;
    const long long total = a.rows * tiles_per_row;
    const long long first = static_cast<long long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const long long stride = static_cast<long long>(gridDim.x) * (blockDim.x >> 6);
    for (long long tile = first; tile < total; tile += stride) {
        const long long row = tile / tiles_per_row;
        const int p = static_cast<int>(tile - row * tiles_per_row) * 32 + within;
        const bool column_ok = p < a.power;
        const size_t base = static_cast<size_t>(row) * a.order * a.power + (column_ok ? p : 0);
        float right[kMaxPairs];
#pragma unroll
        for (int q = 0; q < kMaxPairs; ++q) {
            const int in = 2 * q + half;
            const bool inside = q < pairs && in < a.order && column_ok;
            const float loaded = a.source[base + static_cast<size_t>(inside ? in : 0) * a.power];
            right[q] = inside ? loaded : 0.0f;
        }
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            mk_mix16 sums;
#pragma unroll
            for (int r = 0; r < 16; ++r) sums[r] = 0.0f;
#pragma unroll
            for (int q = 0; q < kMaxPairs; ++q)
                if (q < pairs) sums = __builtin_amdgcn_mfma_f32_32x32x2f32(left[t][q], right[q], sums, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int out = 32 * t + (r >> 2) * 8 + half * 4 + (r & 3);
                if (out < a.order && column_ok) {
                    float value = sums[r];
                    if (a.signs_after) value *= a.signs_after[out * a.power + p];
                    a.target[base + static_cast<size_t>(out) * a.power] = value;
                }
            }
        }
    }
}

template <int TILES>
void launch_mix_mfma(const MixArgs &a, hipStream_t stream) {
    const long long tiles = a.rows * ((a.power + 31) / 32);
    long long blocks = (tiles + 3) / 4;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL((basis_mix_mfma_kernel<TILES>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a);
}

}  // namespace

extern "C" int mk_fwht(const void *source, int source_dtype, void *target, int target_dtype, long long rows,
                       int width, const float *signs_before, const float *signs_after, int sign_period,
                       float scale, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(rows >= 0, MK_ERR_INVALID, "mk_fwht: negative row count");
    MK_REQUIRE(width >= 1 && (width & (width - 1)) == 0, MK_ERR_INVALID,
               "mk_fwht: hadamard currently requires a power-of-two final dimension (got %d)", width);
    MK_REQUIRE(width <= 32768, MK_ERR_UNSUPPORTED, "mk_fwht: rows longer than 32768 values are not supported");
    if (rows == 0) return MK_OK;
    MK_REQUIRE(source && target, MK_ERR_INVALID, "mk_fwht: null tensor pointer");
    MK_REQUIRE(mk_dtype_valid(source_dtype) && mk_dtype_valid(target_dtype), MK_ERR_INVALID,
               "mk_fwht: unknown dtype code");
    MK_REQUIRE(!(signs_before || signs_after) || (sign_period >= width && sign_period % width == 0), MK_ERR_INVALID,
               "mk_fwht: the sign period must be a multiple of the row width");
    MK_REQUIRE((rows + 255) / 256 < (1ll << 31), MK_ERR_INVALID, "mk_fwht: too many rows");
    FwhtArgs a{};
    a.source = source; a.target = target; a.signs_before = signs_before; a.signs_after = signs_after;
    a.rows = rows; a.width = width; a.source_dtype = source_dtype; a.target_dtype = target_dtype;
    a.sign_period = (signs_before || signs_after) ? sign_period : 0; a.scale = scale;
    a.log_width = 0;
    while ((1 << a.log_width) < width) ++a.log_width;
    int status = launch_fwht_rows(a, stream);
    if (status >= 0) {
        MK_LAUNCH_CHECK("mk_fwht");
        return MK_OK;
    }
    if (width >= 32768) status = launch_fwht<32>(a, stream);
    else if (width >= 16) status = launch_fwht<16>(a, stream);
    else if (width == 8) status = launch_fwht<8>(a, stream);
    else if (width == 4) status = launch_fwht<4>(a, stream);
    else if (width == 2) status = launch_fwht<2>(a, stream);
    else status = launch_fwht<1>(a, stream);
    if (status) return status;
    MK_LAUNCH_CHECK("mk_fwht");
    return MK_OK;
}

extern "C" int mk_rotate_blocks(const void *source, int source_dtype, void *target, int target_dtype, long long rows,
                                int order, int power, const float *basis, int transpose, const float *signs_before,
                                const float *signs_after, float scale, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(rows >= 0 && order >= 1, MK_ERR_INVALID, "mk_rotate_blocks: sizes must be positive");
    MK_REQUIRE(power >= 1 && (power & (power - 1)) == 0, MK_ERR_INVALID,
               "mk_rotate_blocks: the block width must be a power of two (got %d)", power);
    MK_REQUIRE(order <= 96 && power >= 32 && power <= 32768, MK_ERR_UNSUPPORTED,
               "mk_rotate_blocks: %d blocks of %d values do not fit one workgroup", order, power);
    if (rows == 0) return MK_OK;
    MK_REQUIRE(source && target && basis, MK_ERR_INVALID, "mk_rotate_blocks: null tensor pointer");
    MK_REQUIRE(source != target, MK_ERR_INVALID, "mk_rotate_blocks: source and target must not alias");
    MK_REQUIRE(mk_dtype_valid(source_dtype) && mk_dtype_valid(target_dtype), MK_ERR_INVALID,
               "mk_rotate_blocks: unknown dtype code");
    MK_REQUIRE(rows < (1ll << 31) / order, MK_ERR_INVALID, "mk_rotate_blocks: too many rows");
    FwhtArgs a{};
    a.source = source; a.target = target; a.signs_before = signs_before; a.signs_after = signs_after;
    a.rows = rows * order; a.width = power; a.source_dtype = source_dtype; a.target_dtype = target_dtype;
    a.sign_period = (signs_before || signs_after) ? order * power : 0; a.scale = scale;
    a.basis = basis; a.order = order; a.transpose = transpose;
    a.log_width = 0;
    while ((1 << a.log_width) < power) ++a.log_width;
    int status = -1;
    // Weight-sized tensors (more outer rows than the GPU has workgroup slots) take the lean one-pass kernel.
    if (rows > kLeanRotationRows) status = launch_rotate_matrix(a, rows, stream);
    if (status >= 0) {
        if (status) return status;
        MK_LAUNCH_CHECK("mk_rotate_blocks");
        return MK_OK;
    }
    if (order * (power / 16) <= kMaxThreads) {
        status = order <= 32 ? launch_blocked<16, 1>(a, stream)
                             : order <= 64 ? launch_blocked<16, 2>(a, stream) : launch_blocked<16, 3>(a, stream);
    } else if (order * (power / 32) <= kMaxThreads) {
        status = order <= 32 ? launch_blocked<32, 1>(a, stream)
                             : order <= 64 ? launch_blocked<32, 2>(a, stream) : launch_blocked<32, 3>(a, stream);
    }
    if (status < 0)
        return mk_fail(MK_ERR_UNSUPPORTED, "mk_rotate_blocks: %d blocks of %d values do not fit one workgroup", order, power);
    if (status) return status;
    MK_LAUNCH_CHECK("mk_rotate_blocks");
    return MK_OK;
}

extern "C" int mk_basis_mix(const float *source, float *target, const float *basis, long long rows, int order,
                            int power, int transpose, const float *signs_after, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(rows >= 0 && order >= 1 && power >= 1, MK_ERR_INVALID, "mk_basis_mix: sizes must be positive");
    MK_REQUIRE(order <= kMaxOrder, MK_ERR_UNSUPPORTED, "mk_basis_mix: basis order %d exceeds %d", order, kMaxOrder);
    if (rows == 0) return MK_OK;
    MK_REQUIRE(source && target && basis, MK_ERR_INVALID, "mk_basis_mix: null tensor pointer");
    MK_REQUIRE(source != target, MK_ERR_INVALID, "mk_basis_mix: source and target must not alias");
    MixArgs a{source, target, basis, signs_after, rows, order, power, transpose};
    if (order <= 32) {
        launch_mix_mfma<1>(a, stream);
    } else if (order <= 64) {
        launch_mix_mfma<2>(a, stream);
    } else if (order <= 96) {
        launch_mix_mfma<3>(a, stream);
    } else {
        // One LDS column of `order` floats per thread: fewer threads for larger bases (64 KB).
        const int threads = order <= 128 ? 128 : 64;
        long long blocks = (rows * power + threads - 1) / threads;
        if (blocks > 256 * 64) blocks = 256 * 64;
        hipLaunchKernelGGL(basis_mix_kernel, dim3(static_cast<unsigned>(blocks)), dim3(threads),
                           static_cast<size_t>(order) * threads * sizeof(float), stream, a);
    }
    MK_LAUNCH_CHECK("mk_basis_mix");
    return MK_OK;
}
