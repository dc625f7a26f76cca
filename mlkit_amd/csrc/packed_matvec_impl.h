// Packed scalar-codec matrix-vector product for 1..8 input rows on gfx950: kernel templates.
//
// y[m, n] = sum_k dequant(code[n, k]) * x[m, k] (+ bias[n]),  fp32 accumulate.
//
// Streaming kernel (HBM bound, no matrix cores).  A lane owns up to C chunks of 32
// consecutive codes of a row (BITS dwords each, one coalesced 4*BITS-byte load); the
// matching 32 activations of every sample stay in registers for the life of the
// workgroup, so the only per-row traffic is the code stream itself plus one scale per
// chunk read from LDS, where the workgroup's scale tile is staged once as fp32.
// A row's lanes form a segment of the workgroup: a power of two up to 64 lanes, or a
// whole number of wavefronts.  Partial sums meet by a segment reduction inside the
// wavefront and, when a row spans several wavefronts, by a fixed-order sum through LDS,
// so results do not depend on scheduling.
//
// Rows of the weight whose width or scale groups are not multiples of 32 codes take
// the word-at-a-time kernel at the end of this file.
//
// Replaces the reference's Triton kernel `packed_matrix_vector`
// (kernels/packed_linear.py:107-173 in /root/reference/src/mlkit).

#pragma once
#include "mk_common.h"

namespace mk_matvec {

constexpr int kChunkCodes = 32;
constexpr int kMaxTableEntries = 256;

struct MatvecArgs {
    const void *x;
    const uint8_t *packed;
    const void *scales;
    const void *zeros;
    const float *values;
    const void *bias;
    void *y;
    int samples;
    int rows;
    int width;
    int group;
    int groups;
    int n_values;
    int scale_dtype;
    int bias_dtype;
    int seg_lanes;        // lanes (incl. idle ones) that share one row
    int rows_parallel;    // rows in flight per workgroup pass
    int rows_per_thread;  // passes per workgroup
    int chunks_per_row;   // width / 32
    float grid_min;
    float grid_step;
};

// ---------------------------------------------------------------------------------
// Activation registers.  XT: MK_F32 keeps 32 floats per chunk; MK_F16 / MK_BF16 keep
// 16 packed pairs.  `kPairs48` stores fp16 pairs as (x[i], x[i+4]) inside every group
// of eight codes, the order in which the 4-bit extraction below produces its pairs.
// ---------------------------------------------------------------------------------
template <int XT>
struct XChunk {
    uint32_t r[XT == MK_F32 ? 32 : 16];
};

template <int XT>
__device__ __forceinline__ float x_element(const XChunk<XT> &x, int k) {
    if constexpr (XT == MK_F32) {
        return __uint_as_float(x.r[k]);
    } else if constexpr (XT == MK_F16) {
        const mk_h2 pair = __builtin_bit_cast(mk_h2, x.r[k >> 1]);
        return static_cast<float>(pair[k & 1]);
    } else {
        const uint32_t word = x.r[k >> 1];
        return __uint_as_float((k & 1) ? (word & 0xffff0000u) : (word << 16));
    }
}

template <int XT>
__device__ __forceinline__ void load_x_chunk(XChunk<XT> &x, const void *base, size_t element,
                                             bool active, float &sum) {
    constexpr int kWords = XT == MK_F32 ? 32 : 16;
    if (active) {
        const mk_u32x4 *src = reinterpret_cast<const mk_u32x4 *>(
            static_cast<const uint8_t *>(base) + element * (XT == MK_F32 ? 4 : 2));
#pragma unroll
        for (int i = 0; i < kWords / 4; ++i) {
            const mk_u32x4 v = src[i];
            x.r[4 * i + 0] = v.x;
            x.r[4 * i + 1] = v.y;
            x.r[4 * i + 2] = v.z;
            x.r[4 * i + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < kWords; ++i) x.r[i] = 0u;
    }
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < 32; ++k) total += x_element<XT>(x, k);
    sum = total;
}

// (x0,x1)(x2,x3)(x4,x5)(x6,x7) -> (x0,x4)(x1,x5)(x2,x6)(x3,x7) for every eight codes.
__device__ __forceinline__ void pair_for_nibbles(XChunk<MK_F16> &x) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t p0 = x.r[4 * g + 0], p1 = x.r[4 * g + 1];
        const uint32_t p2 = x.r[4 * g + 2], p3 = x.r[4 * g + 3];
        x.r[4 * g + 0] = __builtin_amdgcn_perm(p2, p0, 0x05040100u);
        x.r[4 * g + 1] = __builtin_amdgcn_perm(p2, p0, 0x07060302u);
        x.r[4 * g + 2] = __builtin_amdgcn_perm(p3, p1, 0x05040100u);
        x.r[4 * g + 3] = __builtin_amdgcn_perm(p3, p1, 0x07060302u);
    }
}

// ---------------------------------------------------------------------------------
// Code chunks: BITS dwords hold 32 codes.
// ---------------------------------------------------------------------------------
template <int BITS>
struct CodeChunk {
    uint32_t w[BITS];
};

template <int BITS>
__device__ __forceinline__ void load_codes(CodeChunk<BITS> &c, const uint8_t *address) {
    // `address` is 4-byte aligned; wide loads need no more than that on gfx9.
    typedef uint32_t u1 __attribute__((aligned(4)));
    typedef mk_u32x2 u2 __attribute__((aligned(4)));
    typedef mk_u32x3 u3 __attribute__((aligned(4)));
    typedef mk_u32x4 u4 __attribute__((aligned(4)));
    if constexpr (BITS == 1) {
        c.w[0] = __builtin_nontemporal_load(reinterpret_cast<const u1 *>(address));
    } else if constexpr (BITS == 2) {
        const mk_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u2 *>(address));
        c.w[0] = v.x; c.w[1] = v.y;
    } else if constexpr (BITS == 3) {
        const mk_u32x3 v = __builtin_nontemporal_load(reinterpret_cast<const u3 *>(address));
        c.w[0] = v.x; c.w[1] = v.y; c.w[2] = v.z;
    } else {
        const mk_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(address));
        c.w[0] = v.x; c.w[1] = v.y; c.w[2] = v.z; c.w[3] = v.w;
        if constexpr (BITS == 5) {
            c.w[4] = __builtin_nontemporal_load(reinterpret_cast<const u1 *>(address + 16));
        } else if constexpr (BITS == 6) {
            const mk_u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u2 *>(address + 16));
            c.w[4] = t.x; c.w[5] = t.y;
        } else if constexpr (BITS == 7) {
            const mk_u32x3 t = __builtin_nontemporal_load(reinterpret_cast<const u3 *>(address + 16));
            c.w[4] = t.x; c.w[5] = t.y; c.w[6] = t.z;
        } else if constexpr (BITS == 8) {
            const mk_u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(address + 16));
            c.w[4] = t.x; c.w[5] = t.y; c.w[6] = t.z; c.w[7] = t.w;
        }
    }
}

// Code k (0..31) of a chunk; k is a compile-time constant after unrolling, so this is
// one bit-field extract, or a funnel shift and a mask when the code crosses a dword.
template <int BITS>
__device__ __forceinline__ uint32_t code_at(const CodeChunk<BITS> &c, int k) {
    const int bit = k * BITS;
    const int word = bit >> 5, shift = bit & 31;
    constexpr uint32_t mask = (1u << BITS) - 1u;
    if (shift + BITS <= 32) return (c.w[word] >> shift) & mask;
    return __builtin_amdgcn_alignbit(c.w[(word + 1) % BITS], c.w[word], shift) & mask;
}

// sum_k T[code_k] * x_k for one chunk and MT samples; T = identity (uniform grids,
// the affine map is applied once per chunk by the caller) or the LDS table.
template <int BITS, int XT, int MT, bool UNIFORM>
__device__ __forceinline__ void chunk_dot(const CodeChunk<BITS> &codes, const XChunk<XT> (&x)[MT],
                                          const float *table, float (&dot)[MT]) {
#pragma unroll
    for (int m = 0; m < MT; ++m) dot[m] = 0.0f;
    if constexpr (BITS == 4 && XT == MK_F16 && UNIFORM) {
        // Two codes at a time: a nibble OR-ed into the mantissa of fp16 1024.0 is
        // 1024 + c (or 1024 + 16 c one nibble up), which one packed op turns into c
        // exactly; v_dot2_f32_f16 then accumulates both products in fp32.
        const mk_h2 bias_low = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
        const mk_h2 sixteenth = {static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
        const mk_h2 bias_high = {static_cast<_Float16>(-64.0f), static_cast<_Float16>(-64.0f)};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = codes.w[i];
            const uint32_t w8 = w >> 8;
            const mk_h2 t0 = __builtin_bit_cast(mk_h2, (w & 0x000f000fu) | 0x64006400u);
            const mk_h2 t1 = __builtin_bit_cast(mk_h2, (w & 0x00f000f0u) | 0x64006400u);
            const mk_h2 t2 = __builtin_bit_cast(mk_h2, (w8 & 0x000f000fu) | 0x64006400u);
            const mk_h2 t3 = __builtin_bit_cast(mk_h2, (w8 & 0x00f000f0u) | 0x64006400u);
            const mk_h2 h0 = t0 - bias_low;
            const mk_h2 h1 = t1 * sixteenth + bias_high;
            const mk_h2 h2 = t2 - bias_low;
            const mk_h2 h3 = t3 * sixteenth + bias_high;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float d = dot[m];
                d = __builtin_amdgcn_fdot2(h0, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 0]), d, false);
                d = __builtin_amdgcn_fdot2(h1, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 1]), d, false);
                d = __builtin_amdgcn_fdot2(h2, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 2]), d, false);
                d = __builtin_amdgcn_fdot2(h3, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 3]), d, false);
                dot[m] = d;
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const uint32_t code = code_at<BITS>(codes, k);
            float value;
            if constexpr (UNIFORM) {
                value = static_cast<float>(code);
            } else {
                value = table[code];
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) dot[m] = __builtin_fmaf(value, x_element<XT>(x[m], k), dot[m]);
        }
    }
}

template <int BITS, int C>
constexpr int rows_in_flight() {
    int u = 32 / (C * BITS);
    return u < 1 ? 1 : (u > 8 ? 8 : u);
}

template <int BITS, int XT, int MT, int C, bool UNIFORM>
struct RowBatch {
    static constexpr int U = rows_in_flight<BITS, C>();
    CodeChunk<BITS> codes[U][C];

    // Issues the code loads of rows `pass .. pass+U-1` of this thread.
    __device__ __forceinline__ void load(const MatvecArgs &a, int pass, int row_base, int row_phase,
                                         int lane_in_row, const bool (&chunk_active)[C]) {
        const size_t row_bytes = static_cast<size_t>(a.chunks_per_row) * (4 * BITS);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int row = row_base + (pass + u) * a.rows_parallel + row_phase;
            row = row < a.rows ? row : a.rows - 1;
            const uint8_t *row_ptr = a.packed + static_cast<size_t>(row) * row_bytes;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if (chunk_active[c]) {
                    const int chunk = lane_in_row + c * a.seg_lanes;
                    load_codes<BITS>(codes[u][c], row_ptr + static_cast<size_t>(chunk) * (4 * BITS));
                } else {
#pragma unroll
                    for (int i = 0; i < BITS; ++i) codes[u][c].w[i] = 0u;
                }
            }
        }
    }
};

template <int BITS, int XT, int MT, int C, bool UNIFORM>
__global__ void packed_matvec_kernel(const MatvecArgs a) {
    extern __shared__ float lds[];
    using Batch = RowBatch<BITS, XT, MT, C, UNIFORM>;
    constexpr int U = Batch::U;
    constexpr bool kNibblePairs = (BITS == 4 && XT == MK_F16 && UNIFORM);

    const int tid = threadIdx.x;
    const int threads = blockDim.x;
    const int lane_in_row = tid % a.seg_lanes;
    const int row_phase = tid / a.seg_lanes;
    const int tile_rows = a.rows_parallel * a.rows_per_thread;
    const int row_base = blockIdx.x * tile_rows;
    const int sample_base = blockIdx.y * MT;
    const bool has_zero = a.zeros != nullptr;
    const int waves_per_row = a.seg_lanes > 64 ? a.seg_lanes / 64 : 1;

    bool chunk_active[C];
    int group_of[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int chunk = lane_in_row + c * a.seg_lanes;
        chunk_active[c] = chunk < a.chunks_per_row;
        group_of[c] = chunk_active[c] ? (chunk * kChunkCodes) / a.group : 0;
    }

    // The code stream depends on nothing: its first loads go out before anything else.
    Batch even, odd;
    even.load(a, 0, row_base, row_phase, lane_in_row, chunk_active);

    // LDS: [value table][scale tile][zero tile][cross-wave partial sums]
    float *table = lds;
    float *scale_tile = table + (UNIFORM ? 0 : kMaxTableEntries);
    float *zero_tile = scale_tile + tile_rows * a.groups;
    float *partials = zero_tile + (has_zero ? tile_rows * a.groups : 0);

    if constexpr (!UNIFORM) {
        for (int i = tid; i < kMaxTableEntries; i += threads)
            table[i] = i < a.n_values ? a.values[i] : 0.0f;
    }
    {
        const size_t first = static_cast<size_t>(row_base) * a.groups;
        const size_t last = static_cast<size_t>(a.rows) * a.groups - 1;
        const int count = tile_rows * a.groups;
        for (int i = tid; i < count; i += threads) {
            size_t index = first + i;
            index = index > last ? last : index;
            scale_tile[i] = mk_load_as_float(a.scales, index, a.scale_dtype);
            if (has_zero) zero_tile[i] = mk_load_as_float(a.zeros, index, a.scale_dtype);
        }
    }

    // Activations of this lane's chunks, resident for the whole workgroup.
    XChunk<XT> x[C][MT];
    float x_sum[C][MT];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int chunk = lane_in_row + c * a.seg_lanes;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int sample = sample_base + m;
            const bool active = chunk_active[c] && sample < a.samples;
            load_x_chunk<XT>(x[c][m], a.x,
                             static_cast<size_t>(sample) * a.width + static_cast<size_t>(chunk) * kChunkCodes,
                             active, x_sum[c][m]);
            if constexpr (kNibblePairs) pair_for_nibbles(x[c][m]);
        }
    }
    __syncthreads();

    auto consume = [&](const Batch &batch, int pass) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int local_row = (pass + u) * a.rows_parallel + row_phase;
            float acc[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[m] = 0.0f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if (chunk_active[c]) {
                    float dot[MT];
                    chunk_dot<BITS, XT, MT, UNIFORM>(batch.codes[u][c], x[c], table, dot);
                    const int slot = local_row * a.groups + group_of[c];
                    const float scale = scale_tile[slot];
                    const float zero = has_zero ? zero_tile[slot] : 0.0f;
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        float value = dot[m];
                        if constexpr (UNIFORM)
                            value = __builtin_fmaf(a.grid_step, value, a.grid_min * x_sum[c][m]);
                        acc[m] = __builtin_fmaf(scale, value, acc[m]);
                        acc[m] = __builtin_fmaf(zero, x_sum[c][m], acc[m]);
                    }
                }
            }
            // Meet the lanes of this row inside the wavefront.
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float total = acc[m];
                if (a.seg_lanes >= 64) total = mk_segment_sum<64>(total);
                else if (a.seg_lanes == 32) total = mk_segment_sum<32>(total);
                else if (a.seg_lanes == 16) total = mk_segment_sum<16>(total);
                else if (a.seg_lanes == 8) total = mk_segment_sum<8>(total);
                else if (a.seg_lanes == 4) total = mk_segment_sum<4>(total);
                else if (a.seg_lanes == 2) total = mk_segment_sum<2>(total);
                acc[m] = total;
            }
            const int row = row_base + local_row;
            if (waves_per_row == 1) {
                if (lane_in_row == 0 && row < a.rows) {
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        const int sample = sample_base + m;
                        if (sample < a.samples) {
                            float result = acc[m];
                            if (a.bias) result += mk_load_as_float(a.bias, row, a.bias_dtype);
                            mk_store_from_float(a.y, static_cast<size_t>(sample) * a.rows + row, XT, result);
                        }
                    }
                }
            } else if ((lane_in_row & 63) == 0) {
                const int wave_in_row = lane_in_row >> 6;
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    partials[(local_row * MT + m) * waves_per_row + wave_in_row] = acc[m];
            }
        }
    };

    // Two register batches alternate: the next rows are in flight while these are summed.
    for (int pass = 0; pass < a.rows_per_thread; pass += 2 * U) {
        const bool more = pass + U < a.rows_per_thread;
        if (more) odd.load(a, pass + U, row_base, row_phase, lane_in_row, chunk_active);
        consume(even, pass);
        if (more) {
            if (pass + 2 * U < a.rows_per_thread)
                even.load(a, pass + 2 * U, row_base, row_phase, lane_in_row, chunk_active);
            consume(odd, pass + U);
        }
    }

    if (waves_per_row > 1) {
        __syncthreads();
        for (int i = tid; i < tile_rows * MT; i += threads) {
            const int local = i / MT, m = i % MT;
            const int row = row_base + local, sample = sample_base + m;
            if (row < a.rows && sample < a.samples) {
                float result = 0.0f;
                for (int w = 0; w < waves_per_row; ++w) result += partials[i * waves_per_row + w];
                if (a.bias) result += mk_load_as_float(a.bias, row, a.bias_dtype);
                mk_store_from_float(a.y, static_cast<size_t>(sample) * a.rows + row, XT, result);
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// Launch of one instantiation chosen by the host-side plan.
// ---------------------------------------------------------------------------------
struct Plan {
    int sample_tile;  // MT
    int chunks;       // C
    int seg_lanes;
    int rows_parallel;
    int rows_per_thread;
    int threads;
    int grid_x;
    size_t lds_bytes;
};

template <int BITS, int XT, int MT, int C, bool UNIFORM>
void launch_chunked(const MatvecArgs &a, const Plan &p, hipStream_t stream) {
    dim3 grid(p.grid_x, mk_cdiv(a.samples, MT));
    hipLaunchKernelGGL((packed_matvec_kernel<BITS, XT, MT, C, UNIFORM>), grid, dim3(p.threads),
                       p.lds_bytes, stream, a);
}

template <int BITS, int XT, bool UNIFORM>
bool dispatch_tile(const MatvecArgs &a, const Plan &p, hipStream_t stream) {
#define MK_CASE(MT_, C_)                                              \
    if (p.sample_tile == MT_ && p.chunks == C_) {                     \
        launch_chunked<BITS, XT, MT_, C_, UNIFORM>(a, p, stream);     \
        return true;                                                  \
    }
    MK_CASE(1, 1) MK_CASE(1, 2) MK_CASE(1, 4) MK_CASE(1, 8)
    MK_CASE(2, 1) MK_CASE(2, 2) MK_CASE(2, 4)
    MK_CASE(4, 1) MK_CASE(4, 2)
    if constexpr (XT != MK_F32) { MK_CASE(8, 1) }
#undef MK_CASE
    return false;
}

template <int BITS>
bool dispatch_bits(const MatvecArgs &a, const Plan &p, int x_dtype, bool uniform, hipStream_t stream) {
    if (uniform) {
        if (x_dtype == MK_F16) return dispatch_tile<BITS, MK_F16, true>(a, p, stream);
        if (x_dtype == MK_BF16) return dispatch_tile<BITS, MK_BF16, true>(a, p, stream);
        return dispatch_tile<BITS, MK_F32, true>(a, p, stream);
    }
    if (x_dtype == MK_F16) return dispatch_tile<BITS, MK_F16, false>(a, p, stream);
    if (x_dtype == MK_BF16) return dispatch_tile<BITS, MK_BF16, false>(a, p, stream);
    return dispatch_tile<BITS, MK_F32, false>(a, p, stream);
}

}  // namespace mk_matvec
