// 4-bit uniform-grid packed matvec with fp16 activations and fp16 scales: the decode-time
// kernel for INT4 layers whose rows are whole multiples of 32 codes (K = 32 ... 16384).
//
// The kernel is bound by whichever is larger: the HBM stream of the codes, or the vector
// ALU time of the busiest SIMD (a wavefront issues one vector instruction per four
// cycles).  With one workgroup per compute unit the second term is
// (instructions per wavefront) x (wavefronts per SIMD) x 4 cycles, so this file is written
// for instruction count: straight-line code, uniform (scalar) row addresses, scales
// loaded by the lane that uses them, nine vector instructions per eight codes, and one
// transposed reduction for all rows of a wavefront instead of one reduction per row.
//
// Work split: a workgroup of ceil(K/2048) wavefronts multiplies 16 adjacent rows; lane `tid`
// owns codes [32 tid, 32 tid + 32) of every row and keeps the matching activations of
// all samples in registers.  Codes are requested eight rows ahead of the row being
// summed.  Per-wavefront row sums meet in LDS in a fixed order, so results do not depend
// on scheduling.
//
// Replaces the reference's Triton kernel `packed_matrix_vector`
// (kernels/packed_linear.py:107-173 in /root/reference/src/mlkit) for this layout.

#include "packed_matvec_impl.h"

namespace mk_matvec {

namespace {

// Rows per workgroup: 16 when that still gives every compute unit a workgroup, 4 for
// layers with fewer rows (more, shorter workgroups).  Up to 8 rows of codes are in flight
// per wavefront (both values swept on the GPU together with 8 / 32 rows and 4 - 16 ahead).
constexpr int kWideRows = 16, kNarrowRows = 4;

template <int ROWS>
constexpr int rows_ahead_of() {
    return ROWS < 8 ? ROWS : 8;
}

// Rows per transposed reduction: all 16 when that is at most 64 sums per lane (measured
// faster than splitting the reduction to hide part of it behind the stream).
template <int MT, int ROWS>
constexpr int reduce_rows() {
    return ROWS * MT <= 64 ? ROWS : 64 / MT;
}

template <int MT, bool HAS_ZERO, int ROWS>
__global__ void __launch_bounds__(512) stream4_kernel(const Stream4Args a) {
    __shared__ float partials[64 * 8];  // [row sum][wavefront]
    constexpr int kStreamRows = ROWS;
    constexpr int kStreamAhead = rows_ahead_of<ROWS>();
    constexpr int kReduceRows = reduce_rows<MT, ROWS>();
    constexpr int kSums = kReduceRows * MT;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int row_base = blockIdx.x * kStreamRows;
    const int sample_base = blockIdx.y * MT;
    const uint32_t row_bytes = static_cast<uint32_t>(a.width) >> 1;
    const uint8_t *codes_base = a.packed + static_cast<size_t>(row_base) * row_bytes;  // uniform
    // Lanes past the end of a row (K is not a multiple of 2048) read chunk 0 with zeroed
    // activations: they add nothing.
    const bool in_row = tid * kChunkCodes < a.width;
    const int chunk = in_row ? tid : 0;
    const uint32_t code_offset = static_cast<uint32_t>(chunk) * 16u;

    // The workgroup is aligned first: a compute unit serves loads first come, first served,
    // and a wavefront that starts late would queue its small loads behind the others' codes.
    __syncthreads();

    // Activations: 32 per sample, as 16 fp16 pairs (L2 hits).
    XChunk<MK_F16> x[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int sample = sample_base + m < a.samples ? sample_base + m : a.samples - 1;
        load_x_chunk<MK_F16>(x[m], a.x, static_cast<size_t>(sample) * a.width + static_cast<size_t>(chunk) * kChunkCodes);
    }
    // The scale (and offset) of this lane's chunk in every row, 2 bytes each.
    const uint32_t group_offset = ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * 2u;
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * 2u;
    const uint8_t *scale_base = static_cast<const uint8_t *>(a.scales) + static_cast<size_t>(row_base) * scale_row_bytes;
    const uint8_t *zero_base = HAS_ZERO ? static_cast<const uint8_t *>(a.zeros) + static_cast<size_t>(row_base) * scale_row_bytes
                                        : nullptr;
    uint16_t scale_raw[kStreamRows], zero_raw[HAS_ZERO ? kStreamRows : 1];
#pragma unroll
    for (int r = 0; r < kStreamRows; ++r) {
        scale_raw[r] = *reinterpret_cast<const uint16_t *>(scale_base + static_cast<size_t>(r) * scale_row_bytes + group_offset);
        if constexpr (HAS_ZERO)
            zero_raw[r] = *reinterpret_cast<const uint16_t *>(zero_base + static_cast<size_t>(r) * scale_row_bytes + group_offset);
    }
    __builtin_amdgcn_sched_barrier(0);

    CodeChunk<4> codes[kStreamRows];
#pragma unroll
    for (int r = 0; r < kStreamAhead; ++r) {
        load_codes<4>(codes[r], codes_base + static_cast<size_t>(r) * row_bytes + code_offset);
        __builtin_amdgcn_sched_barrier(0);  // in row order
    }

    // sum_k (min + step c_k) x_k = step * dot + min * sum(x) - step * (code-free part of dot).
    float x_sum[MT], grid_term[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const uint32_t keep = in_row && sample_base + m < a.samples ? 0xffffffffu : 0u;
#pragma unroll
        for (int i = 0; i < 16; ++i) x[m].r[i] &= keep;
        const float code_free = pair_for_nibbles(x[m], &x_sum[m]);
        grid_term[m] = a.grid_min * x_sum[m] - a.grid_step * code_free;
    }

#pragma unroll
    for (int pass = 0; pass < kStreamRows / kReduceRows; ++pass) {
        float sums[kSums];
#pragma unroll
        for (int j = 0; j < kReduceRows; ++j) {
            const int r = pass * kReduceRows + j;
            float dot[MT];
            chunk_dot<4, MK_F16, MT, true>(codes[r], x, nullptr, dot);
            if (r + kStreamAhead < kStreamRows)
                load_codes<4>(codes[r + kStreamAhead],
                              codes_base + static_cast<size_t>(r + kStreamAhead) * row_bytes + code_offset);
            const float scale = static_cast<float>(__builtin_bit_cast(_Float16, scale_raw[r]));
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float value = scale * __builtin_fmaf(a.grid_step, dot[m], grid_term[m]);
                if constexpr (HAS_ZERO)
                    value = __builtin_fmaf(static_cast<float>(__builtin_bit_cast(_Float16, zero_raw[r])), x_sum[m], value);
                sums[j * MT + m] = value;
            }
            // Keeps the rows in arrival order and their temporaries short-lived.
            __builtin_amdgcn_sched_barrier(0);
        }

        // All row sums of this pass over the 64 lanes at once, then over the wavefronts.
        transposed_wave_sum<kSums>(sums, lane);
        if (pass > 0) __syncthreads();  // the previous pass's readers are done
        if (lane < kSums) partials[transposed_value_of_lane<kSums>(lane) * 8 + wave] = sums[0];
        __syncthreads();
        if (tid < kSums) {
            float total = partials[tid * 8];
#pragma unroll
            for (int w = 1; w < 8; ++w) total += w < waves ? partials[tid * 8 + w] : 0.0f;
            const int j = tid / MT, m = tid - j * MT;
            const int row = row_base + pass * kReduceRows + j;
            const int sample = sample_base + m;
            if (sample < a.samples) {
                if (a.bias) total += mk_load_as_float(a.bias, row, a.bias_dtype);
                static_cast<_Float16 *>(a.y)[static_cast<size_t>(sample) * a.rows + row] = static_cast<_Float16>(total);
            }
        }
    }
}

template <int MT, int ROWS>
void launch_tile(const Stream4Args &a, int tiles, hipStream_t stream) {
    const dim3 grid(tiles, mk_cdiv(a.samples, MT));
    const dim3 block(mk_cdiv(a.width, 2048) * 64);
    if (a.zeros)
        hipLaunchKernelGGL((stream4_kernel<MT, true, ROWS>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((stream4_kernel<MT, false, ROWS>), grid, block, 0, stream, a);
}

template <int ROWS>
int launch_rows(const Stream4Args &a, hipStream_t stream) {
    const int tiles = a.rows / ROWS;
    if (tiles == 0) return 0;
    int tile = 1;
    while (tile < a.samples && tile < 8) tile <<= 1;
    switch (tile) {
        case 1: launch_tile<1, ROWS>(a, tiles, stream); break;
        case 2: launch_tile<2, ROWS>(a, tiles, stream); break;
        case 4: launch_tile<4, ROWS>(a, tiles, stream); break;
        default: launch_tile<8, ROWS>(a, tiles, stream); break;
    }
    return tiles * ROWS;
}

}  // namespace

bool stream4_accepts(int width, int group, int bits, int x_dtype, int scale_dtype, bool uniform) {
    return bits == 4 && uniform && x_dtype == MK_F16 && scale_dtype == MK_F16 && width % kChunkCodes == 0 &&
           width <= 16384 && (group % kChunkCodes == 0 || group >= width);
}

// Multiplies the leading whole tiles of rows; returns the number of rows covered.
int stream4_launch(const Stream4Args &a, hipStream_t stream) {
    constexpr int kComputeUnits = 256;
    if (a.rows / kWideRows >= kComputeUnits) return launch_rows<kWideRows>(a, stream);
    return launch_rows<kNarrowRows>(a, stream);
}

}  // namespace mk_matvec
