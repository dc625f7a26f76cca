// Packed matvec for 2- to 8-bit codes of any scalar grid (integer grids, NF4, small
// codebooks) with fp16 or bf16 activations and 16-bit scales, rows of K = 32 ... 16384 codes (K % 32 == 0).
//
// Adjacent codes (one, two or four, by code width) index a table of 16-bit values held in
// LDS, so one LDS read decodes up to four weights and one v_dot2_f32_f16 (v_dot2_f32_bf16)
// per pair multiplies them with the matching activations, accumulating in fp32.  Table entries are the grid
// values rounded to the activations' type (exact for integer grids and minifloats; NF4-like
// tables lose at most half an ulp of that type per weight, as the activations themselves do).  Entries of different
// pairs fall in different LDS banks except by coincidence, so the lookups mostly proceed
// at full rate.  Work split, load order and the reduction are those of the 4-bit streaming
// kernel: a workgroup of ceil(K/2048) wavefronts owns 16 rows; lane t owns codes [32t, 32t + 32)
// of every row; codes are requested eight rows ahead; per-wavefront row sums meet in LDS in
// a fixed order.
//
// Replaces the reference's Triton kernel `packed_matrix_vector`
// (kernels/packed_linear.py:107-173 in /root/reference/src/mlkit) for these layouts.

#include "packed_matvec_impl.h"

namespace mk_matvec {

namespace {

constexpr int kPairRows = 16;
// Rows of codes in flight per wavefront: eight rows of 16 bytes per lane, or as many wider
// rows as hold the same number of bytes.
template <int BITS>
constexpr int rows_in_flight() {
    return BITS <= 4 ? 8 : 32 / BITS;
}

// A 16-bit scale or offset (fp16 or bf16, uniform per launch) as fp32.
__device__ __forceinline__ float side_value(uint16_t raw, int dtype) {
    const float from_half = static_cast<float>(__builtin_bit_cast(_Float16, raw));
    const float from_brain = __uint_as_float(static_cast<uint32_t>(raw) << 16);
    return dtype == MK_F16 ? from_half : from_brain;
}

template <int MT>
constexpr int pair_reduce_rows() {
    return kPairRows * MT <= 64 ? kPairRows : 64 / MT;
}

// LOOKUP = codes decoded per table read: 1 (an entry is one 16-bit value; two reads make a
// pair), 2 (an entry is one pair) or 4 (two pairs).  Wider fields mean fewer reads but a
// table of 2^(LOOKUP * BITS) entries that every workgroup has to fill first.
//
// Byte offset into the table of field i of a chunk of BITS dwords.  i is a compile-time
// constant after unrolling.
template <int BITS, int LOOKUP>
__device__ __forceinline__ uint32_t lookup_offset(const CodeChunk<BITS> &c, int i) {
    constexpr int kField = LOOKUP * BITS;
    constexpr int kEntryShift = LOOKUP == 4 ? 3 : LOOKUP == 2 ? 2 : 1;
    constexpr uint32_t mask = ((1u << kField) - 1u) << kEntryShift;
    const int bit = i * kField;
    const int word = bit >> 5, shift = bit & 31;
    if (shift + kField <= 32) {
        if (shift >= kEntryShift) return (c.w[word] >> (shift - kEntryShift)) & mask;
        return (c.w[word] << (kEntryShift - shift)) & mask;
    }
    return (__builtin_amdgcn_alignbit(c.w[(word + 1) % BITS], c.w[word], shift) << kEntryShift) & mask;
}

template <int BITS, int MT, bool HAS_ZERO, int XT, int LOOKUP>
__global__ void __launch_bounds__(512) pairs_kernel(const Stream4Args a) {
    constexpr int kLookup = LOOKUP;
    constexpr int kPairAhead = rows_in_flight<BITS>();
    constexpr int kEntries = 1 << (kLookup * BITS);
    constexpr int kTableWords = kEntries * kLookup / 2;
    constexpr int kEntryWords = kLookup >= 2 ? kLookup / 2 : 1;
    __shared__ __attribute__((aligned(8))) uint32_t table[kTableWords];  // 16-bit values, pairs or double pairs
    __shared__ float partials[64 * 8];    // [row sum][wavefront]
    constexpr int kReduceRows = pair_reduce_rows<MT>();
    constexpr int kSums = kReduceRows * MT;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int row_base = blockIdx.x * kPairRows;
    const int sample_base = blockIdx.y * MT;
    const uint32_t row_bytes = (static_cast<uint32_t>(a.width) * BITS) >> 3;
    const uint8_t *codes_base = a.packed + static_cast<size_t>(row_base) * row_bytes;  // uniform
    // Lanes past the end of a row (K is not a multiple of 2048) read chunk 0 with zeroed
    // activations: they add nothing.
    const bool in_row = tid * kChunkCodes < a.width;
    const int chunk = in_row ? tid : 0;
    const uint32_t code_offset = static_cast<uint32_t>(chunk) * (4u * BITS);

    // The grid's values first (one global load per value), then every table entry from them.
    __shared__ float grid_values[1 << BITS];
    for (int code = tid; code < (1 << BITS); code += blockDim.x) {
        float value = 0.0f;
        if (a.uniform) value = __builtin_fmaf(static_cast<float>(code), a.grid_step, a.grid_min);
        else if (code < a.n_values) value = a.values[code];
        grid_values[code] = value;
    }
    __syncthreads();
    for (int word = tid; word < kTableWords; word += blockDim.x) {
        int low, high;  // the codes whose values share this dword
        if constexpr (kLookup == 1) {
            low = 2 * word;
            high = 2 * word + 1;
        } else {
            const int entry = word / kEntryWords, half = word - entry * kEntryWords;
            low = (entry >> (2 * half * BITS)) & ((1 << BITS) - 1);
            high = (entry >> ((2 * half + 1) * BITS)) & ((1 << BITS) - 1);
        }
        const float first = grid_values[low];
        const float second = grid_values[high];
        if constexpr (XT == MK_F16) {
            const mk_h2 pair = {static_cast<_Float16>(first), static_cast<_Float16>(second)};
            table[word] = __builtin_bit_cast(uint32_t, pair);
        } else {
            table[word] = static_cast<uint32_t>(mk_float_to_bf16(first)) | (static_cast<uint32_t>(mk_float_to_bf16(second)) << 16);
        }
    }
    // Also aligns the wavefronts, so that nobody's small loads queue behind another's codes.
    __syncthreads();

    XChunk<XT> x[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int sample = sample_base + m < a.samples ? sample_base + m : a.samples - 1;
        load_x_chunk<XT>(x[m], a.x, static_cast<size_t>(sample) * a.width + static_cast<size_t>(chunk) * kChunkCodes);
    }
    const uint32_t group_offset = ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * 2u;
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * 2u;
    const uint8_t *scale_base = static_cast<const uint8_t *>(a.scales) + static_cast<size_t>(row_base) * scale_row_bytes;
    const uint8_t *zero_base = HAS_ZERO ? static_cast<const uint8_t *>(a.zeros) + static_cast<size_t>(row_base) * scale_row_bytes
                                        : nullptr;
    uint16_t scale_raw[kPairRows], zero_raw[HAS_ZERO ? kPairRows : 1];
#pragma unroll
    for (int r = 0; r < kPairRows; ++r) {
        scale_raw[r] = *reinterpret_cast<const uint16_t *>(scale_base + static_cast<size_t>(r) * scale_row_bytes + group_offset);
        if constexpr (HAS_ZERO)
            zero_raw[r] = *reinterpret_cast<const uint16_t *>(zero_base + static_cast<size_t>(r) * scale_row_bytes + group_offset);
    }
    __builtin_amdgcn_sched_barrier(0);

    CodeChunk<BITS> codes[kPairRows];
#pragma unroll
    for (int r = 0; r < kPairAhead; ++r) {
        load_codes<BITS>(codes[r], codes_base + static_cast<size_t>(r) * row_bytes + code_offset);
        __builtin_amdgcn_sched_barrier(0);  // in row order
    }

    float x_sum[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const uint32_t keep = in_row && sample_base + m < a.samples ? 0xffffffffu : 0u;
#pragma unroll
        for (int i = 0; i < 16; ++i) x[m].r[i] &= keep;
        x_sum[m] = HAS_ZERO ? chunk_sum<XT>(x[m]) : 0.0f;
    }

    const uint8_t *table_bytes = reinterpret_cast<const uint8_t *>(table);
#pragma unroll
    for (int pass = 0; pass < kPairRows / kReduceRows; ++pass) {
        float sums[kSums];
#pragma unroll
        for (int j = 0; j < kReduceRows; ++j) {
            const int r = pass * kReduceRows + j;
            float dot[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) dot[m] = 0.0f;
#pragma unroll
            for (int i = 0; i < (kLookup == 1 ? 16 : 32 / kLookup); ++i) {
                uint32_t entry[kEntryWords];
                if constexpr (kLookup == 4) {
                    const mk_u32x2 both = *reinterpret_cast<const mk_u32x2 *>(table_bytes + lookup_offset<BITS, 4>(codes[r], i));
                    entry[0] = both.x;
                    entry[1] = both.y;
                } else if constexpr (kLookup == 2) {
                    entry[0] = *reinterpret_cast<const uint32_t *>(table_bytes + lookup_offset<BITS, 2>(codes[r], i));
                } else {
                    const uint32_t even = *reinterpret_cast<const uint16_t *>(table_bytes + lookup_offset<BITS, 1>(codes[r], 2 * i));
                    const uint32_t odd = *reinterpret_cast<const uint16_t *>(table_bytes + lookup_offset<BITS, 1>(codes[r], 2 * i + 1));
                    entry[0] = even | (odd << 16);
                }
#pragma unroll
                for (int h = 0; h < kEntryWords; ++h)
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        const uint32_t inputs = x[m].r[kEntryWords * i + h];
                        if constexpr (XT == MK_F16)
                            dot[m] = __builtin_amdgcn_fdot2(__builtin_bit_cast(mk_h2, entry[h]),
                                                            __builtin_bit_cast(mk_h2, inputs), dot[m], false);
                        else
                            dot[m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(mk_bf2, entry[h]),
                                                                     __builtin_bit_cast(mk_bf2, inputs), dot[m], false);
                    }
            }
            if (r + kPairAhead < kPairRows)
                load_codes<BITS>(codes[r + kPairAhead],
                                 codes_base + static_cast<size_t>(r + kPairAhead) * row_bytes + code_offset);
            const float scale = side_value(scale_raw[r], a.scale_dtype);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float value = scale * dot[m];
                if constexpr (HAS_ZERO) value = __builtin_fmaf(side_value(zero_raw[r], a.scale_dtype), x_sum[m], value);
                sums[j * MT + m] = value;
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        transposed_wave_sum<kSums>(sums, lane);
        if (pass > 0) __syncthreads();
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
                const size_t index = static_cast<size_t>(sample) * a.rows + row;
                if constexpr (XT == MK_F16)
                    static_cast<_Float16 *>(a.y)[index] = static_cast<_Float16>(total);
                else
                    static_cast<uint16_t *>(a.y)[index] = mk_float_to_bf16(total);
            }
        }
    }
}

template <int BITS, int MT, int XT, int LOOKUP>
void launch_tile_with(const Stream4Args &a, int tiles, hipStream_t stream) {
    const dim3 grid(tiles, mk_cdiv(a.samples, MT));
    const dim3 block(mk_cdiv(a.width, 2048) * 64);
    if (a.zeros)
        hipLaunchKernelGGL((pairs_kernel<BITS, MT, true, XT, LOOKUP>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((pairs_kernel<BITS, MT, false, XT, LOOKUP>), grid, block, 0, stream, a);
}

// Field width per code width: the widest whose table a workgroup fills quickly.
template <int BITS, int MT, int XT>
void launch_tile_as(const Stream4Args &a, int tiles, hipStream_t stream) {
    if constexpr (BITS == 2) {
        launch_tile_with<BITS, MT, XT, 4>(a, tiles, stream);                                   // 256 entries
    } else if constexpr (BITS == 3) {
        if (a.width >= 8192) launch_tile_with<BITS, MT, XT, 4>(a, tiles, stream);              // 4096 entries
        else launch_tile_with<BITS, MT, XT, 2>(a, tiles, stream);                              // 64
    } else if constexpr (BITS <= 5) {
        launch_tile_with<BITS, MT, XT, 2>(a, tiles, stream);                                   // 256 / 1024
    } else if constexpr (BITS == 6) {
        if (a.width >= 4096) launch_tile_with<BITS, MT, XT, 2>(a, tiles, stream);              // 4096
        else launch_tile_with<BITS, MT, XT, 1>(a, tiles, stream);                              // 64
    } else {
        launch_tile_with<BITS, MT, XT, 1>(a, tiles, stream);                                   // 128 / 256
    }
}

template <int BITS, int MT>
void launch_tile(const Stream4Args &a, int tiles, hipStream_t stream) {
    if (a.x_dtype == MK_F16) launch_tile_as<BITS, MT, MK_F16>(a, tiles, stream);
    else launch_tile_as<BITS, MT, MK_BF16>(a, tiles, stream);
}

template <int BITS>
void launch_bits(const Stream4Args &a, int tiles, hipStream_t stream) {
    int tile = 1;
    while (tile < a.samples && tile < 8) tile <<= 1;
    switch (tile) {
        case 1: launch_tile<BITS, 1>(a, tiles, stream); break;
        case 2: launch_tile<BITS, 2>(a, tiles, stream); break;
        case 4: launch_tile<BITS, 4>(a, tiles, stream); break;
        default: launch_tile<BITS, 8>(a, tiles, stream); break;
    }
}

}  // namespace

bool pairs_accepts(int width, int group, int bits, int x_dtype, int scale_dtype) {
    return bits >= 2 && bits <= 8 && x_dtype != MK_F32 && scale_dtype != MK_F32 && width % kChunkCodes == 0 &&
           width <= 16384 && (group % kChunkCodes == 0 || group >= width);
}

// Multiplies rows [0, 16 * tiles); returns the number of rows covered.
int pairs_launch(const Stream4Args &a, hipStream_t stream) {
    const int tiles = a.rows / kPairRows;
    if (tiles == 0) return 0;
    switch (a.bits) {
        case 2: launch_bits<2>(a, tiles, stream); break;
        case 3: launch_bits<3>(a, tiles, stream); break;
        case 4: launch_bits<4>(a, tiles, stream); break;
        case 5: launch_bits<5>(a, tiles, stream); break;
        case 6: launch_bits<6>(a, tiles, stream); break;
        case 7: launch_bits<7>(a, tiles, stream); break;
        default: launch_bits<8>(a, tiles, stream); break;
    }
    return tiles * kPairRows;
}

}  // namespace mk_matvec
