// Packed matvec for 2- to 8-bit codes of any scalar grid (integer grids, NF4, small
// codebooks) with fp16 or bf16 activations and 16-bit scales, rows of K = 32 ... 131072 codes (K % 32 == 0).
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

#include <type_traits>

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

// Rows of a workgroup of the v_dot2 kernel.  A single sample with long rows leaves the
// wavefronts waiting on table lookups, so its rows are spread over twice as many workgroups
// (two per CU at 4096 rows); short rows keep sixteen rows per table fill.
constexpr int kShortTileRows = 8;
constexpr int kShortTileWidth = 4096;
// A workgroup of eight wavefronts covers 16384 codes of a row at once; longer rows (up to eight times that) take
// several turns (the LONG kernels), with sixteen rows per workgroup and table decoding.
constexpr int kMostRowCodes = 16384;
constexpr int kMostTurns = 8;
// Uniform 2-, 3- and 8-bit grids with fp16 activations, one or two samples: decoded by shifts and masks.
inline bool shifted_decoding(const Stream4Args &a) {
    return a.uniform && a.x_dtype == MK_F16 && (a.bits == 2 || a.bits == 3 || a.bits == 8) && a.samples <= 2 && a.width <= kMostRowCodes;
}

// (Without lookups to wait on, sixteen rows per workgroup measure faster: 5.8 against 6.0 us for two bits, 6.5
// against 6.8 us for three bits at 4096 x 14336.)
inline int tile_rows(const Stream4Args &a) {
    return a.samples == 1 && a.width >= kShortTileWidth && a.width <= kMostRowCodes && !shifted_decoding(a) ? kShortTileRows : kPairRows;
}

template <int MT, int ROWS>
constexpr int pair_reduce_rows() {
    return ROWS * MT <= 64 ? ROWS : 64 / MT;
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

// Fills `table` (kEntries * LOOKUP / 2 dwords) with the grid's values as 16-bit floats: one
// value, one pair or two pairs per entry.  The grid's values come first (one global load per
// value), then every entry from them.  Ends before the caller's barrier.
template <int BITS, int LOOKUP, int XT>
__device__ __forceinline__ void fill_table(uint32_t *table, const Stream4Args &a) {
    constexpr int kLookup = LOOKUP;
    constexpr int kEntries = 1 << (kLookup * BITS);
    constexpr int kTableWords = kEntries * kLookup / 2;
    constexpr int kEntryWords = kLookup >= 2 ? kLookup / 2 : 1;
    const int tid = threadIdx.x;
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
}

// ---- uniform 2- and 3-bit grids without a table ----------------------------------------------
//
// A code c left where it is in the low ten bits of a half word IS the fp16 number c * 2^(p - 24),
// p its bit position: a subnormal, and v_dot2_f32_f16 multiplies subnormal inputs exactly.  So one
// AND with a mask that keeps one code in each half of a (shifted) word of the stream makes an fp16
// pair of two codes, and one v_dot2 multiplies it with the two matching activations.  Pairs whose
// codes sit at the same position share a power of two; each such class has its own sum and the
// classes meet once per chunk.  Nothing is looked up and nothing has to be removed afterwards;
// the affine map of the grid is applied to the chunk's sum.
//
// Two bits: a word holds codes 0 - 7 in its low half and 8 - 15 in its high half; code i and code
// i + 8 sit at the same position of their halves.  Positions 0, 2, 4, 6 of the word and of the
// word shifted by 8: nine instructions (one shift, eight ANDs) and eight v_dot2 per 16 codes.
//
// Three bits: the chunk is a string of 96 bits, code i at bit 3 i.  A 32-bit window at bit 3 a - 1
// has codes a, a + 1, a + 2 at positions 1, 4, 7 of its low half and codes a + 5, a + 6, a + 7 at
// positions 0, 3, 6 of its high half: three ANDs make the pairs (a, a + 5) (a + 1, a + 6)
// (a + 2, a + 7), whose low codes count double, so the activations of the low codes are kept
// halved (exact).  Windows at a = 0, 3, 10, 13, 20, 23 (the second of each ten codes with two pairs
// only) and one at a = 30 for the last two codes: seven funnel shifts, seventeen ANDs and
// seventeen v_dot2 per 32 codes, classes 1, 8, 64.

template <int BITS>
struct ShiftedPlan;

template <>
struct ShiftedPlan<2> {
    static constexpr int kPairs = 16, kClasses = 4;
    // pair k of word j (k = 4 s + i: position 2 i of the word shifted by 8 s): codes 16 j + 4 s + i and + 8
    static constexpr int low_code(int pair) { return 16 * (pair / 8) + (pair % 8); }
    static constexpr int high_code(int pair) { return low_code(pair) + 8; }
    static constexpr bool halve_low = false;
};

template <>
struct ShiftedPlan<3> {
    static constexpr int kPairs = 17, kClasses = 3;
    // ten codes per two windows: pairs (b, b+5) (b+1, b+6) (b+2, b+7) | (b+3, b+8) (b+4, b+9); then 30 and 31 alone
    static constexpr int low_code(int pair) { return pair < 15 ? 10 * (pair / 5) + pair % 5 : 30 + (pair - 15); }
    static constexpr int high_code(int pair) { return pair < 15 ? low_code(pair) + 5 : -1; }
    static constexpr bool halve_low = true;
};

// Eight bits: a byte left in the low byte of a half word is the subnormal c * 2^-24 as it stands (eight of the ten
// mantissa bits).  A word holds codes 4 j ... 4 j + 3; the word and the word shifted by 8, each masked with
// 0x00ff00ff, are the pairs (4 j, 4 j + 2) and (4 j + 1, 4 j + 3): one shift, two ANDs and two v_dot2 per four codes,
// one class.
template <>
struct ShiftedPlan<8> {
    static constexpr int kPairs = 16, kClasses = 2;   // (two sums only to shorten the dependent chains)
    static constexpr int low_code(int pair) { return 4 * (pair / 2) + (pair % 2); }
    static constexpr int high_code(int pair) { return low_code(pair) + 2; }
    static constexpr bool halve_low = false;
};

// The activations of a chunk as the pairs of the plan, from their natural order (x.r[k] = elements 2 k, 2 k + 1).
template <int BITS>
__device__ __forceinline__ void pair_for_shifted_codes(const XChunk<MK_F16> &x, uint32_t (&pairs)[ShiftedPlan<BITS>::kPairs]) {
    using Plan = ShiftedPlan<BITS>;
    const mk_h2 half_low = {static_cast<_Float16>(0.5f), static_cast<_Float16>(1.0f)};
#pragma unroll
    for (int k = 0; k < Plan::kPairs; ++k) {
        const int low = Plan::low_code(k), high = Plan::high_code(k);
        uint32_t pair;
        if (high >= 0) {
            const uint32_t selector = ((low & 1) ? 0x0302u : 0x0100u) | ((high & 1) ? 0x07060000u : 0x05040000u);
            pair = __builtin_amdgcn_perm(x.r[high >> 1], x.r[low >> 1], selector);
        } else {
            pair = (low & 1) ? x.r[low >> 1] >> 16 : x.r[low >> 1] & 0xffffu;
        }
        if (Plan::halve_low) pair = __builtin_bit_cast(uint32_t, __builtin_bit_cast(mk_h2, pair) * half_low);
        pairs[k] = pair;
    }
}

// sum_k code_k x_k of a chunk for MT samples, times 2^-24.
template <int BITS, int MT>
__device__ __forceinline__ void shifted_chunk_dot(const CodeChunk<BITS> &codes, const uint32_t (&pairs)[MT][ShiftedPlan<BITS>::kPairs],
                                                  float (&dot)[MT]) {
    using Plan = ShiftedPlan<BITS>;
    float sums[Plan::kClasses][MT];
#pragma unroll
    for (int c = 0; c < Plan::kClasses; ++c)
#pragma unroll
        for (int m = 0; m < MT; ++m) sums[c][m] = 0.0f;
    auto add = [&](int cls, uint32_t fields, int pair) __attribute__((always_inline)) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            sums[cls][m] = __builtin_amdgcn_fdot2(__builtin_bit_cast(mk_h2, fields), __builtin_bit_cast(mk_h2, pairs[m][pair]), sums[cls][m], false);
    };
    if constexpr (BITS == 8) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t word = codes.w[j];
            add(0, word & 0x00ff00ffu, 2 * j);
            add(1, (word >> 8) & 0x00ff00ffu, 2 * j + 1);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) dot[m] = sums[0][m] + sums[1][m];
    } else if constexpr (BITS == 2) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t word = codes.w[j], shifted = word >> 8;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                add(i, word & (0x00030003u << (2 * i)), 8 * j + i);
                add(i, shifted & (0x00030003u << (2 * i)), 8 * j + 4 + i);
            }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m)
            dot[m] = __builtin_fmaf(sums[3][m], 0.015625f, __builtin_fmaf(sums[2][m], 0.0625f, __builtin_fmaf(sums[1][m], 0.25f, sums[0][m])));
    } else {
        // window at bit `offset` (may be -1) of the 96-bit string w[0] | w[1] << 32 | w[2] << 64
        auto window = [&](int offset) __attribute__((always_inline)) {
            if (offset < 0) return codes.w[0] << 1;
            const int word = offset >> 5, shift = offset & 31;
            const uint32_t low = codes.w[word], high = word + 1 < 3 ? codes.w[word + 1] : 0u;
            return shift == 0 ? low : __builtin_amdgcn_alignbit(high, low, shift);
        };
#pragma unroll
        for (int b = 0; b < 3; ++b) {
            const uint32_t first = window(30 * b - 1), second = window(30 * b + 8);
            add(0, first & 0x0007000eu, 5 * b);          // low code at position 1, high code at position 0
            add(1, first & 0x00380070u, 5 * b + 1);      // positions 4 and 3
            add(2, first & 0x01c00380u, 5 * b + 2);      // positions 7 and 6
            add(0, second & 0x0007000eu, 5 * b + 3);
            add(1, second & 0x00380070u, 5 * b + 4);
        }
        const uint32_t last = window(89);
        add(0, last & 0x0000000eu, 15);
        add(1, last & 0x00000070u, 16);
#pragma unroll
        for (int m = 0; m < MT; ++m)
            dot[m] = __builtin_fmaf(sums[2][m], 0.015625f, __builtin_fmaf(sums[1][m], 0.125f, sums[0][m]));
    }
}

// SHIFTED: a uniform 2- or 3-bit grid with fp16 activations, decoded by shifts and masks (no table).
// LONG: rows of more than 16384 codes.  The workgroup covers the row in `phases` turns of blockDim.x chunks, each
// with its own activations, scales and stream of codes, and adds the turns' row sums before the reduction.
template <int BITS, int MT, bool HAS_ZERO, int XT, int LOOKUP, int ROWS, bool SHIFTED = false, bool LONG = false>
__global__ void __launch_bounds__(512) pairs_kernel(const Stream4Args a, const Stream4Group members) {
    static_assert(!SHIFTED || ((BITS == 2 || BITS == 3 || BITS == 8) && XT == MK_F16), "shifted decoding: 2, 3 or 8 bits, fp16 activations");
    static_assert(!LONG || (ROWS * MT <= 64 && !SHIFTED), "long rows: one reduction for all rows of the tile, table decoding");
    constexpr int kLookup = LOOKUP;
    constexpr int kPairRows = ROWS;
    constexpr int kPairAhead = rows_in_flight<BITS>();
    constexpr int kEntries = 1 << (kLookup * BITS);
    constexpr int kTableWords = kEntries * kLookup / 2;
    constexpr int kEntryWords = kLookup >= 2 ? kLookup / 2 : 1;
    __shared__ __attribute__((aligned(8))) uint32_t table[kTableWords];  // 16-bit values, pairs or double pairs
    __shared__ float partials[64 * 8];    // [row sum][wavefront]
    constexpr int kReduceRows = pair_reduce_rows<MT, ROWS>();
    constexpr int kSums = kReduceRows * MT;

    // The matrix of this workgroup: the launch's only one, or member blockIdx.z of a group.
    const TileSource source = tile_source<ROWS>(a, members, blockIdx.z);
    if (static_cast<int>(blockIdx.x) >= source.tiles) return;  // a shorter member: the whole workgroup leaves
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int row_base = blockIdx.x * kPairRows;
    const int sample_base = blockIdx.y * MT;
    const uint32_t row_bytes = (static_cast<uint32_t>(a.width) * BITS) >> 3;
    const uint8_t *codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;  // uniform
    if constexpr (!SHIFTED) fill_table<BITS, LOOKUP, XT>(table, a);
    // Also aligns the wavefronts, so that nobody's small loads queue behind another's codes.
    __syncthreads();

    const int turn_codes = static_cast<int>(blockDim.x) * kChunkCodes;
    const int phases = LONG ? (a.width + turn_codes - 1) / turn_codes : 1;   // uniform
    float long_sums[LONG ? kSums : 1];
    for (int phase = 0; phase < phases; ++phase) {
    // Lanes past the end of a row (K is not a multiple of 2048) read chunk 0 with zeroed
    // activations: they add nothing.
    const int wanted_chunk = LONG ? phase * static_cast<int>(blockDim.x) + tid : tid;
    const bool in_row = wanted_chunk * kChunkCodes < a.width;
    const int chunk = in_row ? wanted_chunk : 0;
    const uint32_t code_offset = static_cast<uint32_t>(chunk) * (4u * BITS);

    XChunk<XT> x[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int sample = sample_base + m < a.samples ? sample_base + m : a.samples - 1;
        load_x_chunk<XT>(x[m], source.x, static_cast<size_t>(sample) * a.width + static_cast<size_t>(chunk) * kChunkCodes);
    }
    const uint32_t group_offset = ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * 2u;
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * 2u;
    const uint8_t *scale_base = source.scales + static_cast<size_t>(row_base) * scale_row_bytes;
    const uint8_t *zero_base = HAS_ZERO ? source.zeros + static_cast<size_t>(row_base) * scale_row_bytes : nullptr;
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
        x_sum[m] = HAS_ZERO || SHIFTED ? chunk_sum<XT>(x[m]) : 0.0f;
    }
    // shifted decoding: the activations as the plan's pairs; the affine map of the grid applies to a chunk's sum:
    // sum (min + step c) x = (step 2^24) (2^-24 sum c x) + min sum x
    constexpr int kPlanPairs = SHIFTED ? ShiftedPlan<SHIFTED ? BITS : 2>::kPairs : 1;   // (BITS has a plan whenever SHIFTED)
    uint32_t shifted_pairs[MT][kPlanPairs];
    float grid_term[MT];
    if constexpr (SHIFTED) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            pair_for_shifted_codes<BITS>(x[m], shifted_pairs[m]);
            grid_term[m] = a.grid_min * x_sum[m];
        }
    }
    const float shifted_step = a.grid_step * 16777216.0f;

    const uint8_t *table_bytes = reinterpret_cast<const uint8_t *>(table);
    // The table entries of a row are read one row ahead of their use: the reads of row r + 1 are in flight (and
    // queue behind each other in the banks they share) while the dot products of row r are issued.
    constexpr int kLookups = kLookup == 1 ? 16 : 32 / kLookup;
    uint32_t looked_up[SHIFTED ? 1 : kLookups][kEntryWords], looked_up_next[SHIFTED ? 1 : kLookups][kEntryWords];
    auto look_up = [&](int r, uint32_t (&entry)[SHIFTED ? 1 : kLookups][kEntryWords]) __attribute__((always_inline)) {
        if constexpr (!SHIFTED) {
#pragma unroll
            for (int i = 0; i < kLookups; ++i) {
                if constexpr (kLookup == 4) {
                    const mk_u32x2 both = *reinterpret_cast<const mk_u32x2 *>(table_bytes + lookup_offset<BITS, 4>(codes[r], i));
                    entry[i][0] = both.x;
                    entry[i][1] = both.y;
                } else if constexpr (kLookup == 2) {
                    entry[i][0] = *reinterpret_cast<const uint32_t *>(table_bytes + lookup_offset<BITS, 2>(codes[r], i));
                } else {
                    const uint32_t even = *reinterpret_cast<const uint16_t *>(table_bytes + lookup_offset<BITS, 1>(codes[r], 2 * i));
                    const uint32_t odd = *reinterpret_cast<const uint16_t *>(table_bytes + lookup_offset<BITS, 1>(codes[r], 2 * i + 1));
                    entry[i][0] = even | (odd << 16);
                }
            }
        }
    };
    look_up(0, looked_up_next);
#pragma unroll
    for (int pass = 0; pass < kPairRows / kReduceRows; ++pass) {
        float sums[kSums];
#pragma unroll
        for (int j = 0; j < kReduceRows; ++j) {
            const int r = pass * kReduceRows + j;
            float dot[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) dot[m] = 0.0f;
            if constexpr (SHIFTED) {
                shifted_chunk_dot<BITS, MT>(codes[r], shifted_pairs, dot);
#pragma unroll
                for (int m = 0; m < MT; ++m) dot[m] = __builtin_fmaf(shifted_step, dot[m], grid_term[m]);
            } else {
#pragma unroll
                for (int i = 0; i < kLookups; ++i)
#pragma unroll
                    for (int h = 0; h < kEntryWords; ++h) looked_up[i][h] = looked_up_next[i][h];
                if (r + 1 < kPairRows) look_up(r + 1, looked_up_next);
                __builtin_amdgcn_sched_barrier(0);   // the next row's reads are issued before this row's products
#pragma unroll
                for (int i = 0; i < kLookups; ++i)
#pragma unroll
                    for (int h = 0; h < kEntryWords; ++h)
#pragma unroll
                        for (int m = 0; m < MT; ++m) {
                            const uint32_t inputs = x[m].r[kEntryWords * i + h];
                            if constexpr (XT == MK_F16)
                                dot[m] = __builtin_amdgcn_fdot2(__builtin_bit_cast(mk_h2, looked_up[i][h]),
                                                                __builtin_bit_cast(mk_h2, inputs), dot[m], false);
                            else
                                dot[m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(mk_bf2, looked_up[i][h]),
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

        if constexpr (LONG) {   // (one pass holds all rows of the tile)
#pragma unroll
            for (int k = 0; k < kSums; ++k) long_sums[k] = phase == 0 ? sums[k] : long_sums[k] + sums[k];
            if (phase + 1 < phases) break;   // the next turn of the row
#pragma unroll
            for (int k = 0; k < kSums; ++k) sums[k] = long_sums[k];
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
                if (source.bias) total += mk_load_as_float(source.bias, row, a.bias_dtype);
                store_output<XT>(source.y, static_cast<size_t>(sample) * source.rows + row, total);
            }
        }
    }
    }
}

// ---- three to eight samples: the dot products on the matrix cores -------------------------
//
// As in the 4-bit streaming kernel: v_mfma_f32_4x4x4_16B_{f16,bf16} multiplies sixteen
// independent 4 x 4 x 4 blocks, block b being "rows 4 q ... 4 q + 3 of the weight x four
// samples over four adjacent codes of chunk b".  Lane 4 b + t looks up the values of row t's
// codes (two table reads per four codes, or one for double-pair tables) and holds sample
// t's activations for chunk b in their natural order.  A wavefront owns 2048 codes of K as
// four sub-slices of sixteen chunks; the four row sums of a result lane take their scales
// from the four lanes of its quad.
// SHIFTED (uniform 8-bit grids, fp16 activations): no table; a word and the word shifted by 8, each masked with
// 0x00ff00ff, are the four codes of one instruction as fp16 subnormals (in the order 0, 2, 1, 3, which the
// activations are permuted to once per tile), and the grid's affine map applies to the block's sums.
// LONG: rows of more than 16384 codes, covered in `phases` turns of the workgroup's width (see pairs_kernel).
template <int BITS, int SETS, bool HAS_ZERO, int XT, int LOOKUP, int SLICES, bool SHIFTED = false, bool LONG = false>
__global__ void __launch_bounds__(512) pairs_blocks_kernel(const Stream4Args a, const Stream4Group members) {
    static_assert(!SHIFTED || (BITS == 8 && XT == MK_F16), "shifted decoding on the matrix cores: 8 bits, fp16 activations");
    constexpr int kQuads = kPairRows / 4;
    constexpr int kSlices = SLICES;  // sub-slices of sixteen chunks per wavefront (rows of up to 512 / 1024 codes: 1 / 2)
    constexpr int kSteps = kQuads * kSlices;
    constexpr int kAhead = rows_in_flight<BITS>() < kSteps ? rows_in_flight<BITS>() : kSteps;
    constexpr int kEntries = 1 << (LOOKUP * BITS);
    constexpr int kTableWords = SHIFTED ? 2 : kEntries * LOOKUP / 2;
    __shared__ __attribute__((aligned(8))) uint32_t table[kTableWords];
    __shared__ float partials[SETS * kPairRows * 4 * 8];  // [set][row][sample in set][wavefront]
    extern __shared__ __attribute__((aligned(16))) uint32_t x_slices_storage[];
    constexpr int kSampleWords = blocks_sample_words(SLICES);

    // The matrix of this workgroup: the launch's only one, or member blockIdx.z of a group.
    const TileSource source = tile_source<kPairRows>(a, members, blockIdx.z);
    if (static_cast<int>(blockIdx.x) >= source.tiles) return;  // a shorter member: the whole workgroup leaves
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int block = lane >> 2, t = lane & 3;
    uint32_t *const x_slice = x_slices_storage + wave * (4 * kSampleWords);   // one buffer per sample of a set
    const int row_base = blockIdx.x * kPairRows;
    const uint32_t row_bytes = (static_cast<uint32_t>(a.width) * BITS) >> 3;
    const uint8_t *codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;  // uniform
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * 2u;
    const uint8_t *scale_base = source.scales + static_cast<size_t>(row_base) * scale_row_bytes;
    const uint8_t *zero_base = HAS_ZERO ? source.zeros + static_cast<size_t>(row_base) * scale_row_bytes : nullptr;

    if constexpr (!SHIFTED) fill_table<BITS, LOOKUP, XT>(table, a);

    float sums[SETS][kPairRows];
#pragma unroll
    for (int set = 0; set < SETS; ++set)
#pragma unroll
        for (int j = 0; j < kPairRows; ++j) sums[set][j] = 0.0f;

    const int turn_codes = waves * (512 * kSlices);
    const int phases = LONG ? (a.width + turn_codes - 1) / turn_codes : 1;   // uniform
    for (int phase = 0; phase < phases; ++phase) {
    const int phase_wave = LONG ? phase * waves + wave : wave;
    // Chunks past the end of a row (K is not a multiple of 2048) read chunk 0 with zeroed
    // activations: they add nothing.
    bool in_row[kSlices];
    uint32_t code_offset[kSlices], group_offset[kSlices];
#pragma unroll
    for (int s = 0; s < kSlices; ++s) {
        const int wanted = phase_wave * (16 * kSlices) + s * 16 + block;
        in_row[s] = wanted * kChunkCodes < a.width;
        const int chunk = in_row[s] ? wanted : 0;
        code_offset[s] = static_cast<uint32_t>(t) * row_bytes + static_cast<uint32_t>(chunk) * (4u * BITS);
        group_offset[s] = static_cast<uint32_t>(t) * scale_row_bytes +
                          ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * 2u;
    }
    if (!LONG || phase == 0) __syncthreads();  // the table is complete; also aligns the wavefronts before their loads

    // Activations of sample t (and t + 4) for this lane's four chunks: the slices of a set's
    // four samples are read coalesced and parked side by side; every lane picks its sample's chunks.
    XChunk<XT> x[SETS][kSlices];
#pragma unroll
    for (int set = 0; set < SETS; ++set) {
        mk_u32x4 pieces[4][kSlices];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int wanted_sample = blockIdx.y * 4 * SETS + 4 * set + j;
            const int sample = wanted_sample < a.samples ? wanted_sample : a.samples - 1;
#pragma unroll
            for (int i = 0; i < kSlices; ++i) pieces[j][i] = request_piece(source.x, a.width, sample, phase_wave * (512 * kSlices), i, lane);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < kSlices; ++i) park_piece_swizzled(x_slice + j * kSampleWords, i, lane, pieces[j][i]);
        wave_exchange_fence();
#pragma unroll
        for (int s = 0; s < kSlices; ++s) chunk_from_swizzled_slice(x[set][s], x_slice + t * kSampleWords, s * 16 + block);
        wave_exchange_fence();   // the next set's pieces go to the same buffers
    }
    uint16_t scale_raw[kSteps], zero_raw[HAS_ZERO ? kSteps : 1];
#pragma unroll
    for (int q = 0; q < kQuads; ++q)
#pragma unroll
        for (int s = 0; s < kSlices; ++s) {
            const size_t quad_offset = static_cast<size_t>(4 * q) * scale_row_bytes;
            scale_raw[q * kSlices + s] = *reinterpret_cast<const uint16_t *>(scale_base + quad_offset + group_offset[s]);
            if constexpr (HAS_ZERO)
                zero_raw[q * kSlices + s] = *reinterpret_cast<const uint16_t *>(zero_base + quad_offset + group_offset[s]);
        }
    __builtin_amdgcn_sched_barrier(0);

    CodeChunk<BITS> codes[kSteps];
#pragma unroll
    for (int step = 0; step < kAhead; ++step) {
        load_codes<BITS>(codes[step], codes_base + static_cast<size_t>(4 * (step / kSlices)) * row_bytes + code_offset[step % kSlices]);
        __builtin_amdgcn_sched_barrier(0);  // in order
    }

    float x_sum[SETS][kSlices];
#pragma unroll
    for (int set = 0; set < SETS; ++set) {
        const bool sample_present = blockIdx.y * 4 * SETS + 4 * set + t < a.samples;
#pragma unroll
        for (int s = 0; s < kSlices; ++s) {
            const bool kept = in_row[s] && sample_present;
            if (__builtin_amdgcn_ballot_w64(!kept) != 0) {  // uniform; rarely taken
                const uint32_t keep = kept ? 0xffffffffu : 0u;
#pragma unroll
                for (int i = 0; i < 16; ++i) x[set][s].r[i] &= keep;
            }
            x_sum[set][s] = HAS_ZERO || SHIFTED ? chunk_sum<XT>(x[set][s]) : 0.0f;
            if constexpr (SHIFTED) {   // (x0,x1)(x2,x3) -> (x0,x2)(x1,x3) for every four values
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t p0 = x[set][s].r[2 * i], p1 = x[set][s].r[2 * i + 1];
                    x[set][s].r[2 * i] = __builtin_amdgcn_perm(p1, p0, 0x05040100u);
                    x[set][s].r[2 * i + 1] = __builtin_amdgcn_perm(p1, p0, 0x07060302u);
                }
            }
        }
    }
    const float shifted_step = a.grid_step * 16777216.0f;   // the subnormal codes are c * 2^-24

    auto blocks = [](uint32_t a_low, uint32_t a_high, uint32_t b_low, uint32_t b_high, mk_f4 sum) __attribute__((always_inline)) {
        const mk_u32x2 left = {a_low, a_high}, right = {b_low, b_high};
        if constexpr (XT == MK_F16)
            return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(mk_h4, left), __builtin_bit_cast(mk_h4, right), sum, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(mk_s4, left), __builtin_bit_cast(mk_s4, right), sum, 0, 0, 0);
    };
    const uint8_t *table_bytes = reinterpret_cast<const uint8_t *>(table);

    // The table entries of a step are read one step ahead of their use (as in pairs_kernel).
    uint32_t looked_up[8][2], looked_up_next[8][2];
    auto look_up = [&](int step, uint32_t (&entry)[8][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {  // codes 4 i ... 4 i + 3
            if constexpr (LOOKUP == 4) {
                const mk_u32x2 both = *reinterpret_cast<const mk_u32x2 *>(table_bytes + lookup_offset<BITS, 4>(codes[step], i));
                entry[i][0] = both.x, entry[i][1] = both.y;
            } else if constexpr (LOOKUP == 2) {
                entry[i][0] = *reinterpret_cast<const uint32_t *>(table_bytes + lookup_offset<BITS, 2>(codes[step], 2 * i));
                entry[i][1] = *reinterpret_cast<const uint32_t *>(table_bytes + lookup_offset<BITS, 2>(codes[step], 2 * i + 1));
            } else {
                const uint32_t v0 = *reinterpret_cast<const uint16_t *>(table_bytes + lookup_offset<BITS, 1>(codes[step], 4 * i));
                const uint32_t v1 = *reinterpret_cast<const uint16_t *>(table_bytes + lookup_offset<BITS, 1>(codes[step], 4 * i + 1));
                const uint32_t v2 = *reinterpret_cast<const uint16_t *>(table_bytes + lookup_offset<BITS, 1>(codes[step], 4 * i + 2));
                const uint32_t v3 = *reinterpret_cast<const uint16_t *>(table_bytes + lookup_offset<BITS, 1>(codes[step], 4 * i + 3));
                entry[i][0] = v0 | (v1 << 16), entry[i][1] = v2 | (v3 << 16);
            }
        }
    };
    if constexpr (!SHIFTED) look_up(0, looked_up_next);
#pragma unroll
    for (int step = 0; step < kSteps; ++step) {
        const int q = step / kSlices, s = step % kSlices;
        mk_f4 dot[SETS];
#pragma unroll
        for (int set = 0; set < SETS; ++set) dot[set] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (SHIFTED) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t word = codes[step].w[i];
                const uint32_t low = word & 0x00ff00ffu, high = (word >> 8) & 0x00ff00ffu;
#pragma unroll
                for (int set = 0; set < SETS; ++set)
                    dot[set] = blocks(low, high, x[set][s].r[2 * i], x[set][s].r[2 * i + 1], dot[set]);
            }
#pragma unroll
            for (int set = 0; set < SETS; ++set)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    dot[set][r] = __builtin_fmaf(shifted_step, dot[set][r], a.grid_min * x_sum[set][s]);
        } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) looked_up[i][0] = looked_up_next[i][0], looked_up[i][1] = looked_up_next[i][1];
        if (step + 1 < kSteps) look_up(step + 1, looked_up_next);
        __builtin_amdgcn_sched_barrier(0);   // the next step's reads are issued before this step's products
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int set = 0; set < SETS; ++set)
                dot[set] = blocks(looked_up[i][0], looked_up[i][1], x[set][s].r[2 * i], x[set][s].r[2 * i + 1], dot[set]);
        }
        if (step + kAhead < kSteps)
            load_codes<BITS>(codes[step + kAhead], codes_base + static_cast<size_t>(4 * ((step + kAhead) / kSlices)) * row_bytes +
                                                       code_offset[(step + kAhead) % kSlices]);
        // Row 4 q + r of the block: scale (and offset) come from lane r of the quad.
        const float scale = side_as_float(scale_raw[step], a.scale_dtype);
        float zero = 0.0f;
        if constexpr (HAS_ZERO) zero = side_as_float(zero_raw[step], a.scale_dtype);
        auto add_row = [&](auto r) __attribute__((always_inline)) {
            constexpr int R = decltype(r)::value;
#pragma unroll
            for (int set = 0; set < SETS; ++set) {
                float total = __builtin_fmaf(quad_value<R>(scale), dot[set][R], sums[set][4 * q + R]);
                if constexpr (HAS_ZERO) total = __builtin_fmaf(quad_value<R>(zero), x_sum[set][s], total);
                sums[set][4 * q + R] = total;
            }
        };
        add_row(std::integral_constant<int, 0>{});
        add_row(std::integral_constant<int, 1>{});
        add_row(std::integral_constant<int, 2>{});
        add_row(std::integral_constant<int, 3>{});
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (LONG) wave_exchange_fence();   // the next turn's activations go to the same LDS buffers
    }

    // Over the sixteen blocks of the wavefront (lane bits 2 - 5), then over the wavefronts.
#pragma unroll
    for (int set = 0; set < SETS; ++set) {
        transposed_wave_sum<kPairRows, 2>(sums[set], lane);
        partials[((set * kPairRows + transposed_value_of_lane<kPairRows>(lane >> 2)) * 4 + t) * 8 + wave] = sums[set][0];
    }
    __syncthreads();
    for (int index = tid; index < SETS * kPairRows * 4; index += blockDim.x) {  // a workgroup may be one wavefront
        float total = partials[index * 8];
#pragma unroll
        for (int w = 1; w < 8; ++w) total += w < waves ? partials[index * 8 + w] : 0.0f;
        const int set = index / (kPairRows * 4), row = row_base + (index / 4) % kPairRows;
        const int sample = blockIdx.y * 4 * SETS + 4 * set + (index & 3);
        if (sample < a.samples) {
            if (source.bias) total += mk_load_as_float(source.bias, row, a.bias_dtype);
            store_output<XT>(source.y, static_cast<size_t>(sample) * source.rows + row, total);
        }
    }
}

template <int BITS, int SETS, int XT, int LOOKUP, int SLICES>
void launch_blocks_sliced(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    const dim3 grid(tiles, mk_cdiv(a.samples, 4 * SETS), members.count > 0 ? members.count : 1);
    const bool long_rows = a.width > kMostRowCodes;   // several turns of an equal share of the row (in whole wavefronts)
    const dim3 block(mk_cdiv(long_rows ? mk_cdiv(a.width, mk_cdiv(a.width, kMostRowCodes)) : a.width, 512 * SLICES) * 64);
    const size_t slices = static_cast<size_t>(block.x / 64) * 4 * blocks_sample_words(SLICES) * sizeof(uint32_t);
    // More than 64 KB of dynamic LDS has to be allowed per kernel (static LDS counts against
    // the CU's 160 KB too, so only what this launch needs is asked for).
    auto launch = [&](auto kernel) {
        static size_t allowed = 64 * 1024;
        if (slices > allowed) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(slices));
            allowed = slices;
        }
        hipLaunchKernelGGL(kernel, grid, block, slices, stream, a, members);
    };
    if constexpr (SLICES == 4 && SETS == 1) {   // (long rows take four samples per pass: launch_bits)
        if (long_rows) {
            if (a.zeros) launch(pairs_blocks_kernel<BITS, SETS, true, XT, LOOKUP, SLICES, false, true>);
            else launch(pairs_blocks_kernel<BITS, SETS, false, XT, LOOKUP, SLICES, false, true>);
            return;
        }
    }
    if constexpr (BITS == 8 && XT == MK_F16) {
        if (a.uniform) {   // no table: the bytes as fp16 subnormals
            if (a.zeros) launch(pairs_blocks_kernel<BITS, SETS, true, XT, LOOKUP, SLICES, true>);
            else launch(pairs_blocks_kernel<BITS, SETS, false, XT, LOOKUP, SLICES, true>);
            return;
        }
    }
    if (a.zeros) launch(pairs_blocks_kernel<BITS, SETS, true, XT, LOOKUP, SLICES>);
    else launch(pairs_blocks_kernel<BITS, SETS, false, XT, LOOKUP, SLICES>);
}

// Short rows get fewer sub-slices per wavefront, so that none lies wholly past the row's end.
template <int BITS, int SETS, int XT, int LOOKUP>
void launch_blocks_with(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if (a.width <= 1024) launch_blocks_sliced<BITS, SETS, XT, LOOKUP, 2>(a, members, tiles, stream);
    else launch_blocks_sliced<BITS, SETS, XT, LOOKUP, 4>(a, members, tiles, stream);
}

template <int BITS, int MT, int XT, int LOOKUP>
void launch_tile_with(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    const dim3 grid(tiles, mk_cdiv(a.samples, MT), members.count > 0 ? members.count : 1);
    if (a.width > kMostRowCodes) {   // several turns of an equal share of the row (in whole wavefronts)
        const dim3 half(mk_cdiv(mk_cdiv(a.width, mk_cdiv(a.width, kMostRowCodes)), 2048) * 64);
        if (a.zeros)
            hipLaunchKernelGGL((pairs_kernel<BITS, MT, true, XT, LOOKUP, kPairRows, false, true>), grid, half, 0, stream, a, members);
        else
            hipLaunchKernelGGL((pairs_kernel<BITS, MT, false, XT, LOOKUP, kPairRows, false, true>), grid, half, 0, stream, a, members);
        return;
    }
    const dim3 block(mk_cdiv(a.width, 2048) * 64);
    if constexpr ((BITS == 2 || BITS == 3 || BITS == 8) && XT == MK_F16 && MT <= 2) {
        if (shifted_decoding(a)) {
            if (a.zeros) {
                hipLaunchKernelGGL((pairs_kernel<BITS, MT, true, XT, LOOKUP, kPairRows, true>), grid, block, 0, stream, a, members);
            } else {
                hipLaunchKernelGGL((pairs_kernel<BITS, MT, false, XT, LOOKUP, kPairRows, true>), grid, block, 0, stream, a, members);
            }
            return;
        }
    }
    if constexpr (MT == 1) {
        if (tile_rows(a) == kShortTileRows) {
            if (a.zeros)
                hipLaunchKernelGGL((pairs_kernel<BITS, MT, true, XT, LOOKUP, kShortTileRows>), grid, block, 0, stream, a, members);
            else
                hipLaunchKernelGGL((pairs_kernel<BITS, MT, false, XT, LOOKUP, kShortTileRows>), grid, block, 0, stream, a, members);
            return;
        }
    }
    if (a.zeros)
        hipLaunchKernelGGL((pairs_kernel<BITS, MT, true, XT, LOOKUP, kPairRows>), grid, block, 0, stream, a, members);
    else
        hipLaunchKernelGGL((pairs_kernel<BITS, MT, false, XT, LOOKUP, kPairRows>), grid, block, 0, stream, a, members);
}

// Field width per code width: the widest whose table a workgroup fills quickly.
template <int BITS, int MT, int XT>
void launch_tile_as(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if constexpr (BITS == 2) {
        launch_tile_with<BITS, MT, XT, 4>(a, members, tiles, stream);                                   // 256 entries
    } else if constexpr (BITS == 3) {
        if (a.width >= 8192) launch_tile_with<BITS, MT, XT, 4>(a, members, tiles, stream);              // 4096 entries
        else launch_tile_with<BITS, MT, XT, 2>(a, members, tiles, stream);                              // 64
    } else if constexpr (BITS <= 5) {
        launch_tile_with<BITS, MT, XT, 2>(a, members, tiles, stream);                                   // 256 / 1024
    } else if constexpr (BITS == 6) {
        if (a.width >= 4096) launch_tile_with<BITS, MT, XT, 2>(a, members, tiles, stream);              // 4096
        else launch_tile_with<BITS, MT, XT, 1>(a, members, tiles, stream);                              // 64
    } else {
        launch_tile_with<BITS, MT, XT, 1>(a, members, tiles, stream);                                   // 128 / 256
    }
}

template <int BITS, int MT>
void launch_tile(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if (a.x_dtype == MK_F16) launch_tile_as<BITS, MT, MK_F16>(a, members, tiles, stream);
    else launch_tile_as<BITS, MT, MK_BF16>(a, members, tiles, stream);
}

// The same field widths for the matrix-core kernel.
template <int BITS, int SETS, int XT>
void launch_blocks_as(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if constexpr (BITS == 2) {
        launch_blocks_with<BITS, SETS, XT, 4>(a, members, tiles, stream);
    } else if constexpr (BITS == 3) {
        // (eight wavefronts' activation buffers leave no room for the 32 KB table)
        if (a.width >= 8192 && a.width <= 14336) launch_blocks_with<BITS, SETS, XT, 4>(a, members, tiles, stream);
        else launch_blocks_with<BITS, SETS, XT, 2>(a, members, tiles, stream);
    } else if constexpr (BITS <= 5) {
        launch_blocks_with<BITS, SETS, XT, 2>(a, members, tiles, stream);
    } else if constexpr (BITS == 6) {
        if (a.width >= 4096) launch_blocks_with<BITS, SETS, XT, 2>(a, members, tiles, stream);
        else launch_blocks_with<BITS, SETS, XT, 1>(a, members, tiles, stream);
    } else {
        launch_blocks_with<BITS, SETS, XT, 1>(a, members, tiles, stream);
    }
}

template <int BITS, int SETS>
void launch_blocks(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if (a.x_dtype == MK_F16) launch_blocks_as<BITS, SETS, MK_F16>(a, members, tiles, stream);
    else launch_blocks_as<BITS, SETS, MK_BF16>(a, members, tiles, stream);
}

template <int BITS>
void launch_bits(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if (a.samples >= 3) {  // measured against the v_dot2 kernel at 4096 x 14336
        // (two sets of four samples and a sum carried over the turns of a long row do not fit the registers)
        if (a.samples <= 4 || a.width > kMostRowCodes) launch_blocks<BITS, 1>(a, members, tiles, stream);
        else launch_blocks<BITS, 2>(a, members, tiles, stream);
        return;
    }
    if (a.samples == 1) launch_tile<BITS, 1>(a, members, tiles, stream);
    else launch_tile<BITS, 2>(a, members, tiles, stream);
}

}  // namespace

bool pairs_accepts(int width, int group, int bits, int x_dtype, int scale_dtype) {
    return bits >= 2 && bits <= 8 && x_dtype != MK_F32 && scale_dtype != MK_F32 && width % kChunkCodes == 0 &&
           width <= kMostTurns * kMostRowCodes && (group % kChunkCodes == 0 || group >= width);
}

namespace {

void launch_for_bits(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    switch (a.bits) {
        case 2: launch_bits<2>(a, members, tiles, stream); break;
        case 3: launch_bits<3>(a, members, tiles, stream); break;
        case 4: launch_bits<4>(a, members, tiles, stream); break;
        case 5: launch_bits<5>(a, members, tiles, stream); break;
        case 6: launch_bits<6>(a, members, tiles, stream); break;
        case 7: launch_bits<7>(a, members, tiles, stream); break;
        default: launch_bits<8>(a, members, tiles, stream); break;
    }
}

}  // namespace

// Multiplies the leading whole tiles of rows; returns the number of rows covered.
int pairs_launch(const Stream4Args &a, hipStream_t stream) {
    const int tile = tile_rows(a);
    const int tiles = a.rows / tile;
    if (tiles == 0) return 0;
    Stream4Group none;
    none.count = 0;
    none.widest_tiles = 0;
    launch_for_bits(a, none, tiles, stream);
    return tiles * tile;
}

int pairs_launch_group(const Stream4Args &shared, Stream4Group &group, const int *member_rows, int *rows_per_tile,
                       hipStream_t stream) {
    const int tile = tile_rows(shared);
    int widest = 0;
    for (int i = 0; i < group.count; ++i) {
        group.member[i].rows = member_rows[i];
        group.member[i].tiles = member_rows[i] / tile;
        if (group.member[i].tiles > widest) widest = group.member[i].tiles;
    }
    group.widest_tiles = widest;
    *rows_per_tile = tile;
    if (widest == 0) return 0;
    Stream4Args a = shared;
    a.zeros = group.member[0].zeros;  // selects the kernel variant; the members agree on it
    launch_for_bits(a, group, widest, stream);
    return 0;
}

}  // namespace mk_matvec
