// Vector grids on gfx950: nearest-codeword search (any codebook of 2-, 4-, 8- or
// 16-dimensional codewords; the structured search of the E8P lattice) and the LDL
// error-feedback tile that rounds blocks of `dimension` columns.
//
// One wavefront owns a row (or a vector): its 64 lanes share out the codebook entries -- four
// E8P magnitude patterns per lane, or every 64th codeword -- and the winner is found by a
// reduction over (cost, index) in which the lower index wins ties, which is what a search in
// ascending order with a strict comparison returns; the reduction moves values between lanes
// with vector-ALU lane moves only.  Costs are formed in fp32 without fused multiply-adds,
// coordinates in ascending order.  The magnitude patterns, and any codebook of up to 48 KiB,
// are staged in LDS once per workgroup.
//
// In the feedback tile everything a row needs of the tile lives in the wavefront's registers,
// lane l holding columns l, l + 64, ...: weights, corrections, scales on the way in,
// reconstructions and codes on the way out (read and written with coalesced accesses before
// and after the block loop).  A block's values are read out of them with wavefront-uniform
// lane reads.  Inside the loop the only memory traffic is the coefficient rows of the NEXT
// block, requested before the search of the current one so that their latency hides behind it.
// An E8P point is rebuilt from its pattern, sign bits and coset instead of being fetched from
// the 2 MiB table.
//
// Replaces, in /root/reference/src/mlkit:
//   kernels/lattice_search.py:10-70       nearest_lattice_code / nearest_lattice -> mk_vector_nearest
//   kernels/error_feedback.py:146-274     round_vector_feedback_tile / round_vector_tile
//                                                                   -> mk_feedback_round_vector_tile

#include "mk_common.h"

namespace {

constexpr int kPatternsPerLane = 4;   // 256 E8P magnitude patterns over 64 lanes
constexpr int kPatternFloats = 256 * 8;
constexpr int kWaveRows = 4;          // wavefronts (rows) per workgroup
constexpr int kStagedBytes = 48 * 1024;

extern __shared__ __align__(16) float staged[];

// The value lane `lane ^ (1 << STAGE)` holds (DPP inside rows of 16 lanes, v_permlane16_swap /
// v_permlane32_swap across rows).
template <int STAGE>
__device__ __forceinline__ int partner(int bits, int lane) {
    if constexpr (STAGE == 0) return __builtin_amdgcn_mov_dpp(bits, 0xB1, 0xf, 0xf, true);   // quad_perm [1,0,3,2]
    else if constexpr (STAGE == 1) return __builtin_amdgcn_mov_dpp(bits, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    else if constexpr (STAGE == 2) {
        int moved = __builtin_amdgcn_update_dpp(bits, bits, 0x104, 0xf, 0x5, false);   // row_shl:4 into lanes 0-3, 8-11
        return __builtin_amdgcn_update_dpp(moved, bits, 0x114, 0xf, 0xa, false);       // row_shr:4 into lanes 4-7, 12-15
    } else if constexpr (STAGE == 3) return __builtin_amdgcn_mov_dpp(bits, 0x128, 0xf, 0xf, true);  // row_ror:8
    else if constexpr (STAGE == 4) {
        const auto swapped = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
        return (lane & 16) ? swapped[0] : swapped[1];
    } else {
        const auto swapped = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
        return (lane & 32) ? swapped[0] : swapped[1];
    }
}

template <int STAGE>
__device__ __forceinline__ void best_of_pair(float &cost, int &index, int lane) {
    const float other_cost = __builtin_bit_cast(float, partner<STAGE>(__builtin_bit_cast(int, cost), lane));
    const int other_index = partner<STAGE>(index, lane);
    const bool take = other_cost < cost || (other_cost == cost && other_index < index);
    cost = take ? other_cost : cost;
    index = take ? other_index : index;
}

// The smaller cost wins, the smaller index on equal costs; every lane receives the result.
__device__ __forceinline__ void wave_best(float &cost, int &index, int lane) {
    best_of_pair<0>(cost, index, lane);
    best_of_pair<1>(cost, index, lane);
    best_of_pair<2>(cost, index, lane);
    best_of_pair<3>(cost, index, lane);
    best_of_pair<4>(cost, index, lane);
    best_of_pair<5>(cost, index, lane);
}

// v_readlane with a wavefront-uniform lane index.
__device__ __forceinline__ float lane_value(float value, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, value), lane));
}

// This lane's four magnitude patterns (pattern lane + 64 j) and their squared norms.
struct LanePatterns {
    float value[kPatternsPerLane][8];
    float norm[kPatternsPerLane];
};

// `patterns`: the 256 x 8 table in LDS.
__device__ __forceinline__ void load_patterns(LanePatterns &p, const float *patterns, int lane) {
#pragma unroll
    for (int j = 0; j < kPatternsPerLane; ++j) {
        float norm = 0.0f;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            const float value = patterns[(lane + 64 * j) * 8 + d];
            p.value[j][d] = value;
            norm = __fadd_rn(norm, __fmul_rn(value, value));
        }
        p.norm[j] = norm;
    }
}

// Code of the E8P point nearest to v, and the point itself (all lanes hold the same v and
// receive the same answer).  Per coset every lane scores its four patterns -- the flip of the
// cheapest coordinate priced in when the pattern's parity disagrees with the signs of v -- the
// wavefront agrees on the winner, and only then are the winner's parity correction and its
// first cheapest coordinate worked out, from its row of the table in LDS.
__device__ __forceinline__ int nearest_lattice_code(const float (&v)[8], const LanePatterns &p, const float *patterns,
                                                    int lane, float (&point)[8]) {
    float best_cost = __builtin_inff();
    int best_code = 0;
    {   // Code 0 (pattern 0, no sign bits, the +1/4 coset): the answer when no cost compares below infinity (NaN).
        float total = 0.0f;
#pragma unroll
        for (int d = 0; d < 8; ++d) total += patterns[d];
        const int parity = static_cast<int>(total) & 1;
#pragma unroll
        for (int d = 0; d < 8; ++d) point[d] = __fadd_rn((d == 7 && parity) ? -patterns[d] : patterns[d], 0.25f);
    }
#pragma unroll
    for (int coset = 0; coset < 2; ++coset) {
        const float shift = coset == 0 ? -0.25f : 0.25f;
        float absolute[8];
        int negatives = 0, sign_bits = 0;
        float squares = 0.0f;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            const float centered = __fsub_rn(v[d], shift);
            absolute[d] = __builtin_fabsf(centered);
            const int negative = centered < 0.0f ? 1 : 0;
            negatives += negative;
            if (d < 7) sign_bits |= negative << d;
            squares = __fadd_rn(squares, __fmul_rn(centered, centered));
        }
        const int sign_parity = negatives & 1;
        float cost = __builtin_inff();
        int pattern = 0;
#pragma unroll
        for (int j = 0; j < kPatternsPerLane; ++j) {
            float dots = 0.0f, cheapest = __builtin_inff(), total = 0.0f;
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                const float product = __fmul_rn(absolute[d], p.value[j][d]);
                dots = __fadd_rn(dots, product);
                cheapest = __builtin_fminf(cheapest, product);
                total += p.value[j][d];  // a sum of half-integers: exact, and constant per lane
            }
            const int mismatch = (static_cast<int>(total) & 1) != sign_parity ? 1 : 0;
            float candidate = __fsub_rn(__fadd_rn(squares, p.norm[j]), __fmul_rn(2.0f, dots));
            candidate = __fadd_rn(candidate, __fmul_rn(__fmul_rn(4.0f, cheapest), static_cast<float>(mismatch)));
            if (candidate < cost) {  // ascending pattern index within the lane
                cost = candidate;
                pattern = lane + 64 * j;
            }
        }
        wave_best(cost, pattern, lane);
        if (cost < best_cost) {  // uniform; the -1/4 coset stays on a tie
            float row[8], total = 0.0f, cheapest = __builtin_inff();
            int axis = 0;
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                row[d] = patterns[pattern * 8 + d];
                total += row[d];
                const float product = __fmul_rn(absolute[d], row[d]);
                if (product < cheapest) {  // the first minimum
                    cheapest = product;
                    axis = d;
                }
            }
            const int parity = static_cast<int>(total) & 1;
            const int flipped = (parity != sign_parity && axis < 7) ? (1 << axis) : 0;
            const int signs = sign_bits ^ flipped;
            best_cost = cost;
            best_code = pattern * 128 + signs + (coset == 0 ? 32768 : 0);
            const int eighth = (__builtin_popcount(signs) + parity) & 1;
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                const int negative = d < 7 ? (signs >> d) & 1 : eighth;
                point[d] = __fadd_rn(negative ? -row[d] : row[d], shift);
            }
        }
    }
    return best_code;
}

// Index of the nearest of `count` codewords of DIM floats (lowest index on ties).
template <int DIM>
__device__ __forceinline__ int nearest_codeword(const float (&v)[DIM], const float *codebook, int count, int lane) {
    float cost = __builtin_inff();
    int index = 0x7fffffff;
    for (int entry = lane; entry < count; entry += 64) {
        const float *word = codebook + static_cast<size_t>(entry) * DIM;
        float candidate = 0.0f;
#pragma unroll
        for (int d = 0; d < DIM; ++d) {
            const float difference = __fsub_rn(word[d], v[d]);
            candidate = __fadd_rn(candidate, __fmul_rn(difference, difference));
        }
        if (candidate < cost) {
            cost = candidate;
            index = entry;
        }
    }
    wave_best(cost, index, lane);
    return index < count ? index : 0;  // no cost compared below infinity (NaN inputs): the first codeword
}

// Copies the workgroup's table into LDS: the magnitude patterns of the lattice, or the whole
// codebook when STAGED says it fits.
template <int DIM, bool LATTICE, bool STAGED>
__device__ __forceinline__ void stage_table(const float *codebook, int codebook_size) {
    const float *source = LATTICE ? codebook + static_cast<size_t>(codebook_size) * 8 : codebook;
    const int floats = LATTICE ? kPatternFloats : (STAGED ? codebook_size * DIM : 0);
    for (int i = threadIdx.x; i < floats; i += blockDim.x) staged[i] = source[i];
    __syncthreads();
}

struct NearestArgs {
    const float *vectors;
    const float *codebook;  // [count, dim]; lattice: the 256 magnitude patterns follow
    int32_t *codes;
    long long vectors_count;
    int count;
};

template <int DIM, bool LATTICE, bool STAGED>
__global__ void __launch_bounds__(256) vector_nearest_kernel(const NearestArgs a) {
    stage_table<DIM, LATTICE, STAGED>(a.codebook, a.count);
    const int lane = threadIdx.x & 63;
    const long long wave = static_cast<long long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const long long waves = static_cast<long long>(gridDim.x) * (blockDim.x >> 6);
    LanePatterns patterns;
    if constexpr (LATTICE) load_patterns(patterns, staged, lane);
    for (long long vector = wave; vector < a.vectors_count; vector += waves) {
        float v[DIM];
#pragma unroll
        for (int d = 0; d < DIM; ++d) v[d] = a.vectors[vector * DIM + d];
        int code;
        if constexpr (LATTICE) {
            float point[8];
            code = nearest_lattice_code(v, patterns, staged, lane, point);
        } else if constexpr (STAGED) {
            code = nearest_codeword<DIM>(v, staged, a.count, lane);
        } else {
            code = nearest_codeword<DIM>(v, a.codebook, a.count, lane);
        }
        if (lane == 0) a.codes[vector] = code;
    }
}

struct VectorTileArgs {
    const float *original, *feedback, *coeff, *scales, *codebook;
    float *output;
    int32_t *encoded;
    int rows, width, region_start, tile_start, tile_width, group, groups_per_row, codebook_size;
};

// A tile of up to 256 columns in a wavefront's registers: lane l holds columns 4 l .. 4 l + 3 in
// slots 0 .. 3, so a block of 4, 8 or 16 columns (which starts at a multiple of 4) occupies
// whole lanes and every slot index below is a compile-time constant.
constexpr int kPerLane = 4;

// Element d of the block at `local` (wavefront-uniform) out of such registers.
template <int DIM>
__device__ __forceinline__ float block_element(const float (&values)[kPerLane], int local, int d) {
    if constexpr (DIM == 2) {  // a pair sits in slots 0-1 or 2-3 of one lane
        const float low = lane_value(values[d], local >> 2), high = lane_value(values[2 + d], local >> 2);
        return (local & 2) ? high : low;
    } else {
        return lane_value(values[d & 3], (local >> 2) + (d >> 2));
    }
}

// Coefficient rows of the block at `local` for the lane's columns behind that block (zero elsewhere).
template <int DIM>
__device__ __forceinline__ void request_rows(float (&rows)[DIM][kPerLane], const float *coeff, int width,
                                             int tile_start, int tile_width, int local, int lane) {
#pragma unroll
    for (int d = 0; d < DIM; ++d)
#pragma unroll
        for (int s = 0; s < kPerLane; ++s) {
            const int column = kPerLane * lane + s;
            const bool later = column >= local + DIM && column < tile_width;
            rows[d][s] = later ? coeff[static_cast<size_t>(tile_start + local + d) * width + tile_start + column] : 0.0f;
        }
}

template <int DIM, bool LATTICE, bool STAGED>
__global__ void __launch_bounds__(64 * kWaveRows) round_vector_tile_kernel(const VectorTileArgs a) {
    stage_table<DIM, LATTICE, STAGED>(a.codebook, a.codebook_size);
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kWaveRows + (threadIdx.x >> 6);
    if (row >= a.rows) return;  // whole wavefronts leave; nothing below synchronises the workgroup
    const size_t row_base = static_cast<size_t>(row) * a.width;
    LanePatterns patterns;
    if constexpr (LATTICE) load_patterns(patterns, staged, lane);

    float corrections[kPerLane], weights[kPerLane], scale_at[kPerLane], restored[kPerLane];
    int codes_at[2] = {0, 0};  // one code per block, block b in lane b % 64: at most 128 blocks (pairs) in a tile
#pragma unroll
    for (int s = 0; s < kPerLane; ++s) {
        const int column = kPerLane * lane + s;
        const bool inside = column < a.tile_width;
        const size_t at = row_base + a.tile_start + (inside ? column : 0);
        corrections[s] = inside ? a.feedback[at] : 0.0f;
        weights[s] = inside ? a.original[at] : 0.0f;
        const int group = (a.tile_start + (inside ? column : 0) - a.region_start) / a.group;
        scale_at[s] = a.scales[static_cast<size_t>(row) * a.groups_per_row + group];
        restored[s] = 0.0f;
    }
    float ahead[DIM][kPerLane];
    request_rows<DIM>(ahead, a.coeff, a.width, a.tile_start, a.tile_width, 0, lane);
    for (int local = 0; local < a.tile_width; local += DIM) {
        float along[DIM][kPerLane];
#pragma unroll
        for (int d = 0; d < DIM; ++d)
#pragma unroll
            for (int s = 0; s < kPerLane; ++s) along[d][s] = ahead[d][s];
        if (local + DIM < a.tile_width)  // uniform
            request_rows<DIM>(ahead, a.coeff, a.width, a.tile_start, a.tile_width, local + DIM, lane);

        const float scale = block_element<DIM>(scale_at, local, 0);  // a block lies inside one scale group
        float weight[DIM], normalized[DIM];
#pragma unroll
        for (int d = 0; d < DIM; ++d) {
            weight[d] = block_element<DIM>(weights, local, d);
            normalized[d] = __fdiv_rn(__fadd_rn(weight[d], block_element<DIM>(corrections, local, d)), scale);
        }
        int code;
        float word[DIM];
        if constexpr (LATTICE) {
            code = nearest_lattice_code(normalized, patterns, staged, lane, word);
        } else if constexpr (STAGED) {
            code = nearest_codeword<DIM>(normalized, staged, a.codebook_size, lane);
#pragma unroll
            for (int d = 0; d < DIM; ++d) word[d] = staged[code * DIM + d];
        } else {
            code = nearest_codeword<DIM>(normalized, a.codebook, a.codebook_size, lane);
#pragma unroll
            for (int d = 0; d < DIM; ++d) word[d] = a.codebook[static_cast<size_t>(code) * DIM + d];
        }
        float deviation[DIM];
#pragma unroll
        for (int d = 0; d < DIM; ++d) {
            const float reconstruction = __fmul_rn(word[d], scale);
            deviation[d] = __fsub_rn(weight[d], reconstruction);
            if constexpr (DIM == 2) {
                const bool holds = lane == (local >> 2);
                restored[d] = holds && !(local & 2) ? reconstruction : restored[d];
                restored[2 + d] = holds && (local & 2) ? reconstruction : restored[2 + d];
            } else {
                restored[d & 3] = lane == (local >> 2) + (d >> 2) ? reconstruction : restored[d & 3];
            }
        }
        const int block = local / DIM;
        const bool keeps = lane == (block & 63);
        codes_at[0] = keeps && block < 64 ? code : codes_at[0];
        codes_at[1] = keeps && block >= 64 ? code : codes_at[1];
#pragma unroll
        for (int s = 0; s < kPerLane; ++s) {
            float pushed = __fmul_rn(deviation[0], along[0][s]);
#pragma unroll
            for (int d = 1; d < DIM; ++d) pushed = __fadd_rn(pushed, __fmul_rn(deviation[d], along[d][s]));
            corrections[s] = __fadd_rn(corrections[s], pushed);  // columns that are not later hold zeros in `along`
        }
    }
#pragma unroll
    for (int s = 0; s < kPerLane; ++s) {
        const int column = kPerLane * lane + s;
        if (column < a.tile_width) a.output[row_base + a.tile_start + column] = restored[s];
    }
    const int blocks = a.tile_width / DIM;
    int32_t *codes = a.encoded + static_cast<size_t>(row) * (a.width / DIM) + a.tile_start / DIM;
#pragma unroll
    for (int c = 0; c < 2; ++c)
        if (64 * c + lane < blocks) codes[64 * c + lane] = codes_at[c];
}

// LDS a launch needs: the pattern table, or the codebook when it is staged.
inline bool fits_in_lds(int entries, int dimension) {
    return static_cast<size_t>(entries) * dimension * sizeof(float) <= kStagedBytes;
}

}  // namespace

extern "C" int mk_vector_nearest(const float *vectors, long long count, int dimension, const float *codebook,
                                 int codebook_size, int lattice, int32_t *codes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(count >= 0 && codebook_size >= 1, MK_ERR_INVALID, "mk_vector_nearest: sizes must be positive");
    MK_REQUIRE(dimension == 2 || dimension == 4 || dimension == 8 || dimension == 16, MK_ERR_UNSUPPORTED,
               "mk_vector_nearest: codewords of 2, 4, 8 or 16 coordinates (got %d)", dimension);
    MK_REQUIRE(!lattice || (dimension == 8 && codebook_size == 65536), MK_ERR_INVALID,
               "mk_vector_nearest: the lattice search needs the 65536-point table of 8 coordinates");
    if (count == 0) return MK_OK;
    MK_REQUIRE(vectors && codebook && codes, MK_ERR_INVALID, "mk_vector_nearest: null tensor pointer");
    NearestArgs a{vectors, codebook, codes, count, codebook_size};
    long long blocks = (count + 3) / 4;
    if (blocks > 256 * 16) blocks = 256 * 16;
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    const bool staged_codebook = !lattice && fits_in_lds(codebook_size, dimension);
    const size_t lds = lattice ? kPatternFloats * sizeof(float)
                               : (staged_codebook ? static_cast<size_t>(codebook_size) * dimension * sizeof(float) : 0);
#define MK_NEAREST(DIM)                                                                                          \
    if (staged_codebook) hipLaunchKernelGGL((vector_nearest_kernel<DIM, false, true>), grid, block, lds, stream, a); \
    else hipLaunchKernelGGL((vector_nearest_kernel<DIM, false, false>), grid, block, 0, stream, a)
    if (lattice) hipLaunchKernelGGL((vector_nearest_kernel<8, true, false>), grid, block, lds, stream, a);
    else if (dimension == 2) { MK_NEAREST(2); }
    else if (dimension == 4) { MK_NEAREST(4); }
    else if (dimension == 8) { MK_NEAREST(8); }
    else { MK_NEAREST(16); }
#undef MK_NEAREST
    MK_LAUNCH_CHECK("mk_vector_nearest");
    return MK_OK;
}

extern "C" int mk_feedback_round_vector_tile(const float *original, const float *feedback, const float *coeff,
                                             const float *scales, const float *codebook, float *output,
                                             int32_t *encoded, int rows, int width, int region_start,
                                             int tile_start, int tile_width, int group, int groups_per_row,
                                             int dimension, int codebook_size, int lattice, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(original && feedback && coeff && scales && codebook && output && encoded, MK_ERR_INVALID,
               "mk_feedback_round_vector_tile: null tensor pointer");
    MK_REQUIRE(rows >= 1 && width >= 1 && group >= 1 && codebook_size >= 1, MK_ERR_INVALID,
               "mk_feedback_round_vector_tile: sizes must be positive");
    MK_REQUIRE(dimension == 2 || dimension == 4 || dimension == 8 || dimension == 16, MK_ERR_UNSUPPORTED,
               "mk_feedback_round_vector_tile: codewords of 2, 4, 8 or 16 coordinates (got %d)", dimension);
    MK_REQUIRE(tile_start >= 0 && tile_width >= 1 && tile_start + tile_width <= width && tile_start >= region_start,
               MK_ERR_INVALID, "mk_feedback_round_vector_tile: columns [%d, %d) lie outside a row of %d", tile_start,
               tile_start + tile_width, width);
    MK_REQUIRE(tile_width <= 64 * kPerLane, MK_ERR_UNSUPPORTED,
               "mk_feedback_round_vector_tile: at most %d columns per call (got %d)", 64 * kPerLane, tile_width);
    MK_REQUIRE(width % dimension == 0 && tile_start % dimension == 0 && tile_width % dimension == 0 &&
                   group % dimension == 0,
               MK_ERR_INVALID, "mk_feedback_round_vector_tile: rows, tiles and scale groups must hold whole codewords");
    MK_REQUIRE(!lattice || (dimension == 8 && codebook_size == 65536), MK_ERR_INVALID,
               "mk_feedback_round_vector_tile: the lattice search needs the 65536-point table of 8 coordinates");
    VectorTileArgs a{original, feedback, coeff, scales, codebook, output, encoded, rows, width, region_start, tile_start,
                     tile_width, group, groups_per_row, codebook_size};
    const dim3 grid(mk_cdiv(rows, kWaveRows)), block(64 * kWaveRows);
    const bool staged_codebook = !lattice && fits_in_lds(codebook_size, dimension);
    const size_t lds = lattice ? kPatternFloats * sizeof(float)
                               : (staged_codebook ? static_cast<size_t>(codebook_size) * dimension * sizeof(float) : 0);
#define MK_TILE(DIM)                                                                                                \
    if (staged_codebook) hipLaunchKernelGGL((round_vector_tile_kernel<DIM, false, true>), grid, block, lds, stream, a); \
    else hipLaunchKernelGGL((round_vector_tile_kernel<DIM, false, false>), grid, block, 0, stream, a)
    if (lattice) hipLaunchKernelGGL((round_vector_tile_kernel<8, true, false>), grid, block, lds, stream, a);
    else if (dimension == 2) { MK_TILE(2); }
    else if (dimension == 4) { MK_TILE(4); }
    else if (dimension == 8) { MK_TILE(8); }
    else { MK_TILE(16); }
#undef MK_TILE
    MK_LAUNCH_CHECK("mk_feedback_round_vector_tile");
    return MK_OK;
}
