// Vector grids on gfx950: nearest-codeword search (any codebook of 2-, 4-, 8- or
// 16-dimensional codewords; the structured search of the E8P lattice) and the LDL
// error-feedback tile that rounds blocks of `dimension` columns.
//
// One wavefront owns a row (or a vector): its 64 lanes share out the codebook entries -- four
// E8P magnitude patterns per lane, or every 64th codeword -- and the winner is found by a
// reduction over (cost, index) in which the lower index wins ties, which is what a search in
// ascending order with a strict comparison returns.  Costs are formed in fp32 without fused
// multiply-adds, coordinates in ascending order.
//
// In the feedback tile the corrections of the tile's columns live in the wavefront's
// registers (lane l holds columns l, l + 64, ...); a block's targets are read out of them with
// wavefront-uniform lane reads, and the coefficient rows the block will push its deviations
// along are requested before the search starts, so their latency hides behind it.
//
// Replaces, in /root/reference/src/mlkit:
//   kernels/lattice_search.py:10-70       nearest_lattice_code / nearest_lattice -> mk_vector_nearest
//   kernels/error_feedback.py:146-274     round_vector_feedback_tile / round_vector_tile
//                                                                   -> mk_feedback_round_vector_tile

#include "mk_common.h"

namespace {

constexpr int kPatterns = 256;        // E8P magnitude patterns
constexpr int kPatternsPerLane = 4;
constexpr int kMaxSlots = 4;          // tile columns per lane: tiles of up to 256 columns
constexpr int kWaveRows = 4;          // wavefronts (rows) per workgroup

// The smaller cost wins, the smaller index on equal costs; every lane receives the result.
__device__ __forceinline__ void wave_best(float &cost, int &index, int &extra) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const float other_cost = __shfl_xor(cost, offset, 64);
        const int other_index = __shfl_xor(index, offset, 64);
        const int other_extra = __shfl_xor(extra, offset, 64);
        const bool take = other_cost < cost || (other_cost == cost && other_index < index);
        cost = take ? other_cost : cost;
        index = take ? other_index : index;
        extra = take ? other_extra : extra;
    }
}

// This lane's four magnitude patterns (pattern lane + 64 j), their squared norms and parities.
struct LanePatterns {
    float value[kPatternsPerLane][8];
    float norm[kPatternsPerLane];
    int parity[kPatternsPerLane];
};

__device__ __forceinline__ void load_patterns(LanePatterns &p, const float *magnitudes, int lane) {
#pragma unroll
    for (int j = 0; j < kPatternsPerLane; ++j) {
        const float *row = magnitudes + static_cast<size_t>(lane + 64 * j) * 8;
        float norm = 0.0f, total = 0.0f;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            p.value[j][d] = row[d];
            norm = __fadd_rn(norm, __fmul_rn(row[d], row[d]));
            total += row[d];  // a sum of half-integers: exact
        }
        p.norm[j] = norm;
        p.parity[j] = static_cast<int>(total) & 1;
    }
}

// Code of the E8P point nearest to v (all lanes hold the same v and receive the same code).
__device__ __forceinline__ int nearest_lattice_code(const float (&v)[8], const LanePatterns &p, int lane) {
    float best_cost = __builtin_inff();
    int best_code = 0;
#pragma unroll
    for (int coset = 0; coset < 2; ++coset) {
        const float shift = coset == 0 ? -0.25f : 0.25f;
        float centered[8], absolute[8];
        int negatives = 0, sign_bits = 0;
        float squares = 0.0f;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            centered[d] = __fsub_rn(v[d], shift);
            absolute[d] = __builtin_fabsf(centered[d]);
            const int negative = centered[d] < 0.0f ? 1 : 0;
            negatives += negative;
            if (d < 7) sign_bits |= negative << d;
            squares = __fadd_rn(squares, __fmul_rn(centered[d], centered[d]));
        }
        const int sign_parity = negatives & 1;
        float cost = __builtin_inff();
        int pattern = 0, extra = 0;
#pragma unroll
        for (int j = 0; j < kPatternsPerLane; ++j) {
            float dots = 0.0f, cheapest = __builtin_inff();
            int axis = 0;
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                const float product = __fmul_rn(absolute[d], p.value[j][d]);
                dots = __fadd_rn(dots, product);
                if (product < cheapest) {  // the first minimum
                    cheapest = product;
                    axis = d;
                }
            }
            const int mismatch = p.parity[j] != sign_parity ? 1 : 0;
            float candidate = __fsub_rn(__fadd_rn(squares, p.norm[j]), __fmul_rn(2.0f, dots));
            candidate = __fadd_rn(candidate, __fmul_rn(__fmul_rn(4.0f, cheapest), static_cast<float>(mismatch)));
            if (candidate < cost) {  // ascending pattern index within the lane
                cost = candidate;
                pattern = lane + 64 * j;
                extra = axis | (mismatch << 3);
            }
        }
        wave_best(cost, pattern, extra);
        const int axis = extra & 7, mismatch = extra >> 3;
        const int flipped = (mismatch && axis < 7) ? (1 << axis) : 0;
        const int code = pattern * 128 + (sign_bits ^ flipped) + (coset == 0 ? 32768 : 0);
        if (cost < best_cost) {  // the -1/4 coset stays on a tie
            best_cost = cost;
            best_code = code;
        }
    }
    return best_code;
}

// Index of the nearest of `count` codewords of DIM floats (lowest index on ties).
template <int DIM>
__device__ __forceinline__ int nearest_codeword(const float (&v)[DIM], const float *codebook, int count, int lane) {
    float cost = __builtin_inff();
    int index = 0x7fffffff, unused = 0;
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
    wave_best(cost, index, unused);
    return index;
}

struct NearestArgs {
    const float *vectors;
    const float *codebook;  // [count, dim]; lattice: the 256 magnitude patterns follow
    int32_t *codes;
    long long vectors_count;
    int count;
};

template <int DIM, bool LATTICE>
__global__ void __launch_bounds__(256) vector_nearest_kernel(const NearestArgs a) {
    const int lane = threadIdx.x & 63;
    const long long wave = static_cast<long long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const long long waves = static_cast<long long>(gridDim.x) * (blockDim.x >> 6);
    LanePatterns patterns;
    if constexpr (LATTICE) load_patterns(patterns, a.codebook + static_cast<size_t>(a.count) * 8, lane);
    for (long long vector = wave; vector < a.vectors_count; vector += waves) {
        float v[DIM];
#pragma unroll
        for (int d = 0; d < DIM; ++d) v[d] = a.vectors[vector * DIM + d];
        int code;
        if constexpr (LATTICE) code = nearest_lattice_code(v, patterns, lane);
        else code = nearest_codeword<DIM>(v, a.codebook, a.count, lane);
        if (lane == 0) a.codes[vector] = code;
    }
}

struct VectorTileArgs {
    const float *original, *feedback, *coeff, *scales, *codebook;
    float *output;
    int32_t *encoded;
    int rows, width, region_start, tile_start, tile_width, group, groups_per_row, codebook_size;
};

// v_readlane with a wavefront-uniform lane index.
__device__ __forceinline__ float lane_value(float value, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, value), lane));
}

template <int DIM, bool LATTICE>
__global__ void __launch_bounds__(64 * kWaveRows) round_vector_tile_kernel(const VectorTileArgs a) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kWaveRows + (threadIdx.x >> 6);
    if (row >= a.rows) return;  // whole wavefronts leave; nothing below synchronises the workgroup
    const size_t row_base = static_cast<size_t>(row) * a.width;
    LanePatterns patterns;
    if constexpr (LATTICE) load_patterns(patterns, a.codebook + static_cast<size_t>(a.codebook_size) * 8, lane);

    float corrections[kMaxSlots];
#pragma unroll
    for (int s = 0; s < kMaxSlots; ++s) {
        const int column = 64 * s + lane;
        corrections[s] = column < a.tile_width ? a.feedback[row_base + a.tile_start + column] : 0.0f;
    }
    for (int local = 0; local < a.tile_width; local += DIM) {
        const int position = a.tile_start + local;
        // The coefficient rows of this block for the lane's later columns, requested first.
        float along[DIM][kMaxSlots];
#pragma unroll
        for (int d = 0; d < DIM; ++d)
#pragma unroll
            for (int s = 0; s < kMaxSlots; ++s) {
                const int column = 64 * s + lane;
                const bool later = column >= local + DIM && column < a.tile_width;
                along[d][s] = later ? a.coeff[static_cast<size_t>(position + d) * a.width + a.tile_start + column] : 0.0f;
            }
        const float scale = a.scales[static_cast<size_t>(row) * a.groups_per_row + (position - a.region_start) / a.group];
        float weight[DIM], normalized[DIM];
#pragma unroll
        for (int d = 0; d < DIM; ++d) {
            const int column = local + d;  // uniform
            float correction = 0.0f;
#pragma unroll
            for (int s = 0; s < kMaxSlots; ++s)
                if ((column >> 6) == s) correction = lane_value(corrections[s], column & 63);
            weight[d] = a.original[row_base + position + d];
            normalized[d] = __fdiv_rn(__fadd_rn(weight[d], correction), scale);
        }
        int code;
        if constexpr (LATTICE) code = nearest_lattice_code(normalized, patterns, lane);
        else code = nearest_codeword<DIM>(normalized, a.codebook, a.codebook_size, lane);
        float deviation[DIM];
#pragma unroll
        for (int d = 0; d < DIM; ++d) {
            const float reconstruction = __fmul_rn(a.codebook[static_cast<size_t>(code) * DIM + d], scale);
            deviation[d] = __fsub_rn(weight[d], reconstruction);
            if (lane == d) a.output[row_base + position + d] = reconstruction;
        }
        if (lane == 0) a.encoded[static_cast<size_t>(row) * (a.width / DIM) + position / DIM] = code;
#pragma unroll
        for (int s = 0; s < kMaxSlots; ++s) {
            float pushed = __fmul_rn(deviation[0], along[0][s]);
#pragma unroll
            for (int d = 1; d < DIM; ++d) pushed = __fadd_rn(pushed, __fmul_rn(deviation[d], along[d][s]));
            corrections[s] = __fadd_rn(corrections[s], pushed);  // columns that are not later hold zeros in `along`
        }
    }
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
    if (lattice) hipLaunchKernelGGL((vector_nearest_kernel<8, true>), grid, block, 0, stream, a);
    else if (dimension == 2) hipLaunchKernelGGL((vector_nearest_kernel<2, false>), grid, block, 0, stream, a);
    else if (dimension == 4) hipLaunchKernelGGL((vector_nearest_kernel<4, false>), grid, block, 0, stream, a);
    else if (dimension == 8) hipLaunchKernelGGL((vector_nearest_kernel<8, false>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((vector_nearest_kernel<16, false>), grid, block, 0, stream, a);
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
    MK_REQUIRE(tile_width <= 64 * kMaxSlots, MK_ERR_UNSUPPORTED,
               "mk_feedback_round_vector_tile: at most %d columns per call (got %d)", 64 * kMaxSlots, tile_width);
    MK_REQUIRE(width % dimension == 0 && tile_start % dimension == 0 && tile_width % dimension == 0 &&
                   group % dimension == 0,
               MK_ERR_INVALID, "mk_feedback_round_vector_tile: rows, tiles and scale groups must hold whole codewords");
    MK_REQUIRE(!lattice || (dimension == 8 && codebook_size == 65536), MK_ERR_INVALID,
               "mk_feedback_round_vector_tile: the lattice search needs the 65536-point table of 8 coordinates");
    VectorTileArgs a{original, feedback, coeff, scales, codebook, output, encoded, rows, width, region_start, tile_start,
                     tile_width, group, groups_per_row, codebook_size};
    const dim3 grid(mk_cdiv(rows, kWaveRows)), block(64 * kWaveRows);
    if (lattice) hipLaunchKernelGGL((round_vector_tile_kernel<8, true>), grid, block, 0, stream, a);
    else if (dimension == 2) hipLaunchKernelGGL((round_vector_tile_kernel<2, false>), grid, block, 0, stream, a);
    else if (dimension == 4) hipLaunchKernelGGL((round_vector_tile_kernel<4, false>), grid, block, 0, stream, a);
    else if (dimension == 8) hipLaunchKernelGGL((round_vector_tile_kernel<8, false>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((round_vector_tile_kernel<16, false>), grid, block, 0, stream, a);
    MK_LAUNCH_CHECK("mk_feedback_round_vector_tile");
    return MK_OK;
}
