// 4-bit uniform-grid packed matvec with fp16 or bf16 activations (codes as fp16 subnormals or with the exponent of
// 128 inserted, v_dot2; 4 x 4 x 4 matrix-core blocks from three samples on) or fp32 activations (planes of 4-bit
// digits against v_dot8_i32_i4) and 16-bit or fp32 scales: the decode-time kernel for INT4 layers whose rows are
// whole multiples of 32 codes (K = 32 ... 16384).
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

#include <atomic>
#include <type_traits>

namespace mk_matvec {

namespace {

// Rows per workgroup: 16 when that still gives every compute unit a workgroup, 4 for
// layers with fewer rows (more, shorter workgroups); 8 for three and more samples on short rows (stream4_launch).  Up to 8 rows of codes are in flight
// per wavefront (both values swept on the GPU together with 8 / 32 rows and 4 - 16 ahead).
constexpr int kWideRows = 16, kMidRows = 8, kNarrowRows = 4;
constexpr int kComputeUnits = 256;

template <int ROWS>
constexpr int rows_ahead_of() {
    return ROWS < 8 ? ROWS : 8;
}

// ---- the input rotation inside the kernel -------------------------------------------------
//
// A rotated layer multiplies its codes with H(x * signs) * scale, H the Walsh-Hadamard
// transform over the whole row.  With one sample the kernel has the row spread over its lanes
// anyway (lane l of wavefront w holds elements 32 (64 w + l) ... + 31), and its first codes take
// a microsecond to arrive: the transform runs in that shadow instead of in a launch of its own.
// Stages in ascending stride as everywhere: index bits 0-4 between registers, bits 5-10
// between lanes (DPP moves, swizzles and a permute through the LDS crossbar; the lane whose bit
// is set computes partner - own as one exactly rounded fma with -1), bits 11 and up between
// wavefronts through LDS.

template <int STAGE>
__device__ __forceinline__ float lane_partner(float value, int lane) {
    const int bits = __builtin_bit_cast(int, value);
    int moved;
    if constexpr (STAGE == 0) moved = __builtin_amdgcn_mov_dpp(bits, 0xB1, 0xf, 0xf, true);        // quad_perm [1,0,3,2]
    else if constexpr (STAGE == 1) moved = __builtin_amdgcn_mov_dpp(bits, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    else if constexpr (STAGE == 3) moved = __builtin_amdgcn_mov_dpp(bits, 0x128, 0xf, 0xf, true);  // row_ror:8
    else if constexpr (STAGE == 5) moved = __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, bits);
    else moved = __builtin_amdgcn_ds_swizzle(bits, 0x1F | ((1 << STAGE) << 10));  // bit mode: xor 1 << STAGE within 32 lanes
    return __builtin_bit_cast(float, moved);
}

template <int STAGE>
__device__ __forceinline__ void rotation_lane_stage(float (&v)[kChunkCodes], int lane) {
    const float sign = (lane >> STAGE) & 1 ? -1.0f : 1.0f;
#pragma unroll
    for (int k = 0; k < kChunkCodes; ++k) v[k] = __builtin_fmaf(v[k], sign, lane_partner<STAGE>(v[k], lane));
}

// x: this lane's 32 fp16 activations (elements 32 (64 wave + lane) ...), replaced by the
// rotated ones.  `exchange`: waves * 8 KB of LDS that nothing else uses until the next barrier.
// `sign`: the +-1 factors of this lane's 32 elements (all ones without a sign vector), requested
// by the caller ahead of the codes: loads return in the order of their requests, and the
// rotation is to run while the codes are still on their way.
// `log_block`: the transform spans aligned blocks of 1 << log_block elements (64 at least): the
// stages of higher index bits are left out (uniform branches).
template <int XT>
__device__ __forceinline__ void rotate_activations(XChunk<XT> &x, const float4 (&sign)[kChunkCodes / 4], float scale,
                                                   float *exchange, int wave, int waves, int lane, int log_block) {
    static_assert(XT == MK_F16 || XT == MK_BF16, "16-bit activations");
    float v[kChunkCodes];
#pragma unroll
    for (int k = 0; k < kChunkCodes; ++k) v[k] = x_element<XT>(x, k);
#pragma unroll
    for (int q = 0; q < kChunkCodes / 4; ++q) {
        v[4 * q] *= sign[q].x; v[4 * q + 1] *= sign[q].y; v[4 * q + 2] *= sign[q].z; v[4 * q + 3] *= sign[q].w;
    }
#pragma unroll
    for (int bit = 0; bit < 5; ++bit)
#pragma unroll
        for (int k = 0; k < kChunkCodes; ++k) {
            if ((k >> bit) & 1) continue;
            const float first = v[k], second = v[k | (1 << bit)];
            v[k] = first + second;
            v[k | (1 << bit)] = first - second;
        }
    rotation_lane_stage<0>(v, lane);
    if (log_block > 6) rotation_lane_stage<1>(v, lane);
    if (log_block > 7) rotation_lane_stage<2>(v, lane);
    if (log_block > 8) rotation_lane_stage<3>(v, lane);
    if (log_block > 9) rotation_lane_stage<4>(v, lane);
    if (log_block > 10) rotation_lane_stage<5>(v, lane);
    const int wave_stages = log_block > 11 ? 1 << (log_block - 11) : 1;  // wavefronts a block spans
    (void)waves;
    for (int stage = 1; stage < wave_stages; stage <<= 1) {  // uniform
        __syncthreads();  // the buffer's earlier readers are done
#pragma unroll
        for (int k = 0; k < kChunkCodes; ++k) exchange[(wave * kChunkCodes + k) * 64 + lane] = v[k];
        __syncthreads();
        const float sign = wave & stage ? -1.0f : 1.0f;
        const float *partner = exchange + ((wave ^ stage) * kChunkCodes) * 64 + lane;
#pragma unroll
        for (int k = 0; k < kChunkCodes; ++k) v[k] = __builtin_fmaf(v[k], sign, partner[k * 64]);
    }
#pragma unroll
    for (int i = 0; i < kChunkCodes / 2; ++i) {
        if constexpr (XT == MK_F16) {
            const mk_h2 pair = {static_cast<_Float16>(v[2 * i] * scale), static_cast<_Float16>(v[2 * i + 1] * scale)};
            x.r[i] = __builtin_bit_cast(uint32_t, pair);
        } else {
            x.r[i] = static_cast<uint32_t>(mk_float_to_bf16(v[2 * i] * scale)) |
                     (static_cast<uint32_t>(mk_float_to_bf16(v[2 * i + 1] * scale)) << 16);
        }
    }
}

// PARTS = 2: rows of at most 1024 codes, one wavefront per workgroup; lanes 0 - 31 take one
// row and lanes 32 - 63 the next, so that a step covers two rows instead of leaving half the
// wavefront without codes.
// ROTATE: the activations are rotated in the kernel (one sample, rows of whole 2048-code slices).
// SPLIT: the activations are fp32 and the outputs too.  Every chunk of 32 is scaled by a power of two 2^k of its
// own, rounded to integers of 22 bits and a sign and cut into six planes of signed 4-bit digits (planes_of_piece);
// v_dot8_i32_i4 multiplies them with the codes as c - 8 exactly, and a lane's sums are multiplied by 2^-k.
// WIDE_SIDES: scales and offsets are fp32.
template <int MT, bool HAS_ZERO, int ROWS, int XT, int PARTS, bool ROTATE = false, bool SPLIT = false, bool WIDE_SIDES = false>
__device__ __forceinline__ void stream4_body(const Stream4Args &a, const Stream4Group &members) {
    static_assert(ROWS * MT <= 64 && ROWS % PARTS == 0, "one transposed reduction per workgroup");
    static_assert(!ROTATE || (MT == 1 && PARTS == 1), "the fused rotation takes one sample of long rows");
    static_assert(!SPLIT || (XT == MK_F16 && !ROTATE), "fp32 activations: XT only names the unused fp16 chunk type");
    using SideRaw = std::conditional_t<WIDE_SIDES, uint32_t, uint16_t>;
    constexpr uint32_t kSideBytes = WIDE_SIDES ? 4u : 2u;
    auto side_of = [&](SideRaw raw) __attribute__((always_inline)) {
        if constexpr (WIDE_SIDES) return __uint_as_float(raw);
        else return side_as_float(raw, a.scale_dtype);
    };
    // fp16 activations: codes enter the dot products as fp16 subnormals (c * 2^-24; no exponent is inserted and the
    // activations stay unscaled, measured as fast as the exponent trick: 7.43 against 7.45 us).  The factor 2^24
    // goes into the grid's step.  bf16 has too few mantissa bits and too small subnormals for that.
    // fp32 activations (SPLIT) enter as planes of signed 4-bit digits against the codes as c - 8 (chunk_dot_planes).
    constexpr bool kSubnormalCodes = XT == MK_F16;
    const float code_step = kSubnormalCodes && !SPLIT ? a.grid_step * 16777216.0f : a.grid_step;
    const float sum_factor = SPLIT ? __builtin_fmaf(8.0f, a.grid_step, a.grid_min) : a.grid_min;
    __shared__ float partials[64 * 8];  // [row sum][wavefront]
    // One 5 KB activation buffer per wavefront, sized at launch (a workgroup of one wavefront
    // must not hold LDS for eight).
    extern __shared__ __attribute__((aligned(16))) uint32_t x_slices_storage[];
    uint32_t *const x_slice = x_slices_storage + (threadIdx.x >> 6) * (SPLIT ? kPlaneSliceWords : kSliceWords);
    constexpr int kStreamRows = ROWS / PARTS;            // steps: PARTS rows each
    constexpr int kStreamAhead = rows_ahead_of<kStreamRows>();  // (with ROTATE too: all 16 rows ahead measured slower)
    constexpr int kSums = kStreamRows * MT;
    constexpr int kRowLanes = 64 / PARTS;
    constexpr bool kSpansMeet = !SPLIT && PARTS == 1 && MT <= 2;
    // words of a wavefront's share of the dynamic LDS that precedes the handed-over terms
    const uint32_t handed_after_words = ROTATE && a.rotate_log_block > 11 ? 64u * kChunkCodes : static_cast<uint32_t>(kSliceWords);

    const TileSource source = tile_source<ROWS>(a, members, blockIdx.z);
    if (static_cast<int>(blockIdx.x) >= source.tiles) return;  // a shorter member of a group: the whole workgroup leaves
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int part = lane / kRowLanes;                   // this lane's row within a step
    const int chunk_lane = wave * 64 + (lane & (kRowLanes - 1));
    const int sample_base = blockIdx.y * MT;
    const uint32_t row_bytes = static_cast<uint32_t>(a.width) >> 1;
    // Lanes past the end of a row (K is not a multiple of 2048) read chunk 0 with zeroed
    // activations: they add nothing.
    const bool in_row = chunk_lane * kChunkCodes < a.width;
    const int chunk = in_row ? chunk_lane : 0;
    const uint32_t code_offset = static_cast<uint32_t>(part) * row_bytes + static_cast<uint32_t>(chunk) * 16u;

    // The workgroup is aligned first: a compute unit serves loads first come, first served,
    // and a wavefront that starts late would queue its small loads behind the others' codes.
    __syncthreads();

    // Activations: 32 per sample, as 16 fp16 pairs (L2 hits), requested first.
    mk_u32x4 pieces[SPLIT ? 2 * MT : MT][4];   // SPLIT: [2 m] and [2 m + 1] hold the first and second four floats of a lane's eight
    auto request_activations = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int sample = sample_base + m < a.samples ? sample_base + m : a.samples - 1;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if constexpr (SPLIT) {
                    pieces[2 * m][i] = request_wide_piece(source.x, a.width, sample, wave * 2048, i, lane, 0);
                    pieces[2 * m + 1][i] = request_wide_piece(source.x, a.width, sample, wave * 2048, i, lane, 1);
                } else {
                    pieces[m][i] = request_piece(source.x, a.width, sample, wave * 2048, i, lane);
                }
            }
        }
    };
    request_activations();
    float4 rotation_sign[ROTATE ? kChunkCodes / 4 : 1];
    if constexpr (ROTATE) {
#pragma unroll
        for (int q = 0; q < kChunkCodes / 4; ++q) {
            rotation_sign[q] = float4{1.0f, 1.0f, 1.0f, 1.0f};
            if (a.rotate_signs)  // uniform
                rotation_sign[q] = reinterpret_cast<const float4 *>(a.rotate_signs + (wave * 64 + lane) * kChunkCodes)[q];
        }
    }
    // The scale (and offset) of this lane's chunk in every row, 2 bytes each.
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * kSideBytes;
    const uint32_t group_offset = static_cast<uint32_t>(part) * scale_row_bytes +
                                  ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * kSideBytes;
    // Short rows (two per wavefront step): a workgroup takes every gridDim.x-th tile of ROWS
    // rows and prepares its activations once, during the first tile's loads; tall matrices
    // then pay for that preparation once per workgroup instead of once per tile.
    constexpr bool kStrided = PARTS == 2;
    XChunk<XT> x[SPLIT ? 1 : MT];
    uint32_t planes[SPLIT ? MT : 1][4 * kPlaneDigits];   // SPLIT: this lane's chunk of every sample as digit planes
    float x_sum[MT], grid_term[MT];
    float unscale[SPLIT ? MT : 1];   // SPLIT: 2^-k of this lane's chunk, per sample
    int tile = blockIdx.x;
    bool first_tile = true;
    do {
    const int row_base = tile * ROWS;
    const uint8_t *codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;
    const uint8_t *scale_base = source.scales + static_cast<size_t>(row_base) * scale_row_bytes;
    const uint8_t *zero_base = HAS_ZERO ? source.zeros + static_cast<size_t>(row_base) * scale_row_bytes : nullptr;
    SideRaw scale_raw[kStreamRows], zero_raw[HAS_ZERO ? kStreamRows : 1];
    CodeChunk<4> codes[kStreamRows];
    auto request_sides = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < kStreamRows; ++r) {
            scale_raw[r] = *reinterpret_cast<const SideRaw *>(scale_base + static_cast<size_t>(PARTS * r) * scale_row_bytes + group_offset);
            if constexpr (HAS_ZERO)
                zero_raw[r] = *reinterpret_cast<const SideRaw *>(zero_base + static_cast<size_t>(PARTS * r) * scale_row_bytes + group_offset);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto request_codes = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < kStreamAhead; ++r) {
            load_codes<4>(codes[r], codes_base + static_cast<size_t>(PARTS * r) * row_bytes + code_offset);
            __builtin_amdgcn_sched_barrier(0);  // in row order
        }
    };
    request_sides();
    request_codes();

    if (first_tile) {  // uniform
    // Each lane's chunk of every sample, through the wavefront's own LDS buffer (no workgroup barrier:
    // nobody else touches the buffer).
    if constexpr (SPLIT) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m > 0) wave_exchange_fence();   // the last sample's readers before this one's planes
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t plane[kPlaneDigits];
                int total;
                const float inverse = planes_of_piece(pieces[2 * m][i], pieces[2 * m + 1][i], plane, total);
                park_planes(x_slice, i, lane, plane, inverse, total);
            }
            wave_exchange_fence();
            const uint32_t keep = in_row && sample_base + m < a.samples ? 0xffffffffu : 0u;
            planes_from_slice(planes[m], unscale[m], x_sum[m], x_slice, lane & (kRowLanes - 1), keep);
            grid_term[m] = sum_factor * x_sum[m];
        }
    } else {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if (m > 0) wave_exchange_fence();   // the last sample's readers before this one's pieces
#pragma unroll
        for (int i = 0; i < 4; ++i) park_piece(x_slice, i, lane, pieces[m][i]);
        wave_exchange_fence();
        chunk_from_slice(x[m], x_slice, lane & (kRowLanes - 1));
    }
    }
    if constexpr (ROTATE)
        rotate_activations<XT>(x[0], rotation_sign, a.rotate_scale, reinterpret_cast<float *>(x_slices_storage), wave, waves, lane,
                           a.rotate_log_block);

    // sum_k (min + step c_k) x_k = step * dot + min * sum(x) - step * (code-free part of dot).
    if constexpr (!SPLIT) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const uint32_t keep = in_row && sample_base + m < a.samples ? 0xffffffffu : 0u;
#pragma unroll
        for (int i = 0; i < 16; ++i) x[m].r[i] &= keep;
        float code_free;   // what the dot products accumulate for all-zero codes (bf16: the inserted exponent of 128)
        if constexpr (kSubnormalCodes) {
            x_sum[m] = pair_for_subnormal_nibbles(x[m]);
            code_free = 0.0f;
        } else {
            x_sum[m] = pair_for_nibbles_bf16(x[m]);
            code_free = 128.0f * x_sum[m];
        }
        grid_term[m] = sum_factor * x_sum[m] - a.grid_step * code_free;
    }
    }
    }
    first_tile = false;

    float sums[kSums];
#pragma unroll
    for (int r = 0; r < kStreamRows; ++r) {
        float dot[MT];
        if constexpr (SPLIT) chunk_dot_planes<MT>(codes[r], planes, dot);
        else if constexpr (kSubnormalCodes) chunk_dot_subnormal<MT>(codes[r], x, dot);
        else chunk_dot_bf16<MT>(codes[r], x, dot);
        if (r + kStreamAhead < kStreamRows)
            load_codes<4>(codes[r + kStreamAhead],
                          codes_base + static_cast<size_t>(PARTS * (r + kStreamAhead)) * row_bytes + code_offset);
        const float scale = side_of(scale_raw[r]);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float value = scale * __builtin_fmaf(code_step, dot[m], grid_term[m]);
            if constexpr (HAS_ZERO)
                value = __builtin_fmaf(side_of(zero_raw[r]), x_sum[m], value);
            if constexpr (SPLIT) value *= unscale[m];
            sums[r * MT + m] = value;
        }
        // Keeps the rows in arrival order and their temporaries short-lived.
        __builtin_amdgcn_sched_barrier(0);
    }

    // One and two 16-bit samples of rows of six and seven wavefronts: the upper wavefronts hand their terms, lane by
    // lane, to the wavefronts `meeting` below them, which add them to their own before the lanes meet.  That is the
    // order in which the two-span kernel (a wavefront owns both spans, packed_matvec_long.hip) sums such a row, and
    // the single call, the grouped launch and the rotating kernel promise each other's results bit for bit.
    int meeting = waves;   // wavefronts whose sums reach `partials`
    if constexpr (kSpansMeet) {
        if (waves == 6 || waves == 7) {   // uniform
            meeting = (waves + 1) >> 1;
            float *const handed = reinterpret_cast<float *>(x_slices_storage + waves * handed_after_words);
            if (wave >= meeting) {
#pragma unroll
                for (int j = 0; j < kSums; ++j) handed[((wave - meeting) * kSums + j) * 64 + lane] = sums[j];
            }
            __syncthreads();
            if (wave + meeting < waves) {
#pragma unroll
                for (int j = 0; j < kSums; ++j) sums[j] += handed[(wave * kSums + j) * 64 + lane];
            }
        }
    }

    // All row sums over the lanes of a row at once, then over the wavefronts.
    if (wave < meeting) {   // uniform per wavefront
        transposed_wave_sum<kSums, 0, PARTS == 1 ? 6 : 5>(sums, lane);
        const int lane_in_row = lane & (kRowLanes - 1);
        if (lane_in_row < kSums)
            partials[(transposed_value_of_lane<kSums>(lane_in_row) * PARTS + part) * 8 + wave] = sums[0];
    }
    __syncthreads();
    if (tid < kSums * PARTS) {
        float total = partials[tid * 8];
#pragma unroll
        for (int w = 1; w < 8; ++w) total += w < meeting ? partials[tid * 8 + w] : 0.0f;
        const int value = tid / PARTS, j = value / MT, m = value - j * MT;
        const int row = row_base + PARTS * j + (tid - value * PARTS);
        const int sample = sample_base + m;
        if (sample < a.samples) {
            if (source.bias) total += mk_load_as_float(source.bias, row, a.bias_dtype);
            if constexpr (SPLIT) static_cast<float *>(source.y)[static_cast<size_t>(sample) * source.rows + row] = total;
            else store_output<XT>(source.y, static_cast<size_t>(sample) * source.rows + row, total);
        }
    }
    if constexpr (!kStrided) break;
    tile += gridDim.x;
    if (tile >= source.tiles) break;
    __syncthreads();  // `partials` is reused by the next tile
    } while (true);
}

template <int MT, bool HAS_ZERO, int ROWS, int XT, int PARTS, bool SPLIT = false, bool WIDE_SIDES = false>
__global__ void __launch_bounds__(512) stream4_kernel(const Stream4Args a, const Stream4Group members) {
    stream4_body<MT, HAS_ZERO, ROWS, XT, PARTS, false, SPLIT, WIDE_SIDES>(a, members);
}

template <bool HAS_ZERO, int ROWS, int XT>
__global__ void __launch_bounds__(512) stream4_rotating_kernel(const Stream4Args a, const Stream4Group members) {
    stream4_body<1, HAS_ZERO, ROWS, XT, 1, true>(a, members);
}

// ---- two to eight samples: the dot products on the matrix cores ---------------------------
//
// With several samples the kernel above is bound by its v_dot2 count (four per eight codes
// and sample).  v_mfma_f32_4x4x4_16B_f16 multiplies sixteen independent 4 x 4 blocks per
// instruction: lane 4 b + t supplies row t of block b's left operand and column t of its
// right operand (four fp16 each) and receives column t of the 4 x 4 result.  Block b is
// made "four rows of the weight x four samples over four codes of chunk b": lane 4 b + t
// loads the 32 codes of row t, chunk b (the same 16-byte load and nibble insertion as
// above, the two fp16 pairs of each half word being the four codes of one instruction) and
// holds the activations of sample t for chunk b.  Eight instructions cover a chunk for four
// samples; a second set of activations covers samples 4 - 7.
//
// A wavefront owns 2048 codes of K as four sub-slices of sixteen chunks and walks the
// workgroup's rows four at a time.  The result lane holds sums for four rows; their scales
// sit in the four lanes of its quad (each loaded by the lane that loads that row's codes)
// and reach the multiply as DPP quad broadcasts.

// WALK: long rows too take every gridDim.x-th tile (launched with as many workgroups as the GPU holds at once).
template <int SETS, bool HAS_ZERO, int ROWS, int XT, int SLICES, bool WALK = false>
__global__ void __launch_bounds__(512) stream4_blocks_kernel(const Stream4Args a, const Stream4Group members) {
    // Short rows (one or two sub-slices per wavefront) leave registers for the tile loop below.
    constexpr bool kStrided = SLICES <= 2;
    constexpr int kQuads = ROWS / 4;
    constexpr int kSlices = SLICES;                 // sub-slices of sixteen chunks per wavefront (rows of up to 512 / 1024 codes: 1 / 2)
    constexpr int kSteps = kQuads * kSlices;        // code loads per lane
    constexpr int kAhead = kSteps < 8 ? kSteps : 8;
    constexpr int kSums = ROWS;                     // per set and lane before the reduction
    __shared__ float partials[SETS * ROWS * 4 * 8];  // [set][row][sample in set][wavefront]
    // Four activation buffers per wavefront (one per sample of a set), sized at launch (a
    // workgroup of one wavefront must not hold LDS for eight).
    extern __shared__ __attribute__((aligned(16))) uint32_t x_slices_storage[];
    constexpr int kSampleWords = blocks_sample_words(SLICES);
    uint32_t *const x_slice = x_slices_storage + (threadIdx.x >> 6) * (4 * kSampleWords);

    const TileSource source = tile_source<ROWS>(a, members, blockIdx.z);
    if (static_cast<int>(blockIdx.x) >= source.tiles) return;  // a shorter member of a group: the whole workgroup leaves
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int block = lane >> 2, t = lane & 3;
    const uint32_t row_bytes = static_cast<uint32_t>(a.width) >> 1;
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * 2u;

    // Chunks past the end of a row (K is not a multiple of 2048) read chunk 0 with zeroed
    // activations: they add nothing.
    bool in_row[kSlices];
    uint32_t code_offset[kSlices], group_offset[kSlices];
#pragma unroll
    for (int s = 0; s < kSlices; ++s) {
        const int wanted = wave * (16 * kSlices) + s * 16 + block;
        in_row[s] = wanted * kChunkCodes < a.width;
        const int chunk = in_row[s] ? wanted : 0;
        code_offset[s] = static_cast<uint32_t>(t) * row_bytes + static_cast<uint32_t>(chunk) * 16u;
        group_offset[s] = static_cast<uint32_t>(t) * scale_row_bytes +
                          ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * 2u;
    }

    __syncthreads();  // aligns the workgroup's wavefronts before their first loads

    // Scales and the first codes of a tile (defined here, because long rows ask for them before
    // the activations are in place).
    uint16_t scale_raw[kSteps], zero_raw[HAS_ZERO ? kSteps : 1];
    CodeChunk<4> codes[kSteps];
    auto request_tile = [&](int tile) __attribute__((always_inline)) {
        const int row_base = tile * ROWS;
        const uint8_t *codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;
        const uint8_t *scale_base = source.scales + static_cast<size_t>(row_base) * scale_row_bytes;
        const uint8_t *zero_base = HAS_ZERO ? source.zeros + static_cast<size_t>(row_base) * scale_row_bytes : nullptr;
        // Scale (and offset) of row 4 q + t at every sub-slice, 2 bytes each.
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
#pragma unroll
        for (int step = 0; step < kAhead; ++step) {
            load_codes<4>(codes[step], codes_base + static_cast<size_t>(4 * (step / kSlices)) * row_bytes + code_offset[step % kSlices]);
            __builtin_amdgcn_sched_barrier(0);  // in order
        }
    };

    // Activations of sample t (and t + 4) for this lane's four chunks, 16 fp16 pairs each:
    // the wavefront reads the slices of a set's four samples coalesced, parks them side by
    // side in LDS, and every lane picks its sample's chunks.  Long rows (one tile per
    // workgroup): all activations are requested first and the tile's first codes right behind
    // them, before any activation is waited for -- eight samples are 28 KB per wavefront, and
    // the codes should stream while those arrive and are laid out.
    XChunk<XT> x[SETS][kSlices];
    {
        mk_u32x4 pieces[SETS][4][kSlices];
        auto request_set = [&](int set) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int wanted_sample = blockIdx.y * 4 * SETS + 4 * set + j;
                const int sample = wanted_sample < a.samples ? wanted_sample : a.samples - 1;
#pragma unroll
                for (int i = 0; i < kSlices; ++i)
                    pieces[set][j][i] = request_piece(source.x, a.width, sample, wave * (512 * kSlices), i, lane);
            }
        };
        auto place_set = [&](int set) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < kSlices; ++i) park_piece_swizzled(x_slice + j * kSampleWords, i, lane, pieces[set][j][i]);
            wave_exchange_fence();
#pragma unroll
            for (int s = 0; s < kSlices; ++s) chunk_from_swizzled_slice(x[set][s], x_slice + t * kSampleWords, s * 16 + block);
            wave_exchange_fence();   // the next set's pieces go to the same buffers
        };
        if constexpr (kStrided) {
#pragma unroll
            for (int set = 0; set < SETS; ++set) {
                request_set(set);
                place_set(set);
            }
        } else {
#pragma unroll
            for (int set = 0; set < SETS; ++set) request_set(set);
            __builtin_amdgcn_sched_barrier(0);
            request_tile(blockIdx.x);
#pragma unroll
            for (int set = 0; set < SETS; ++set) place_set(set);
        }
    }
    float x_sum[SETS][kSlices], grid_term[SETS][kSlices];
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
            float code_free;
            if constexpr (XT == MK_F16) {
                code_free = pair_for_nibbles(x[set][s], &x_sum[set][s]);
            } else {
                x_sum[set][s] = pair_for_nibbles_bf16(x[set][s]);
                code_free = 128.0f * x_sum[set][s];
            }
            grid_term[set][s] = a.grid_min * x_sum[set][s] - a.grid_step * code_free;
        }
    }

    // A workgroup prepares its activations once and then (short rows) takes every
    // gridDim.x-th tile of ROWS rows: tall matrices, with many more tiles than the GPU holds
    // workgroups, pay for the preparation once per workgroup instead of once per tile.
    int tile = blockIdx.x;
    do {
    const int row_base = tile * ROWS;
    const uint8_t *codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;
    if constexpr (kStrided) request_tile(tile);

    float sums[SETS][kSums];
#pragma unroll
    for (int set = 0; set < SETS; ++set)
#pragma unroll
        for (int j = 0; j < kSums; ++j) sums[set][j] = 0.0f;

    uint32_t magic = XT == MK_F16 ? 0x64006400u : 0x43004300u;
    asm volatile("" : "+v"(magic));
    auto insert = [&](uint32_t mask, uint32_t word) __attribute__((always_inline)) {
        return (word & mask) | (magic & ~mask);
    };
    // One instruction: sixteen 4 x 4 x 4 blocks, four 16-bit values per lane and operand.
    auto blocks = [](uint32_t a_low, uint32_t a_high, uint32_t b_low, uint32_t b_high, mk_f4 sum) __attribute__((always_inline)) {
        const mk_u32x2 left = {a_low, a_high}, right = {b_low, b_high};
        if constexpr (XT == MK_F16)
            return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(mk_h4, left), __builtin_bit_cast(mk_h4, right), sum, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(mk_s4, left), __builtin_bit_cast(mk_s4, right), sum, 0, 0, 0);
    };

#pragma unroll
    for (int step = 0; step < kSteps; ++step) {
        const int q = step / kSlices, s = step % kSlices;
        mk_f4 dot[SETS];
#pragma unroll
        for (int set = 0; set < SETS; ++set) dot[set] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = codes[step].w[i];
            uint32_t pair[4];  // codes (0, 4), (1, 5), (2, 6), (3, 7) as 16-bit floats
            if constexpr (XT == MK_F16) {
                const uint32_t w8 = w >> 8;
                pair[0] = insert(0x000f000fu, w), pair[1] = insert(0x00f000f0u, w);
                pair[2] = insert(0x000f000fu, w8), pair[3] = insert(0x00f000f0u, w8);
            } else {
                pair[0] = insert(0x000f000fu, w), pair[1] = insert(0x000f000fu, w >> 4);
                pair[2] = insert(0x000f000fu, w >> 8), pair[3] = insert(0x000f000fu, w >> 12);
            }
#pragma unroll
            for (int set = 0; set < SETS; ++set) {
                dot[set] = blocks(pair[0], pair[1], x[set][s].r[4 * i + 0], x[set][s].r[4 * i + 1], dot[set]);
                dot[set] = blocks(pair[2], pair[3], x[set][s].r[4 * i + 2], x[set][s].r[4 * i + 3], dot[set]);
            }
        }
        if (step + kAhead < kSteps)
            load_codes<4>(codes[step + kAhead], codes_base + static_cast<size_t>(4 * ((step + kAhead) / kSlices)) * row_bytes +
                                                    code_offset[(step + kAhead) % kSlices]);
        // Row 4 q + r of the block: scale (and offset) come from lane r of the quad.
        const float scale = side_as_float(scale_raw[step], a.scale_dtype);
        float zero = 0.0f;
        if constexpr (HAS_ZERO) zero = side_as_float(zero_raw[step], a.scale_dtype);
        auto add_row = [&](auto r) __attribute__((always_inline)) {
            constexpr int R = decltype(r)::value;
#pragma unroll
            for (int set = 0; set < SETS; ++set) {
                float total = sums[set][4 * q + R];
                total = __builtin_fmaf(quad_value<R>(scale), __builtin_fmaf(a.grid_step, dot[set][R], grid_term[set][s]), total);
                if constexpr (HAS_ZERO) total = __builtin_fmaf(quad_value<R>(zero), x_sum[set][s], total);
                sums[set][4 * q + R] = total;
            }
        };
        add_row(std::integral_constant<int, 0>{});
        add_row(std::integral_constant<int, 1>{});
        add_row(std::integral_constant<int, 2>{});
        add_row(std::integral_constant<int, 3>{});
        __builtin_amdgcn_sched_barrier(0);  // measured faster than letting steps interleave
    }

    // Over the sixteen blocks of the wavefront (lane bits 2 - 5), then over the wavefronts.
#pragma unroll
    for (int set = 0; set < SETS; ++set) {
        transposed_wave_sum<kSums, 2>(sums[set], lane);
        // With four sums per lane the last two stages leave every total in four lanes.
        static_assert(kSums == 16 || kSums == 8 || kSums == 4, "one, two or four lanes per total");
        const bool writer = ((lane >> 2) >> (kSums == 16 ? 4 : kSums == 8 ? 3 : 2)) == 0;
        if (writer)
            partials[((set * ROWS + transposed_value_of_lane<kSums>(lane >> 2)) * 4 + t) * 8 + wave] = sums[set][0];
    }
    __syncthreads();
    for (int index = tid; index < SETS * ROWS * 4; index += blockDim.x) {  // a workgroup may be one wavefront
        float total = partials[index * 8];
#pragma unroll
        for (int w = 1; w < 8; ++w) total += w < waves ? partials[index * 8 + w] : 0.0f;
        const int set = index / (ROWS * 4), row = row_base + (index / 4) % ROWS;
        const int sample = blockIdx.y * 4 * SETS + 4 * set + (index & 3);
        if (sample < a.samples) {
            if (source.bias) total += mk_load_as_float(source.bias, row, a.bias_dtype);
            store_output<XT>(source.y, static_cast<size_t>(sample) * source.rows + row, total);
        }
    }
    if constexpr (!kStrided && !WALK) break;
    tile += gridDim.x;
    if (tile >= source.tiles) break;
    __syncthreads();  // `partials` is reused by the next tile
    if constexpr (!kStrided) request_tile(tile);
    } while (true);
}

template <int SETS, int ROWS, int SLICES, bool WALK = false>
int launch_blocks_sliced(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    const dim3 block(mk_cdiv(a.width, 512 * SLICES) * 64);
    // at most 8 wavefronts x 4 samples x 4112 bytes = 129 KB of the CU's 160 KB
    const size_t slices = static_cast<size_t>(block.x / 64) * 4 * blocks_sample_words(SLICES) * sizeof(uint32_t);
    dim3 grid(tiles, mk_cdiv(a.samples, 4 * SETS), members.count > 0 ? members.count : 1);
    // More than 64 KB of dynamic LDS has to be allowed per kernel (static LDS counts against
    // the CU's 160 KB too, so only what this launch needs is asked for).
    auto launch = [&](auto kernel) -> int {
        static std::atomic<size_t> allowed{64 * 1024};
        if (slices > allowed.load(std::memory_order_relaxed)) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    static_cast<int>(slices)) != hipSuccess)
                return -1;
            allowed.store(slices, std::memory_order_relaxed);
        }
        if constexpr (SLICES <= 2 || WALK) {
            // Short rows: as many workgroups as the GPU holds at once; each walks the tiles
            // with that stride.  (Asked of the runtime once per kernel and workgroup size.)
            static std::atomic<int> resident[9];
            const int known = resident_workgroups(kernel, static_cast<int>(block.x), slices, resident[block.x / 64]);
            if (grid.x * grid.z > static_cast<unsigned>(known)) grid.x = mk_cdiv(known, static_cast<int>(grid.z));
        }
        hipLaunchKernelGGL(kernel, grid, block, slices, stream, a, members);
        return 0;
    };
    // (eight samples with offsets do not walk long rows: that variant has no registers left for the loop)
    constexpr bool kWithOffsets = !(WALK && SLICES == 4 && SETS == 2);
    if (a.zeros) {
        if constexpr (kWithOffsets) {
            if (a.x_dtype == MK_F16) return launch(stream4_blocks_kernel<SETS, true, ROWS, MK_F16, SLICES, WALK>);
            return launch(stream4_blocks_kernel<SETS, true, ROWS, MK_BF16, SLICES, WALK>);
        } else {
            return -1;
        }
    }
    if (a.x_dtype == MK_F16) return launch(stream4_blocks_kernel<SETS, false, ROWS, MK_F16, SLICES, WALK>);
    return launch(stream4_blocks_kernel<SETS, false, ROWS, MK_BF16, SLICES, WALK>);
}

// A wavefront covers 512 codes per sub-slice: short rows get fewer sub-slices, so that no
// sub-slice lies wholly past the end of the row.
template <int SETS, int ROWS>
int launch_blocks(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if (a.width <= 512) return launch_blocks_sliced<SETS, ROWS, 1>(a, members, tiles, stream);
    if (a.width <= 1024) return launch_blocks_sliced<SETS, ROWS, 2>(a, members, tiles, stream);
    // Rows of 2049 to 4096 codes as 1024 codes per wavefront (twice the wavefronts, no SIMD left idle) in the
    // tile-walking form, which prepares a workgroup's activations once for all its tiles: 6144 x 4096 at eight
    // samples 9.4 -> 7.2 us, 28672 x 4096 23.3 -> 17.5, 14336 x 4096 12.4 -> 11.8, 4096 x 4096 6.3 -> 5.8; with one
    // tile per compute unit and at most four samples it measures 4 % slower (4.8 -> 5.0 us), and so do longer rows.
    if (a.width <= 4096 && (tiles > kComputeUnits || a.samples > 4))
        return launch_blocks_sliced<SETS, ROWS, 2>(a, members, tiles, stream);
    // More tiles of eight long rows than compute units (stream4_launch chooses that height for them): walked.
    if constexpr (ROWS == kMidRows) {
        const int units = tiles * (members.count > 0 ? members.count : 1);
        if (units > kComputeUnits && !(SETS == 2 && a.zeros)) return launch_blocks_sliced<SETS, ROWS, 4, true>(a, members, tiles, stream);
    }
    return launch_blocks_sliced<SETS, ROWS, 4>(a, members, tiles, stream);
}

// LDS for the terms that the upper wavefronts of a row of six or seven hand to the lower ones (stream4_body).
size_t handed_terms_bytes(int row_waves, int sums) {
    if (row_waves != 6 && row_waves != 7) return 0;
    return static_cast<size_t>(row_waves - ((row_waves + 1) >> 1)) * sums * 64 * sizeof(float);
}

template <int MT, int ROWS, int PARTS>
int launch_tile_parts(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    dim3 grid(tiles, mk_cdiv(a.samples, MT), members.count > 0 ? members.count : 1);
    const dim3 block(mk_cdiv(a.width, 2048) * 64);
    const int row_waves = static_cast<int>(block.x / 64);
    size_t slices = static_cast<size_t>(row_waves) * (a.x_dtype == MK_F32 ? kPlaneSliceWords : kSliceWords) * sizeof(uint32_t);
    if (a.x_dtype != MK_F32 && PARTS == 1 && MT <= 2) slices += handed_terms_bytes(row_waves, (ROWS / PARTS) * MT);
    auto launch = [&](auto kernel) -> int {
        if (slices > 48 * 1024) {
            static std::atomic<bool> raised{false};
            if (!raised.load(std::memory_order_relaxed)) {
                if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        64 * 1024) != hipSuccess)
                    return -1;
                raised.store(true, std::memory_order_relaxed);
            }
        }
        if constexpr (PARTS == 2) {  // short rows: one wavefront per workgroup, which walks the tiles
            static std::atomic<int> known{0};
            const int resident = resident_workgroups(kernel, static_cast<int>(block.x), slices, known);
            if (grid.x * grid.z > static_cast<unsigned>(resident)) grid.x = mk_cdiv(resident, static_cast<int>(grid.z));
        }
        hipLaunchKernelGGL(kernel, grid, block, slices, stream, a, members);
        return 0;
    };
    const bool wide_sides = a.scale_dtype == MK_F32;
    if (a.x_dtype != MK_F32 && MT > 2) return -1;   // four samples at once only as digit planes
    if (a.x_dtype == MK_F32) {   // digit planes
        if (wide_sides) {
            if (a.zeros) return launch(stream4_kernel<MT, true, ROWS, MK_F16, PARTS, true, true>);
            return launch(stream4_kernel<MT, false, ROWS, MK_F16, PARTS, true, true>);
        }
        if (a.zeros) return launch(stream4_kernel<MT, true, ROWS, MK_F16, PARTS, true, false>);
        return launch(stream4_kernel<MT, false, ROWS, MK_F16, PARTS, true, false>);
    }
    if constexpr (MT <= 2) {
    if (wide_sides) {
        if (a.x_dtype == MK_F16) {
            if (a.zeros) return launch(stream4_kernel<MT, true, ROWS, MK_F16, PARTS, false, true>);
            return launch(stream4_kernel<MT, false, ROWS, MK_F16, PARTS, false, true>);
        }
        if (a.zeros) return launch(stream4_kernel<MT, true, ROWS, MK_BF16, PARTS, false, true>);
        return launch(stream4_kernel<MT, false, ROWS, MK_BF16, PARTS, false, true>);
    }
    if (a.x_dtype == MK_F16) {
        if (a.zeros) return launch(stream4_kernel<MT, true, ROWS, MK_F16, PARTS>);
        return launch(stream4_kernel<MT, false, ROWS, MK_F16, PARTS>);
    }
    if (a.zeros) return launch(stream4_kernel<MT, true, ROWS, MK_BF16, PARTS>);
    return launch(stream4_kernel<MT, false, ROWS, MK_BF16, PARTS>);
    }
    return -1;
}

template <int MT, int ROWS>
int launch_tile(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    // (short rows keep two samples per pass: the tile loop has no registers for four samples' planes)
    if (a.width <= 1024) return launch_tile_parts<(MT > 2 ? 2 : MT), ROWS, 2>(a, members, tiles, stream);
    return launch_tile_parts<MT, ROWS, 1>(a, members, tiles, stream);
}

// Launches `tiles` tiles of ROWS rows (of the single matrix, or of all members of a group);
// returns 0, or -1 when the runtime refused a launch attribute.
template <int ROWS>
int launch_rows(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if (tiles == 0) return 0;
    // One or two samples: v_dot2 kernel.  Three and more: matrix-core blocks (measured at
    // 4096 x 14336: 9.5 against 10.8 us for four samples, 13.3 against 17.6 us for eight).
    if (a.samples >= 3) {
        // fp32 activations: four samples' planes per lane, samples 5 - 8 in a second pass over the codes; rows of
        // more than 1024 codes as byte planes on the matrix cores, shorter ones as 4-bit planes against v_dot8
        if (a.x_dtype == MK_F32) {
            if (digits_accepts(a, ROWS)) return digits_launch(a, members, tiles, ROWS, stream);
            return launch_tile<4, ROWS>(a, members, tiles, stream);
        }
        if (a.samples <= 4) return launch_blocks<1, ROWS>(a, members, tiles, stream);
        return launch_blocks<2, ROWS>(a, members, tiles, stream);
    }
    if (a.samples == 2) return launch_tile<2, ROWS>(a, members, tiles, stream);
    return launch_tile<1, ROWS>(a, members, tiles, stream);
}

}  // namespace

bool stream4_accepts(int samples, int width, int group, int bits, int x_dtype, int scale_dtype, bool uniform) {
    // fp32 activations run as digit planes at any sample count; fp32 scales under 16-bit activations: the v_dot2
    // kernel, one or two samples
    const bool by_pairs = x_dtype != MK_F32 && scale_dtype == MK_F32;   // fp32 scales with 16-bit activations
    return bits == 4 && uniform && (!by_pairs || samples <= 2) && width % kChunkCodes == 0 && width <= 16384 &&
           (group % kChunkCodes == 0 || group >= width);
}

// Multiplies the leading whole tiles of rows; returns the number of rows covered, or -1 when
// the runtime refused a launch attribute.
int stream4_launch(const Stream4Args &a, hipStream_t stream) {
    Stream4Group none;
    none.count = 0;
    none.widest_tiles = 0;
    if (a.rows / kWideRows >= kComputeUnits) {
        // Three and more samples are bound by instruction issue.  Rows of one wavefront (at most 2048 codes) in
        // fewer than 512 tiles of sixteen rows leave SIMDs without a wavefront: tiles of eight rows fill them
        // (4096 x 2048 at eight samples: 6.2 -> 5.2 us; with two and more wavefronts per row the activation
        // preparation repeated per tile costs more than the idle SIMDs: 4096 x 4096 6.4 -> 7.0 us).
        // Three and more samples of rows over 4096 codes (one workgroup per compute unit at a time) whose second
        // round of sixteen-row tiles would be at most half full: as many workgroups as the GPU holds walk tiles of
        // eight rows on one preparation of their activations (5120 x 13824 at M = 4 / 8: 15.2 -> 12.9 / 21.6 -> 16.4 us;
        // 6144 x 8192: 9.0 -> 8.0 / 11.9 -> 10.9; a second round three quarters full, 7168 x 8192: 9.1 -> 9.3 / 12.1 ->
        // 12.8).  Eight samples with offsets keep sixteen rows: that variant of the walking kernel spills registers.
        if (a.samples >= 3 && a.x_dtype != MK_F32 && a.width > 4096 && a.rows / kWideRows > kComputeUnits &&
            a.rows / kWideRows <= kComputeUnits + kComputeUnits / 2 && !(a.zeros && a.samples > 4)) {
            const int tiles = a.rows / kMidRows;
            return launch_rows<kMidRows>(a, none, tiles, stream) ? -1 : tiles * kMidRows;
        }
        if (a.samples >= 3 && a.x_dtype != MK_F32 && a.width <= 2048 && a.rows / kWideRows < 2 * kComputeUnits) {
            const int tiles = a.rows / kMidRows;
            return launch_rows<kMidRows>(a, none, tiles, stream) ? -1 : tiles * kMidRows;
        }
        // One and two samples: with at most two sixteen-row tiles per compute unit the SIMDs hold one wavefront or
        // none; tiles of eight rows double the wavefronts in flight (8192 x 4096: 6.2 -> 5.2 us at one sample, 7.3 ->
        // 5.8 at two; 5120 x 5120: 5.8 -> 5.3, 7.4 -> 6.5; 8192 x 2048: 4.3 -> 4.0, 5.1 -> 4.4).  Measured no faster
        // or slower: exactly one tile per compute unit of rows over 2048 codes (4096 x 4096: 4.3 -> 4.4), rows of
        // four and more wavefronts in two full rounds (8192 x 8192: 7.5 -> 8.0), more than 512 tiles (12288 x 4096: 6.7 -> 6.9).
        {
            const int wide_tiles = a.rows / kWideRows, row_waves = mk_cdiv(a.width, 2048);
            // (longer rows, one workgroup per compute unit at a time: only where a last round of at most half the
            // compute units becomes a shorter one, 5120 x 13824: 10.4 -> 9.0 / 13.1 -> 11.2 us, 6144 x 8192: 6.9 -> 6.4 /
            // 8.1 -> 7.7; 7168 x 8192, whose second round is three quarters full: 7.0 -> 7.3)
            const int most_tiles = row_waves <= 3 ? 2 * kComputeUnits : kComputeUnits + kComputeUnits / 2;
            const bool few_waves = wide_tiles <= most_tiles && (row_waves == 1 || wide_tiles > kComputeUnits);
            if (a.samples <= 2 && a.x_dtype != MK_F32 && few_waves) {
                const int tiles = a.rows / kMidRows;
                return launch_rows<kMidRows>(a, none, tiles, stream) ? -1 : tiles * kMidRows;
            }
        }
        const int tiles = a.rows / kWideRows;
        return launch_rows<kWideRows>(a, none, tiles, stream) ? -1 : tiles * kWideRows;
    }
    // Fewer than 256 tiles of sixteen rows: tiles of four rows spread them over the compute units.  From three
    // samples on every tile repeats a longer preparation of the activations.  Rows over 4096 codes (one workgroup per
    // compute unit at a time): the lowest tiles that still give every tile a compute unit of its own (M = 4 / 8:
    // 1536 x 8960 8.4 / 11.9 -> 5.8 / 7.9 us with eight rows, 3072 x 8192 7.4 / 10.6 -> 5.8 / 7.7 and 2560 x 10240
    // 8.6 / 11.1 -> 7.4 / 10.2 with sixteen; 1024 x 14336 stays on four).  Shorter rows (several workgroups per
    // compute unit): eight rows on the larger layers (3584 x 3584 5.0 / 7.2 -> 4.7 / 5.8, 2048 x 4096 4.2 / 5.2 ->
    // 4.0 / 4.9; 3072 x 3072 4.25 -> 4.4 / 6.0 -> 5.3).  One and two samples are fastest on four rows throughout.
    if (a.samples >= 3 && a.x_dtype != MK_F32) {
        int rows_per_tile = kNarrowRows;
        if (a.width > 4096) rows_per_tile = a.rows / kNarrowRows <= kComputeUnits ? kNarrowRows : a.rows / kMidRows <= kComputeUnits ? kMidRows : kWideRows;
        else if (a.rows >= 2048 && (a.samples >= 5 || a.width >= 3584)) rows_per_tile = kMidRows;
        if (rows_per_tile == kWideRows) {
            const int tiles = a.rows / kWideRows;
            return launch_rows<kWideRows>(a, none, tiles, stream) ? -1 : tiles * kWideRows;
        }
        if (rows_per_tile == kMidRows) {
            const int tiles = a.rows / kMidRows;
            return launch_rows<kMidRows>(a, none, tiles, stream) ? -1 : tiles * kMidRows;
        }
    }
    const int tiles = a.rows / kNarrowRows;
    return launch_rows<kNarrowRows>(a, none, tiles, stream) ? -1 : tiles * kNarrowRows;
}

// The whole four-row tiles of rows [first_row, a.rows), which a launch of taller tiles left over (first_row is a
// multiple of four): one member of a group whose pointers start at that row.  A row's sums do not depend on its
// tile, so the single call and the grouped launch, which may tile a matrix differently, leave the same rows (the
// last rows % 4) to the word kernel.  Returns the rows covered, or -1.
int stream4_launch_remainder(const Stream4Args &a, int first_row, hipStream_t stream) {
    const int tiles = (a.rows - first_row) / kNarrowRows;
    if (tiles <= 0) return 0;
    Stream4Group one{};
    one.count = 1;
    one.widest_tiles = tiles;
    Stream4Member &member = one.member[0];
    const size_t row = static_cast<size_t>(first_row);
    const size_t side_bytes = static_cast<size_t>(a.groups) * (a.scale_dtype == MK_F32 ? 4 : 2);
    member.x = a.x;
    member.packed = a.packed + row * (static_cast<size_t>(a.width) >> 1);
    member.scales = static_cast<const uint8_t *>(a.scales) + row * side_bytes;
    member.zeros = a.zeros ? static_cast<const uint8_t *>(a.zeros) + row * side_bytes : nullptr;
    member.bias = a.bias ? static_cast<const uint8_t *>(a.bias) + row * mk_dtype_bytes(a.bias_dtype) : nullptr;
    member.y = static_cast<uint8_t *>(a.y) + row * mk_dtype_bytes(a.x_dtype);   // outputs have the activations' type
    member.rows = a.rows;
    member.tiles = tiles;
    return launch_rows<kNarrowRows>(a, one, tiles, stream) ? -1 : tiles * kNarrowRows;
}

int stream4_launch_rotating(const Stream4Args &a, hipStream_t stream) {
    const bool wide = a.rows / kWideRows >= kComputeUnits;
    const int tile_rows = wide ? kWideRows : kNarrowRows;
    // whole 2048-code slices (every lane of every wavefront holds activations), whole blocks
    const long long block_length = 1ll << a.rotate_log_block;
    const bool whole_rows = a.width % 2048 == 0 && a.width >= 2048 && a.width <= 16384 && a.rotate_log_block >= 6 &&
                            a.rotate_log_block <= 14 && a.width % block_length == 0;
    if (a.samples != 1 || (a.x_dtype != MK_F16 && a.x_dtype != MK_BF16) || !whole_rows || a.rows % tile_rows != 0 ||
        (reinterpret_cast<uintptr_t>(a.rotate_signs) & 15u) != 0)
        return -2;
    Stream4Group none;
    none.count = 0;
    none.widest_tiles = 0;
    const int waves = a.width / 2048;
    const dim3 grid(a.rows / tile_rows, 1, 1), block(waves * 64);
    // the exchange between the wavefronts of a block (8 KB each) overlays the activation buffers (5 KB each)
    const size_t lds = static_cast<size_t>(waves) * (a.rotate_log_block > 11 ? 64 * kChunkCodes * sizeof(float)
                                                                                : kSliceWords * sizeof(uint32_t)) +
                       handed_terms_bytes(waves, tile_rows);
    auto launch = [&](auto kernel) -> int {
        static std::atomic<bool> raised{false};
        if (lds > 48 * 1024 && !raised.load(std::memory_order_relaxed)) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    64 * 1024) != hipSuccess)
                return -1;
            raised.store(true, std::memory_order_relaxed);
        }
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, a, none);
        return 0;
    };
    auto of_type = [&](auto xt) -> int {
        constexpr int XT = decltype(xt)::value;
        if (wide) return a.zeros ? launch(stream4_rotating_kernel<true, kWideRows, XT>) : launch(stream4_rotating_kernel<false, kWideRows, XT>);
        return a.zeros ? launch(stream4_rotating_kernel<true, kNarrowRows, XT>) : launch(stream4_rotating_kernel<false, kNarrowRows, XT>);
    };
    if (a.x_dtype == MK_F16) return of_type(std::integral_constant<int, MK_F16>{});
    return of_type(std::integral_constant<int, MK_BF16>{});
}

int stream4_launch_group(const Stream4Args &shared, Stream4Group &group, const int *member_rows, int *rows_per_tile,
                         hipStream_t stream) {
    if (long_group_accepts(shared, group, member_rows)) return long_launch_group(shared, group, member_rows, rows_per_tile, stream);
    long long wide_tiles = 0;
    for (int i = 0; i < group.count; ++i) wide_tiles += member_rows[i] / kWideRows;
    const int rows = wide_tiles >= kComputeUnits ? kWideRows : kNarrowRows;
    int widest = 0;
    for (int i = 0; i < group.count; ++i) {
        group.member[i].rows = member_rows[i];
        group.member[i].tiles = member_rows[i] / rows;
        if (group.member[i].tiles > widest) widest = group.member[i].tiles;
    }
    group.widest_tiles = widest;
    *rows_per_tile = rows;
    Stream4Args a = shared;
    a.zeros = group.member[0].zeros;  // selects the kernel variant; the members agree on it
    if (rows == kWideRows) return launch_rows<kWideRows>(a, group, widest, stream);
    return launch_rows<kNarrowRows>(a, group, widest, stream);
}

}  // namespace mk_matvec
