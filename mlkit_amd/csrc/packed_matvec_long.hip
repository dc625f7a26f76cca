// 4-bit uniform-grid packed matvec for rows of 16416 to 32768 codes (the down projections of the
// larger decoders: K = 18944, 27648, 28672, 29568), fp16 or bf16 activations.
//
// The streaming kernels give a wavefront 2048 codes of a row and a workgroup at most eight
// wavefronts.  Here a wavefront owns two spans of 2048 codes, `waves * 2048` apart: a lane keeps
// the activations of two chunks, requests two 16-byte pieces of a row at a time (half as many
// rows ahead, the same bytes in flight) and adds both chunks' products into one sum per row.
// Arithmetic, reduction and the order of the sums inside a chunk are those of
// packed_matvec_stream4.hip; one and two samples on v_dot2, three to eight on the 4 x 4 x 4
// matrix-core blocks, four samples per pass over the codes.
//
// Replaces the reference's Triton kernel `packed_matrix_vector`
// (kernels/packed_linear.py:107-173 in /root/reference/src/mlkit) for this layout.

#include "packed_matvec_impl.h"

#include <atomic>
#include <type_traits>

namespace mk_matvec {

namespace {

constexpr int kComputeUnits = 256;

// The sums of a tile's rows over this lane's chunks of N spans of 2048 codes (span s of wavefront w of `waves` is span
// s * waves + w of the row): sums[r * MT + m] for row r and sample m, the rest of `sums` zero.
template <int N, int MT, bool HAS_ZERO, int ROWS, int XT, bool WIDE_SIDES, int SUMS>
__device__ __forceinline__ void long_rows_sums(const Stream4Args &a, const TileSource &source, uint32_t *x_slice, float (&sums)[SUMS]) {
    using SideRaw = std::conditional_t<WIDE_SIDES, uint32_t, uint16_t>;
    constexpr uint32_t kSideBytes = WIDE_SIDES ? 4u : 2u;
    auto side_of = [&](SideRaw raw) __attribute__((always_inline)) {
        if constexpr (WIDE_SIDES) return __uint_as_float(raw);
        else return side_as_float(raw, a.scale_dtype);
    };
    // fp16: the codes enter the dot products as fp16 subnormals, c * 2^-24 (the factor goes into the grid's step);
    // bf16: with the exponent of 128 inserted, taken out again through the sum of the activations.
    constexpr bool kSubnormalCodes = XT == MK_F16;
    const float code_step = kSubnormalCodes ? a.grid_step * 16777216.0f : a.grid_step;
    // rows of codes in flight, N pieces each (two spans, 4096 x 14336 at M = 1 / 2: three rows 6.7 / 7.85 us, four 6.7 / 7.7, six 6.8 / 8.25; 4096 x 11008: 6.1, 5.8, 5.9)
    constexpr int kMost = N == 2 ? 4 : 3;
    constexpr int kAhead = ROWS < kMost ? ROWS : kMost;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int waves = blockDim.x >> 6;
    const int sample_base = blockIdx.y * MT;
    const uint32_t row_bytes = static_cast<uint32_t>(a.width) >> 1;
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * kSideBytes;
    // Lanes past the end of a row read chunk 0 with zeroed activations: they add nothing.
    bool in_row[N];
    uint32_t code_offset[N], group_offset[N];
#pragma unroll
    for (int s = 0; s < N; ++s) {
        const int wanted = (s * waves + wave) * 64 + lane;
        in_row[s] = wanted * kChunkCodes < a.width;
        const int chunk = in_row[s] ? wanted : 0;
        code_offset[s] = static_cast<uint32_t>(chunk) * 16u;
        group_offset[s] = ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * kSideBytes;
    }

    mk_u32x4 pieces[N][MT][4];
#pragma unroll
    for (int s = 0; s < N; ++s)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int sample = sample_base + m < a.samples ? sample_base + m : a.samples - 1;
#pragma unroll
            for (int i = 0; i < 4; ++i) pieces[s][m][i] = request_piece(source.x, a.width, sample, (s * waves + wave) * 2048, i, lane);
        }
    __builtin_amdgcn_sched_barrier(0);

    const int row_base = blockIdx.x * ROWS;
    const uint8_t *const codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;
    const uint8_t *const scale_base = source.scales + static_cast<size_t>(row_base) * scale_row_bytes;
    const uint8_t *const zero_base = HAS_ZERO ? source.zeros + static_cast<size_t>(row_base) * scale_row_bytes : nullptr;
    SideRaw scale_raw[ROWS][N], zero_raw[HAS_ZERO ? ROWS : 1][N];
    CodeChunk<4> codes[ROWS][N];
    // A row's pieces of codes and the scales (and offsets) that go with them.
    auto request_row = [&](int r) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < N; ++s) {
            scale_raw[r][s] = *reinterpret_cast<const SideRaw *>(scale_base + static_cast<size_t>(r) * scale_row_bytes + group_offset[s]);
            if constexpr (HAS_ZERO)
                zero_raw[r][s] = *reinterpret_cast<const SideRaw *>(zero_base + static_cast<size_t>(r) * scale_row_bytes + group_offset[s]);
            load_codes<4>(codes[r][s], codes_base + static_cast<size_t>(r) * row_bytes + code_offset[s]);
        }
    };
#pragma unroll
    for (int r = 0; r < kAhead; ++r) {
        request_row(r);
        __builtin_amdgcn_sched_barrier(0);  // in row order
    }

    // Each lane's chunks of every sample, through the wavefront's own LDS buffer.
    XChunk<XT> x[N][MT];
    float x_sum[N][MT], grid_term[N][MT];
#pragma unroll
    for (int s = 0; s < N; ++s)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (s + m > 0) wave_exchange_fence();   // the last readers before these pieces
#pragma unroll
            for (int i = 0; i < 4; ++i) park_piece(x_slice, i, lane, pieces[s][m][i]);
            wave_exchange_fence();
            chunk_from_slice(x[s][m], x_slice, lane);
            const uint32_t keep = in_row[s] && sample_base + m < a.samples ? 0xffffffffu : 0u;
#pragma unroll
            for (int i = 0; i < 16; ++i) x[s][m].r[i] &= keep;
            float code_free;   // what the dot products accumulate for all-zero codes
            if constexpr (kSubnormalCodes) {
                x_sum[s][m] = pair_for_subnormal_nibbles(x[s][m]);
                code_free = 0.0f;
            } else {
                x_sum[s][m] = pair_for_nibbles_bf16(x[s][m]);
                code_free = 128.0f * x_sum[s][m];
            }
            grid_term[s][m] = a.grid_min * x_sum[s][m] - a.grid_step * code_free;
        }

    // A lane adds its spans' terms, each rounded first; then the lanes of the wavefront meet, then the wavefronts
    // in ascending order.  The streaming kernel sums rows of six and seven wavefronts in this order too (its
    // wavefront w + waves hands its terms to wavefront w), so a row's result equals that kernel's bit for bit.
#pragma unroll
    for (int j = ROWS * MT; j < SUMS; ++j) sums[j] = 0.0f;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
#pragma unroll
        for (int s = 0; s < N; ++s) {
            float dot[MT];
            if constexpr (kSubnormalCodes) chunk_dot_subnormal<MT>(codes[r][s], x[s], dot);
            else chunk_dot_bf16<MT>(codes[r][s], x[s], dot);
            const float scale = side_of(scale_raw[r][s]);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
#pragma clang fp contract(off)   // the span's term is rounded before it meets the other spans', as between wavefronts
                float value = scale * __builtin_fmaf(code_step, dot[m], grid_term[s][m]);
                if constexpr (HAS_ZERO) value = __builtin_fmaf(side_of(zero_raw[r][s]), x_sum[s][m], value);
                if (s == 0) sums[r * MT + m] = value;
                else sums[r * MT + m] += value;
            }
        }
        if (r + kAhead < ROWS) request_row(r + kAhead);
        __builtin_amdgcn_sched_barrier(0);  // rows in arrival order, temporaries short-lived
    }
}

// One or two samples.  ROWS rows per workgroup; a wavefront owns up to SPANS spans of 2048 codes, cdiv(K, 2048 SPANS)
// wavefronts.  SPANS = 3 (rows of 16416 to 24576 codes: four wavefronts, one per SIMD, where five or six wavefronts of
// two spans put two on one SIMD): a wavefront whose third span lies past the row runs the two-span body.
template <int MT, bool HAS_ZERO, int ROWS, int XT, bool WIDE_SIDES, int SPANS = 2>
__global__ void __launch_bounds__(512) long_rows_kernel(const Stream4Args a, const Stream4Group members) {
    static_assert(ROWS * MT <= 64, "one transposed reduction per workgroup");
    constexpr int kSums = ROWS * MT;              // row sums of the tile
    constexpr int kMeeting = kSums <= 4 ? 4 : kSums <= 8 ? 8 : kSums <= 16 ? 16 : kSums <= 32 ? 32 : 64;  // the reduction halves
    constexpr int kSlots = 8;                     // wavefronts of the workgroup
    __shared__ float partials[kMeeting * kSlots];  // [row sum][wavefront]
    extern __shared__ __attribute__((aligned(16))) uint32_t x_slices_storage[];
    uint32_t *const x_slice = x_slices_storage + (threadIdx.x >> 6) * kSliceWords;

    const TileSource source = tile_source<ROWS>(a, members, blockIdx.z);
    if (static_cast<int>(blockIdx.x) >= source.tiles) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;

    __syncthreads();  // aligns the workgroup's wavefronts before their first loads

    float sums[kMeeting];
    if constexpr (SPANS == 3) {
        if (((2 * waves + wave) * 2048) < a.width)   // uniform per wavefront
            long_rows_sums<3, MT, HAS_ZERO, ROWS, XT, WIDE_SIDES>(a, source, x_slice, sums);
        else
            long_rows_sums<2, MT, HAS_ZERO, ROWS, XT, WIDE_SIDES>(a, source, x_slice, sums);
    } else {
        long_rows_sums<2, MT, HAS_ZERO, ROWS, XT, WIDE_SIDES>(a, source, x_slice, sums);
    }

    // All sums over the lanes at once, then over the wavefronts in ascending order.
    transposed_wave_sum<kMeeting, 0, 6>(sums, lane);
    if (lane < kMeeting) partials[transposed_value_of_lane<kMeeting>(lane) * kSlots + wave] = sums[0];
    __syncthreads();
    if (tid < kSums) {
        float total = partials[tid * kSlots];
#pragma unroll
        for (int w = 1; w < kSlots; ++w) total += w < waves ? partials[tid * kSlots + w] : 0.0f;
        const int j = tid / MT, m = tid - j * MT;
        const int row = blockIdx.x * ROWS + j;
        const int sample = blockIdx.y * MT + m;
        if (sample < a.samples) {
            if (source.bias) total += mk_load_as_float(source.bias, row, a.bias_dtype);
            store_output<XT>(source.y, static_cast<size_t>(sample) * source.rows + row, total);
        }
    }
}

// Rows of 16416 to 24576 codes take three spans per wavefront (3584 x 18944 at M = 1 / 2: see long_launch).
inline int spans_per_wavefront(int width) { return width > 16384 && width <= 24576 ? 3 : 2; }

template <int MT, int ROWS>
int launch_rows_of(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    if (tiles == 0) return 0;
    const int spans = spans_per_wavefront(a.width);
    const dim3 grid(tiles, mk_cdiv(a.samples, MT), members.count > 0 ? members.count : 1), block(mk_cdiv(a.width, 2048 * spans) * 64);
    const size_t slices = static_cast<size_t>(block.x / 64) * kSliceWords * sizeof(uint32_t);
    auto launch = [&](auto kernel) -> int {
        hipLaunchKernelGGL(kernel, grid, block, slices, stream, a, members);
        return 0;
    };
    auto of = [&](auto has_zero, auto wide) -> int {
        constexpr bool Z = decltype(has_zero)::value, W = decltype(wide)::value;
        if (spans == 3) {
            if (a.x_dtype == MK_F16) return launch(long_rows_kernel<MT, Z, ROWS, MK_F16, W, 3>);
            return launch(long_rows_kernel<MT, Z, ROWS, MK_BF16, W, 3>);
        }
        if (a.x_dtype == MK_F16) return launch(long_rows_kernel<MT, Z, ROWS, MK_F16, W>);
        return launch(long_rows_kernel<MT, Z, ROWS, MK_BF16, W>);
    };
    if (a.scale_dtype == MK_F32) {
        if constexpr (ROWS == 4 || ROWS == 8 || ROWS == 16) {   // (the other heights are built for 16-bit scales only)
            if (a.zeros) return of(std::true_type{}, std::true_type{});
            return of(std::false_type{}, std::true_type{});
        } else {
            return -1;
        }
    }
    if (a.zeros) return of(std::true_type{}, std::false_type{});
    return of(std::false_type{}, std::false_type{});
}

// ---- three to eight samples: 4 x 4 x 4 matrix-core blocks -----------------------------------
//
// As in the streaming kernel's matrix-core variant, lane 4 b + t of a wavefront holds the codes of row t and the
// activations of sample t for chunk b of a sub-slice of sixteen chunks; here a wavefront owns 4096 adjacent codes
// of K as eight sub-slices (128 registers of activations), so one pass takes four samples and samples 5 - 8 are a
// second pass over the codes (blockIdx.y).  A sample's slice goes through the wavefront's LDS buffer by itself
// (8 KB), and with more (tile, pass) units than the GPU holds workgroups each workgroup walks its share of the
// tiles on one preparation of its activations.
template <bool HAS_ZERO, int ROWS, int XT, bool WALK>
__global__ void __launch_bounds__(512) long_blocks_kernel(const Stream4Args a, const Stream4Group members) {
    constexpr int kQuads = ROWS / 4;
    constexpr int kSlices = 8;                       // sub-slices of sixteen chunks per wavefront
    constexpr int kSteps = kQuads * kSlices;
    constexpr int kMostAhead = 4;
    constexpr int kAhead = kSteps < kMostAhead ? kSteps : kMostAhead;
    constexpr int kSums = ROWS;
    constexpr int kSampleWords = kSlices * 16 * 16;  // one sample's 4096 values of a wavefront, 16-bit
    __shared__ float partials[ROWS * 4 * 8];  // [row][sample][wavefront]
    extern __shared__ __attribute__((aligned(16))) uint32_t x_slices_storage[];
    uint32_t *const x_slice = x_slices_storage + (threadIdx.x >> 6) * kSampleWords;

    const TileSource source = tile_source<ROWS>(a, members, blockIdx.z);
    if (static_cast<int>(blockIdx.x) >= source.tiles) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int block = lane >> 2, t = lane & 3;
    const uint32_t row_bytes = static_cast<uint32_t>(a.width) >> 1;
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * 2u;

    // Sub-slice s of this lane is chunk `first_chunk + 16 s`; those past the end of the row read chunk 0 with zeroed
    // activations.  Offsets are worked out where they are used (sixteen of them would not fit beside 128 registers
    // of activations): scale groups are powers of two, or one group spans the row (`group_shift` 31).
    const int first_chunk = wave * (16 * kSlices) + block;
    const int chunks = a.width / kChunkCodes;
    const uint32_t own_row_codes = static_cast<uint32_t>(t) * row_bytes, own_row_sides = static_cast<uint32_t>(t) * scale_row_bytes;
    const int group_shift = a.group >= a.width ? 31 : 31 - __builtin_clz(static_cast<unsigned>(a.group) / kChunkCodes);
    auto in_row = [&](int s) __attribute__((always_inline)) { return first_chunk + 16 * s < chunks; };
    // (`chunk` is first_chunk behind an empty asm: the compiler must not keep every step's offsets in registers)
    auto code_offset = [&](int s, int chunk) __attribute__((always_inline)) {
        return own_row_codes + (chunk + 16 * s < chunks ? static_cast<uint32_t>(chunk + 16 * s) * 16u : 0u);
    };
    auto group_offset = [&](int s, int chunk) __attribute__((always_inline)) {
        return own_row_sides + (chunk + 16 * s < chunks ? (static_cast<uint32_t>(chunk + 16 * s) >> group_shift) * 2u : 0u);
    };

    __syncthreads();  // aligns the workgroup's wavefronts before their first loads

    int tile = blockIdx.x;
    int row_base = tile * ROWS;
    const uint8_t *codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;
    uint16_t scale_raw[kSteps], zero_raw[HAS_ZERO ? kSteps : 1];
    CodeChunk<4> codes[kSteps];
    // Step `step` of a tile is rows 4 q ... 4 q + 3 at sub-slice s: its codes, and the scale (and offset) of row
    // 4 q + t there, are requested kAhead steps before they are used.
    auto request_step = [&](int step) __attribute__((always_inline)) {
        const int q = step / kSlices, s = step % kSlices;
        int chunk = first_chunk;
        asm volatile("" : "+v"(chunk));
        const size_t quad_offset = static_cast<size_t>(row_base + 4 * q) * scale_row_bytes;
        const uint32_t sides_at = group_offset(s, chunk);
        scale_raw[step] = *reinterpret_cast<const uint16_t *>(source.scales + quad_offset + sides_at);
        if constexpr (HAS_ZERO) zero_raw[step] = *reinterpret_cast<const uint16_t *>(source.zeros + quad_offset + sides_at);
        load_codes<4>(codes[step], codes_base + static_cast<size_t>(4 * q) * row_bytes + code_offset(s, chunk));
    };
    auto request_tile = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int step = 0; step < kAhead; ++step) {
            request_step(step);
            __builtin_amdgcn_sched_barrier(0);  // in order
        }
    };

    // Activations of sample t for this lane's eight chunks: the wavefront reads one sample's slice coalesced, parks
    // it in its LDS buffer, and the sixteen lanes of that sample pick their chunks; then the next sample.
    XChunk<XT> x[kSlices];
    {
        const int sample_base = blockIdx.y * 4;
        mk_u32x4 even_pieces[kSlices], odd_pieces[kSlices];   // of samples 0 and 2, of samples 1 and 3
        auto request_sample = [&](int j, mk_u32x4 (&pieces)[kSlices]) __attribute__((always_inline)) {
            const int sample = sample_base + j < a.samples ? sample_base + j : a.samples - 1;
#pragma unroll
            for (int i = 0; i < kSlices; ++i) pieces[i] = request_piece(source.x, a.width, sample, wave * (512 * kSlices), i, lane);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto place_sample = [&](int j, const mk_u32x4 (&pieces)[kSlices]) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < kSlices; ++i) park_piece_swizzled(x_slice, i, lane, pieces[i]);
            wave_exchange_fence();
            if (t == j) {
#pragma unroll
                for (int s = 0; s < kSlices; ++s) chunk_from_swizzled_slice(x[s], x_slice, s * 16 + block);
            }
            wave_exchange_fence();   // the next sample goes to the same buffer
        };
        if constexpr (WALK) {
            // (a walking workgroup prepares once for several tiles and has no registers for loads in flight beside
            // the activations: one sample at a time, the first tile behind them)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                request_sample(j, even_pieces);
                place_sample(j, even_pieces);
            }
            request_tile();
        } else {
            request_sample(0, even_pieces);
            request_sample(1, odd_pieces);
            place_sample(0, even_pieces);
            request_sample(2, even_pieces);
            place_sample(1, odd_pieces);
            request_sample(3, odd_pieces);
            request_tile();
            place_sample(2, even_pieces);
            place_sample(3, odd_pieces);
        }
    }
    float x_sum[kSlices], grid_term[kSlices];
    {
        const bool sample_present = static_cast<int>(blockIdx.y) * 4 + t < a.samples;
#pragma unroll
        for (int s = 0; s < kSlices; ++s) {
            const bool kept = in_row(s) && sample_present;
            if (__builtin_amdgcn_ballot_w64(!kept) != 0) {  // uniform; rarely taken
                const uint32_t keep = kept ? 0xffffffffu : 0u;
#pragma unroll
                for (int i = 0; i < 16; ++i) x[s].r[i] &= keep;
            }
            float code_free;
            if constexpr (XT == MK_F16) {
                code_free = pair_for_nibbles(x[s], &x_sum[s]);
            } else {
                x_sum[s] = pair_for_nibbles_bf16(x[s]);
                code_free = 128.0f * x_sum[s];
            }
            grid_term[s] = a.grid_min * x_sum[s] - a.grid_step * code_free;
        }
    }

    while (true) {
    float sums[kSums];
#pragma unroll
    for (int j = 0; j < kSums; ++j) sums[j] = 0.0f;

    uint32_t magic = XT == MK_F16 ? 0x64006400u : 0x43004300u;
    asm volatile("" : "+v"(magic));
    auto insert = [&](uint32_t mask, uint32_t word) __attribute__((always_inline)) {
        return (word & mask) | (magic & ~mask);
    };
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
        mk_f4 dot = {0.0f, 0.0f, 0.0f, 0.0f};
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
            dot = blocks(pair[0], pair[1], x[s].r[4 * i + 0], x[s].r[4 * i + 1], dot);
            dot = blocks(pair[2], pair[3], x[s].r[4 * i + 2], x[s].r[4 * i + 3], dot);
        }
        if (step + kAhead < kSteps) request_step(step + kAhead);
        // Row 4 q + r of the block: scale (and offset) come from lane r of the quad.
        const float scale = side_as_float(scale_raw[step], a.scale_dtype);
        float zero = 0.0f;
        if constexpr (HAS_ZERO) zero = side_as_float(zero_raw[step], a.scale_dtype);
        auto add_row = [&](auto r) __attribute__((always_inline)) {
            constexpr int R = decltype(r)::value;
            float total = sums[4 * q + R];
            total = __builtin_fmaf(quad_value<R>(scale), __builtin_fmaf(a.grid_step, dot[R], grid_term[s]), total);
            if constexpr (HAS_ZERO) total = __builtin_fmaf(quad_value<R>(zero), x_sum[s], total);
            sums[4 * q + R] = total;
        };
        add_row(std::integral_constant<int, 0>{});
        add_row(std::integral_constant<int, 1>{});
        add_row(std::integral_constant<int, 2>{});
        add_row(std::integral_constant<int, 3>{});
        __builtin_amdgcn_sched_barrier(0);
    }

    // Over the sixteen blocks of the wavefront (lane bits 2 - 5), then over the wavefronts.
    transposed_wave_sum<kSums, 2>(sums, lane);
    static_assert(kSums == 16 || kSums == 8 || kSums == 4, "one, two or four lanes per total");
    const bool writer = ((lane >> 2) >> (kSums == 16 ? 4 : kSums == 8 ? 3 : 2)) == 0;
    if (writer) partials[(transposed_value_of_lane<kSums>(lane >> 2) * 4 + t) * 8 + wave] = sums[0];
    __syncthreads();
    for (int index = tid; index < ROWS * 4; index += blockDim.x) {
        float total = partials[index * 8];
#pragma unroll
        for (int w = 1; w < 8; ++w) total += w < waves ? partials[index * 8 + w] : 0.0f;
        const int row = row_base + index / 4;
        const int sample = blockIdx.y * 4 + (index & 3);
        if (sample < a.samples) {
            if (source.bias) total += mk_load_as_float(source.bias, row, a.bias_dtype);
            store_output<XT>(source.y, static_cast<size_t>(sample) * source.rows + row, total);
        }
    }
    if constexpr (!WALK) break;
    tile += gridDim.x;
    if (tile >= source.tiles) break;
    __syncthreads();  // `partials` is reused by the next tile
    row_base = tile * ROWS;
    codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;
    request_tile();
    }
}

template <int ROWS>
int launch_blocks_of(const Stream4Args &a, hipStream_t stream) {
    const int tiles = a.rows / ROWS;
    if (tiles == 0) return 0;
    Stream4Group none;
    none.count = 0;
    none.widest_tiles = 0;
    const dim3 block(mk_cdiv(a.width, 4096) * 64);
    const size_t slices = static_cast<size_t>(block.x / 64) * 8 * 16 * 16 * sizeof(uint32_t);   // 8 KB per wavefront
    dim3 grid(tiles, mk_cdiv(a.samples, 4), 1);
    auto launch = [&](auto walking, auto plain) -> int {
        // the launch asks for 64 KB of dynamic LDS at eight wavefronts: within the default limit
        static std::atomic<int> resident[9];
        const int known = resident_workgroups(walking, static_cast<int>(block.x), slices, resident[block.x / 64]);
        const int passes = static_cast<int>(grid.y);
        if (static_cast<int>(grid.x) * passes > known) {
            grid.x = known / passes > 0 ? known / passes : 1;
            hipLaunchKernelGGL(walking, grid, block, slices, stream, a, none);
        } else {
            hipLaunchKernelGGL(plain, grid, block, slices, stream, a, none);
        }
        return 0;
    };
    auto of = [&](auto has_zero) -> int {
        constexpr bool Z = decltype(has_zero)::value;
        if (a.x_dtype == MK_F16) return launch(long_blocks_kernel<Z, ROWS, MK_F16, true>, long_blocks_kernel<Z, ROWS, MK_F16, false>);
        return launch(long_blocks_kernel<Z, ROWS, MK_BF16, true>, long_blocks_kernel<Z, ROWS, MK_BF16, false>);
    };
    const int status = a.zeros ? of(std::true_type{}) : of(std::false_type{});
    return status ? -1 : tiles * ROWS;
}

// The tile height with the lowest rounds x (4 + height): a launch takes as many rounds as its tiles need on 256
// compute units, and a workgroup costs about four rows' worth of time before its first row (all of x read and
// prepared).  Tiles of 20 to 32 rows give layers of 4097 to 8192 rows one round (5120 rows: 256 tiles of 20), tiles
// of 12 and 14 rows give layers of 3072 and 3584 rows a tile per compute unit (sixteen rows: 192 and 224 tiles).
// `more`: the heights other than 4, 8 and 16 (built for 16-bit scales only).
int tile_rows_by_rounds(int rows, bool more) {
    constexpr int heights[] = {16, 8, 4, 12, 14, 20, 24, 28, 32};   // earlier wins a tie
    int best = 0, best_cost = 0;
    for (int height : heights) {
        const int tiles = rows / height;
        if (tiles == 0 || (height != 16 && height != 8 && height != 4 && !more)) continue;
        // (rows past the last whole tile take a launch of the word kernel: about eight rows' worth)
        const int cost = mk_cdiv(tiles, kComputeUnits) * (4 + height) + (rows % height ? 8 : 0);
        if (best == 0 || cost < best_cost) best = height, best_cost = cost;
    }
    return best;
}

template <int ROWS>
int launch_tiles(const Stream4Args &a, hipStream_t stream) {
    Stream4Group none;
    none.count = 0;
    none.widest_tiles = 0;
    const int tiles = a.rows / ROWS;
    const int status = a.samples == 1 ? launch_rows_of<1, ROWS>(a, none, tiles, stream) : launch_rows_of<2, ROWS>(a, none, tiles, stream);
    return status ? -1 : tiles * ROWS;
}

// Rows of at most 16384 codes, one and two samples: rows of six and seven wavefronts leave a compute unit's four
// SIMDs with unequal work (seven wavefronts: 2, 2, 2, 1); as three or four wavefronts of two spans
// every SIMD holds one, and a wavefront's fixed costs are paid once for two spans.  Results are the streaming
// kernel's bit for bit (it sums such rows in this kernel's order).  Returns the rows per tile, or 0 where the
// streaming kernel is as fast or faster.
//
// A workgroup costs about four rows' worth of time before its first row (all of x read and prepared), and a launch
// takes as many rounds as its tiles need on 256 compute units: the tile height with the lowest
// rounds x (4 + height) wins.  Measured against the streaming kernel (M = 1 / 2, us): 4096 x 14336 6.98 -> 6.76 / 7.88 ->
// 7.76 and 4096 x 11008 6.07 -> 5.82 / 7.73 -> 7.43 (sixteen rows), 2048 x 14336 5.33 -> 4.81 / 6.42 -> 5.61, 2048 x 11008
// 4.92 -> 4.30 / 6.03 -> 5.36 and 6144 x 14336 9.89 -> 9.68 / 12.4 -> 12.1 (eight), 1024 x 14336 4.08 -> 3.83 (four, one
// sample; two: 4.51 -> 4.63, not taken), 5120 x 13824 9.0 -> 7.7 / 11.5 -> 9.1 (256 tiles of twenty rows), 6144 x 14336
// 9.9 -> 9.05 / 12.1 -> 10.4 (24 rows), 8192 x 12288 10.45 -> 9.95 / 12.3 -> 11.85 (32 rows).  Not taken: fewer than 192 tiles (512 x 14336: 3.61 -> 3.61 / 4.21 -> 4.61), rows
// of five wavefronts (three wavefronts of 2, 2 and 1 spans: 2560 x 10240 5.13 -> 5.65, 1536 x 8960 4.1 -> 4.2 / 5.0 -> 5.3;
// only one sample of tall layers gained, 4096 x 10240 6.25 -> 5.9), eight wavefronts (4096 x 16384: 7.6 -> 7.7), layers
// with fp32 scales (no tiles over sixteen rows are built for them) whose second round of sixteen-row tiles is at
// most half full (5120 x 12288: 8.0 -> 8.6 with eight-row tiles).
int two_span_tile_rows(int samples, int rows, int width, bool wide_sides) {
    const int row_waves = mk_cdiv(width, 2048);
    if (samples > 2 || row_waves < 6 || row_waves > 7) return 0;
    const int best = tile_rows_by_rounds(rows, !wide_sides);
    if (best == 0 || rows / best < 192 || (best == 4 && samples == 2)) return 0;
    // a second round of sixteen-row tiles at most half full (fp32 scales, which have no taller tiles): the streaming
    // kernel's eight-row tiles are as fast
    if (best <= 16 && rows / 16 > kComputeUnits && rows / 16 <= kComputeUnits + kComputeUnits / 2) return 0;
    return best;
}

int launch_tiles_of(int height, const Stream4Args &a, hipStream_t stream) {
    switch (height) {
        case 4: return launch_tiles<4>(a, stream);
        case 8: return launch_tiles<8>(a, stream);
        case 12: return launch_tiles<12>(a, stream);
        case 14: return launch_tiles<14>(a, stream);
        case 20: return launch_tiles<20>(a, stream);
        case 24: return launch_tiles<24>(a, stream);
        case 28: return launch_tiles<28>(a, stream);
        case 32: return launch_tiles<32>(a, stream);
        default: return launch_tiles<16>(a, stream);
    }
}

}  // namespace

bool long_accepts(int samples, int rows, int width, int group, int bits, int x_dtype, int scale_dtype, bool uniform) {
    const bool whole_chunks = group % kChunkCodes == 0 || group >= width;
    if (!(bits == 4 && uniform && (x_dtype == MK_F16 || x_dtype == MK_BF16) && width % kChunkCodes == 0 && whole_chunks && width <= 32768))
        return false;
    if (width > 16384) {
        // one and two samples with 16-bit or fp32 scales, more samples with 16-bit scales (as for shorter rows)
        const bool power_of_two = (group & (group - 1)) == 0 || group >= width;   // the matrix-core kernel shifts instead of dividing
        return samples <= 2 || (scale_dtype != MK_F32 && power_of_two);
    }
    return two_span_tile_rows(samples, rows, width, scale_dtype == MK_F32) != 0;
}

// Up to eight matrices of one input width in one launch of the two-span kernel: the members' whole tiles of
// sixteen rows (`rows_per_tile` receives 16).  For one and two samples of rows of six and seven wavefronts
// when the members bring at least a tile per compute unit together; results equal the streaming
// kernel's, and the single call's, bit for bit.
bool long_group_accepts(const Stream4Args &shared, const Stream4Group &group, const int *member_rows) {
    if (!(shared.bits == 4 && shared.uniform && (shared.x_dtype == MK_F16 || shared.x_dtype == MK_BF16) && shared.samples <= 2 &&
          shared.width <= 16384))
        return false;
    const int row_waves = mk_cdiv(shared.width, 2048);
    if (!(row_waves == 6 || row_waves == 7)) return false;
    long long wide_tiles = 0;
    for (int i = 0; i < group.count; ++i) wide_tiles += member_rows[i] / 16;
    return wide_tiles >= kComputeUnits;
}

int long_launch_group(const Stream4Args &shared, Stream4Group &group, const int *member_rows, int *rows_per_tile, hipStream_t stream) {
    int widest = 0;
    for (int i = 0; i < group.count; ++i) {
        group.member[i].rows = member_rows[i];
        group.member[i].tiles = member_rows[i] / 16;
        if (group.member[i].tiles > widest) widest = group.member[i].tiles;
    }
    group.widest_tiles = widest;
    *rows_per_tile = 16;
    Stream4Args a = shared;
    a.zeros = group.member[0].zeros;  // selects the kernel variant; the members agree on it
    return a.samples == 1 ? launch_rows_of<1, 16>(a, group, widest, stream) : launch_rows_of<2, 16>(a, group, widest, stream);
}

// Multiplies the leading whole tiles of rows; returns the number of rows covered.
int long_launch(const Stream4Args &a, hipStream_t stream) {
    // A workgroup reads all of x (up to 128 KB for two samples) against 8 to 16 KB of codes per row: sixteen rows per
    // workgroup while that leaves half the compute units one each, eight rows where the second round of sixteen-row
    // tiles would be at most half full, fewer rows only for small layers.
    const int wide_tiles = a.rows / 16;
    if (a.samples >= 3) {
        // Every workgroup prepares four samples of all of x, so a launch takes that preparation plus the rows of its
        // tallest share: the lowest tiles that still give every (tile, pass) a compute unit of its own, else sixteen
        // rows, walked.
        const int passes = mk_cdiv(a.samples, 4);
        if ((a.rows / 4) * passes <= kComputeUnits) return launch_blocks_of<4>(a, stream);
        if ((a.rows / 8) * passes <= kComputeUnits) return launch_blocks_of<8>(a, stream);
        return launch_blocks_of<16>(a, stream);
    }
    if (a.width <= 16384) return launch_tiles_of(two_span_tile_rows(a.samples, a.rows, a.width, a.scale_dtype == MK_F32), a, stream);
    // (5120 x 27648 at M = 1 / 2: 15.6 -> 13.75 / 22.2 -> 16.6 us with 256 tiles of twenty rows, 8192 x 28672: 20.6 -> 20.1 /
    // 26.3 -> 23.2 with tiles of 32)
    if (a.rows >= 12 * kComputeUnits) return launch_tiles_of(tile_rows_by_rounds(a.rows, a.scale_dtype != MK_F32), a, stream);
    if (wide_tiles >= kComputeUnits / 2) return launch_tiles<16>(a, stream);
    if (a.rows / 8 >= kComputeUnits / 2) return launch_tiles<8>(a, stream);
    return launch_tiles<4>(a, stream);
}

}  // namespace mk_matvec
