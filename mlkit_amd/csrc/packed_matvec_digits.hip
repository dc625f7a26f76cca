// 4-bit uniform-grid packed matvec for three to eight samples of fp32 activations: integer
// dot products on the matrix cores.
//
// A chunk of 32 activations is scaled by a power of two 2^k of its own (largest magnitude into
// [2^21, 2^22)), rounded to integers X and cut into three signed bytes, X = d0 + 256 d1 + 65536 d2
// with d0, d1 in [-128, 127].  v_mfma_i32_4x4x4_16B_i8 multiplies sixteen independent 4 x 4
// blocks over four values per instruction: lane 4 b + t supplies row t of block b's left operand
// and column t of its right operand (four bytes each) and receives column t of the result.  Block
// b is "four rows of the weight x four samples over four codes of chunk b": the codes of a word
// enter as the bytes (c0, c2, c4, c6) = w & 0x0f0f0f0f and (c1, c3, c5, c7) = (w >> 4) & 0x0f0f0f0f,
// and the activations of sample t are kept as byte planes in the same order.  Six instructions
// cover eight codes for four samples, exactly; the only roundings are the one to X and those of
// the fp32 sums over the chunks, as in the v_dot8_i32_i4 kernel that takes one and two samples
// (packed_matvec_stream4.hip).  Samples 5 - 8 are a second pass over the codes (blockIdx.y): the
// planes of four samples fill the registers.
//
// Work split as in the 16-bit matrix-core kernel: a wavefront owns 512 * SLICES codes of K as
// SLICES sub-slices of sixteen chunks and walks the workgroup's rows four at a time; scales sit
// in the four lanes of a quad and reach the multiply as DPP quad broadcasts.
//
// Replaces the reference's Triton kernel `packed_matrix_vector`
// (kernels/packed_linear.py:107-173 in /root/reference/src/mlkit) for this layout.

#include "packed_matvec_impl.h"

#include <atomic>
#include <type_traits>

namespace mk_matvec {

namespace {

typedef int mk_i4 __attribute__((ext_vector_type(4)));

constexpr int kBytePlanes = 6;   // (even codes, odd codes) x three bytes; park_planes / planes_from_slice move six words per code word

// Eight fp32 activations of a chunk (this lane's quarter of it; the four lanes of a quad hold the
// chunk): plane[2 d] holds byte d of values 0, 2, 4, 6 and plane[2 d + 1] byte d of values 1, 3, 5, 7;
// their sum (of the integers X) in `total`; returns 2^-k.  Chunks of zeros keep k = 0, chunks below
// 2^-106 the largest usable k; a chunk with a value that is not finite returns NaN.
__device__ __forceinline__ float byte_planes_of_piece(mk_u32x4 first, mk_u32x4 second, uint32_t (&plane)[kBytePlanes], int &total) {
    const uint32_t bits[8] = {first.x, first.y, first.z, first.w, second.x, second.y, second.z, second.w};
    uint32_t largest = 0;   // as magnitude bits: NaN above infinity above everything finite
#pragma unroll
    for (int k = 0; k < 8; ++k) largest = max(largest, bits[k] & 0x7fffffffu);
    largest = max(largest, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(largest), 0xB1, 0xf, 0xf, true)));
    largest = max(largest, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(largest), 0x4E, 0xf, 0xf, true)));
    // biased exponent e of the largest value; the factor 2^(148 - e) has biased exponent 275 - e (at least 21)
    const int exponent = static_cast<int>(largest >> 23);
    const int wanted = 275 - exponent;
    const int biased = exponent == 0 ? 127 : (wanted > 253 ? 253 : wanted);
    const float factor = __uint_as_float(static_cast<uint32_t>(biased) << 23);
    const float inverse = __uint_as_float(exponent == 255 ? 0x7fc00000u : static_cast<uint32_t>(254 - biased) << 23);
    // x 2^k + 1.5 * 2^23 holds X + 2^22 in its low 23 bits (rounded to nearest even); adding 128 to every byte
    // makes them unsigned, and flipping each byte's top bit afterwards makes those two's complement again.
    constexpr uint32_t kBias = 0x808080u;
    uint32_t y[8];
    int sum = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        y[k] = __float_as_uint(__builtin_fmaf(__uint_as_float(bits[k]), factor, 12582912.0f)) + (kBias - 0x4B400000u);
        sum += static_cast<int>(y[k]);
    }
    total = sum - 8 * static_cast<int>(kBias);
    auto gather = [](uint32_t v0, uint32_t v1, uint32_t v2, uint32_t v3, uint32_t &d0, uint32_t &d1, uint32_t &d2) __attribute__((always_inline)) {
        const uint32_t t01 = __builtin_amdgcn_perm(v1, v0, 0x05010400u);   // v0.b0 v1.b0 v0.b1 v1.b1
        const uint32_t t23 = __builtin_amdgcn_perm(v3, v2, 0x05010400u);
        d0 = __builtin_amdgcn_perm(t23, t01, 0x05040100u) ^ 0x80808080u;
        d1 = __builtin_amdgcn_perm(t23, t01, 0x07060302u) ^ 0x80808080u;
        const uint32_t u01 = __builtin_amdgcn_perm(v1, v0, 0x0c0c0602u);   // v0.b2 v1.b2 0 0
        const uint32_t u23 = __builtin_amdgcn_perm(v3, v2, 0x0c0c0602u);
        d2 = __builtin_amdgcn_perm(u23, u01, 0x05040100u) ^ 0x80808080u;
    };
    gather(y[0], y[2], y[4], y[6], plane[0], plane[2], plane[4]);
    gather(y[1], y[3], y[5], y[7], plane[1], plane[3], plane[5]);
    return inverse;
}

static_assert(kBytePlanes == kPlaneDigits, "the byte planes travel through LDS in the slots of the 4-bit digit planes");

// WALK: a workgroup takes every gridDim.x-th tile (fewer codes in flight: the loop keeps more registers live).
template <bool HAS_ZERO, int ROWS, int SLICES, bool WIDE_SIDES, bool WALK>
__global__ void __launch_bounds__(512) digits_blocks_kernel(const Stream4Args a, const Stream4Group members) {
    using SideRaw = std::conditional_t<WIDE_SIDES, uint32_t, uint16_t>;
    constexpr uint32_t kSideBytes = WIDE_SIDES ? 4u : 2u;
    auto side_of = [&](SideRaw raw) __attribute__((always_inline)) {
        if constexpr (WIDE_SIDES) return __uint_as_float(raw);
        else return side_as_float(raw, a.scale_dtype);
    };
    constexpr int kQuads = ROWS / 4;
    constexpr int kSlices = SLICES;                 // sub-slices of sixteen chunks per wavefront
    constexpr int kSteps = kQuads * kSlices;        // code loads per lane
    constexpr int kMostAhead = !WALK || ROWS * SLICES < 64 ? 8 : (HAS_ZERO ? 3 : 6);
    constexpr int kAhead = kSteps < kMostAhead ? kSteps : kMostAhead;
    constexpr int kSums = ROWS;
    constexpr int kSliceWords = kSlices * 16 * kPlaneStrideWords;   // one sample's planes of a wavefront's codes
    __shared__ float partials[ROWS * 4 * 8];  // [row][sample][wavefront]
    extern __shared__ __attribute__((aligned(16))) uint32_t x_slices_storage[];
    uint32_t *const x_slice = x_slices_storage + (threadIdx.x >> 6) * kSliceWords;

    const TileSource source = tile_source<ROWS>(a, members, blockIdx.z);
    if (static_cast<int>(blockIdx.x) >= source.tiles) return;  // a shorter member of a group: the whole workgroup leaves
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int block = lane >> 2, t = lane & 3;
    const uint32_t row_bytes = static_cast<uint32_t>(a.width) >> 1;
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * kSideBytes;

    // Chunks past the end of a row (K is not a multiple of the wavefront's codes) read chunk 0 with
    // zeroed activations: they add nothing.
    bool in_row[kSlices];
    uint32_t code_offset[kSlices], group_offset[kSlices];
#pragma unroll
    for (int s = 0; s < kSlices; ++s) {
        const int wanted = wave * (16 * kSlices) + s * 16 + block;
        in_row[s] = wanted * kChunkCodes < a.width;
        const int chunk = in_row[s] ? wanted : 0;
        code_offset[s] = static_cast<uint32_t>(t) * row_bytes + static_cast<uint32_t>(chunk) * 16u;
        group_offset[s] = static_cast<uint32_t>(t) * scale_row_bytes +
                          ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * kSideBytes;
    }

    __syncthreads();  // aligns the workgroup's wavefronts before their first loads

    // A workgroup prepares its activations once and then takes every gridDim.x-th tile of ROWS rows.
    int tile = blockIdx.x;
    int row_base = tile * ROWS;
    const uint8_t *codes_base = source.packed + static_cast<size_t>(row_base) * row_bytes;
    SideRaw scale_raw[kSteps], zero_raw[HAS_ZERO ? kSteps : 1];
    CodeChunk<4> codes[kSteps];
    // Step `step` of a tile is rows 4 q ... 4 q + 3 at sub-slice s: its codes, and the scale (and offset) of row
    // 4 q + t there, are requested kAhead steps before they are used.
    auto request_step = [&](int step) __attribute__((always_inline)) {
        const int q = step / kSlices, s = step % kSlices;
        const size_t quad_offset = static_cast<size_t>(row_base + 4 * q) * scale_row_bytes;
        scale_raw[step] = *reinterpret_cast<const SideRaw *>(source.scales + quad_offset + group_offset[s]);
        if constexpr (HAS_ZERO) zero_raw[step] = *reinterpret_cast<const SideRaw *>(source.zeros + quad_offset + group_offset[s]);
        load_codes<4>(codes[step], codes_base + static_cast<size_t>(4 * q) * row_bytes + code_offset[s]);
    };
    auto request_tile = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int step = 0; step < kAhead; ++step) {
            request_step(step);
            __builtin_amdgcn_sched_barrier(0);  // in order
        }
    };

    // Byte planes of sample t for this lane's chunks: the wavefront reads one sample's slice coalesced, converts
    // it (every quad one chunk), parks the planes in its own LDS buffer, and the sixteen lanes of that sample pick
    // their chunks; then the next sample.  Two samples' loads are in flight at a time, and the tile's first codes
    // are requested behind the last sample's activations, before those are waited for.
    uint32_t planes[kSlices][4 * kBytePlanes];
    float unscale[kSlices], x_sum[kSlices], grid_term[kSlices];
    {
        const int sample_base = blockIdx.y * 4;
        mk_u32x4 even_pieces[kSlices][2], odd_pieces[kSlices][2];   // of samples 0 and 2, of samples 1 and 3
        auto request_sample = [&](int j, mk_u32x4 (&pieces)[kSlices][2]) __attribute__((always_inline)) {
            const int sample = sample_base + j < a.samples ? sample_base + j : a.samples - 1;
#pragma unroll
            for (int i = 0; i < kSlices; ++i) {
                pieces[i][0] = request_wide_piece(source.x, a.width, sample, wave * (512 * kSlices), i, lane, 0);
                pieces[i][1] = request_wide_piece(source.x, a.width, sample, wave * (512 * kSlices), i, lane, 1);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        auto place_sample = [&](int j, const mk_u32x4 (&pieces)[kSlices][2]) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < kSlices; ++i) {
                uint32_t plane[kBytePlanes];
                int total;
                const float inverse = byte_planes_of_piece(pieces[i][0], pieces[i][1], plane, total);
                park_planes(x_slice, i, lane, plane, inverse, total);
            }
            wave_exchange_fence();
            if (t == j) {
#pragma unroll
                for (int s = 0; s < kSlices; ++s) planes_from_slice(planes[s], unscale[s], x_sum[s], x_slice, s * 16 + block, 0xffffffffu);
            }
            wave_exchange_fence();   // the next sample's planes go to the same buffer
        };
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
    // Chunks past the end of the row and samples past the last add nothing.
    const bool sample_present = static_cast<int>(blockIdx.y) * 4 + t < a.samples;
#pragma unroll
    for (int s = 0; s < kSlices; ++s) {
        const bool kept = in_row[s] && sample_present;
        if (__builtin_amdgcn_ballot_w64(!kept) != 0) {  // uniform; rarely taken
            const uint32_t keep = kept ? 0xffffffffu : 0u;
#pragma unroll
            for (int i = 0; i < 4 * kBytePlanes; ++i) planes[s][i] &= keep;
            x_sum[s] = kept ? x_sum[s] : 0.0f;
        }
        grid_term[s] = a.grid_min * x_sum[s];
    }

    while (true) {
    float sums[kSums];
#pragma unroll
    for (int j = 0; j < kSums; ++j) sums[j] = 0.0f;

#pragma unroll
    for (int step = 0; step < kSteps; ++step) {
        const int q = step / kSlices, s = step % kSlices;
        mk_i4 low = {0, 0, 0, 0}, middle = {0, 0, 0, 0}, high = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = codes[step].w[i];
            const int even = static_cast<int>(w & 0x0f0f0f0fu), odd = static_cast<int>((w >> 4) & 0x0f0f0f0fu);
            low = __builtin_amdgcn_mfma_i32_4x4x4i8(even, static_cast<int>(planes[s][4 * 0 + i]), low, 0, 0, 0);
            middle = __builtin_amdgcn_mfma_i32_4x4x4i8(even, static_cast<int>(planes[s][4 * 2 + i]), middle, 0, 0, 0);
            high = __builtin_amdgcn_mfma_i32_4x4x4i8(even, static_cast<int>(planes[s][4 * 4 + i]), high, 0, 0, 0);
            low = __builtin_amdgcn_mfma_i32_4x4x4i8(odd, static_cast<int>(planes[s][4 * 1 + i]), low, 0, 0, 0);
            middle = __builtin_amdgcn_mfma_i32_4x4x4i8(odd, static_cast<int>(planes[s][4 * 3 + i]), middle, 0, 0, 0);
            high = __builtin_amdgcn_mfma_i32_4x4x4i8(odd, static_cast<int>(planes[s][4 * 5 + i]), high, 0, 0, 0);
        }
        if (step + kAhead < kSteps) request_step(step + kAhead);
        // Row 4 q + r of the block: scale (and offset) come from lane r of the quad.
        const float scale = side_of(scale_raw[step]);
        float zero = 0.0f;
        if constexpr (HAS_ZERO) zero = side_of(zero_raw[step]);
        auto add_row = [&](auto r) __attribute__((always_inline)) {
            constexpr int R = decltype(r)::value;
            // sum_k c_k X_k = 65536 * high + (256 * middle + low): the bracket stays below 2^24, so only the
            // last addition rounds
            const float dot = __builtin_fmaf(static_cast<float>(high[R]), 65536.0f, static_cast<float>(middle[R] * 256 + low[R]));
            float value = quad_value<R>(scale) * __builtin_fmaf(a.grid_step, dot, grid_term[s]);
            if constexpr (HAS_ZERO) value = __builtin_fmaf(quad_value<R>(zero), x_sum[s], value);
            sums[4 * q + R] = __builtin_fmaf(value, unscale[s], sums[4 * q + R]);
        };
        add_row(std::integral_constant<int, 0>{});
        add_row(std::integral_constant<int, 1>{});
        add_row(std::integral_constant<int, 2>{});
        add_row(std::integral_constant<int, 3>{});
        __builtin_amdgcn_sched_barrier(0);  // measured faster than letting steps interleave (14.3 against 15.0 us)
    }

    // Over the sixteen blocks of the wavefront (lane bits 2 - 5), then over the wavefronts.
    transposed_wave_sum<kSums, 2>(sums, lane);
    static_assert(kSums == 16 || kSums == 8 || kSums == 4, "one, two or four lanes per total");
    const bool writer = ((lane >> 2) >> (kSums == 16 ? 4 : kSums == 8 ? 3 : 2)) == 0;
    if (writer) partials[(transposed_value_of_lane<kSums>(lane >> 2) * 4 + t) * 8 + wave] = sums[0];
    __syncthreads();
    for (int index = tid; index < ROWS * 4; index += blockDim.x) {  // a workgroup may be one wavefront
        float total = partials[index * 8];
#pragma unroll
        for (int w = 1; w < 8; ++w) total += w < waves ? partials[index * 8 + w] : 0.0f;
        const int row = row_base + index / 4;
        const int sample = blockIdx.y * 4 + (index & 3);
        if (sample < a.samples) {
            if (source.bias) total += mk_load_as_float(source.bias, row, a.bias_dtype);
            static_cast<float *>(source.y)[static_cast<size_t>(sample) * source.rows + row] = total;
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

template <int ROWS, int SLICES>
int launch_sliced(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    const dim3 block(mk_cdiv(a.width, 512 * SLICES) * 64);
    // at most 8 wavefronts x 7 KB
    const size_t planes = static_cast<size_t>(block.x / 64) * SLICES * 16 * kPlaneStrideWords * sizeof(uint32_t);
    dim3 grid(tiles, mk_cdiv(a.samples, 4), members.count > 0 ? members.count : 1);
    auto launch = [&](auto walking, auto plain) -> int {
        // More tiles than the GPU holds workgroups at once: as many workgroups as it holds, each walks its share
        // of the tiles and prepares its activations once.  (Asked of the runtime once per kernel and workgroup size.)
        static std::atomic<int> resident[9];
        const int known = resident_workgroups(walking, static_cast<int>(block.x), planes, resident[block.x / 64]);
        const int passes = static_cast<int>(grid.y * grid.z);
        if (static_cast<int>(grid.x) * passes > known) {
            grid.x = known / passes > 0 ? known / passes : 1;
            hipLaunchKernelGGL(walking, grid, block, planes, stream, a, members);
        } else {
            hipLaunchKernelGGL(plain, grid, block, planes, stream, a, members);
        }
        return 0;
    };
    auto of = [&](auto has_zero, auto wide) -> int {
        constexpr bool Z = decltype(has_zero)::value, W = decltype(wide)::value;
        return launch(digits_blocks_kernel<Z, ROWS, SLICES, W, true>, digits_blocks_kernel<Z, ROWS, SLICES, W, false>);
    };
    if (a.scale_dtype == MK_F32) {
        if (a.zeros) return of(std::true_type{}, std::true_type{});
        return of(std::false_type{}, std::true_type{});
    }
    if (a.zeros) return of(std::true_type{}, std::false_type{});
    return of(std::false_type{}, std::false_type{});
}

template <int ROWS>
int launch_rows_of(const Stream4Args &a, const Stream4Group &members, int tiles, hipStream_t stream) {
    // rows of up to 4096 codes as 1024 codes per wavefront: twice the wavefronts
    if (a.width <= 4096) return launch_sliced<ROWS, 2>(a, members, tiles, stream);
    return launch_sliced<ROWS, 4>(a, members, tiles, stream);
}

}  // namespace

bool digits_accepts(const Stream4Args &a, int rows_per_tile) {
    return a.x_dtype == MK_F32 && a.samples >= 3 && a.width > 1024 && a.width <= 16384 && a.width % kChunkCodes == 0 &&
           (rows_per_tile == 16 || rows_per_tile == 4);
}

int digits_launch(const Stream4Args &a, const Stream4Group &members, int tiles, int rows_per_tile, hipStream_t stream) {
    if (tiles == 0) return 0;
    if (rows_per_tile == 16) return launch_rows_of<16>(a, members, tiles, stream);
    return launch_rows_of<4>(a, members, tiles, stream);
}

}  // namespace mk_matvec
