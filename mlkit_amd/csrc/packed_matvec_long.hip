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

constexpr int kSpans = 2;
constexpr int kComputeUnits = 256;

// One or two samples.  ROWS rows per workgroup, cdiv(K, 4096) wavefronts.
template <int MT, bool HAS_ZERO, int ROWS, int XT, bool WIDE_SIDES>
__global__ void __launch_bounds__(512) long_rows_kernel(const Stream4Args a, const Stream4Group members) {
    static_assert(ROWS * MT <= 64, "one transposed reduction per workgroup");
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
    constexpr int kAhead = ROWS < 4 ? ROWS : 4;   // rows of codes in flight: two pieces each
    constexpr int kSums = ROWS * MT;
    __shared__ float partials[64 * 8];  // [row sum][wavefront]
    extern __shared__ __attribute__((aligned(16))) uint32_t x_slices_storage[];
    uint32_t *const x_slice = x_slices_storage + (threadIdx.x >> 6) * kSliceWords;

    const TileSource source = tile_source<ROWS>(a, members, blockIdx.z);
    if (static_cast<int>(blockIdx.x) >= source.tiles) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int sample_base = blockIdx.y * MT;
    const uint32_t row_bytes = static_cast<uint32_t>(a.width) >> 1;
    const uint32_t scale_row_bytes = static_cast<uint32_t>(a.groups) * kSideBytes;
    // Lanes past the end of a row read chunk 0 with zeroed activations: they add nothing.
    bool in_row[kSpans];
    uint32_t code_offset[kSpans], group_offset[kSpans];
#pragma unroll
    for (int s = 0; s < kSpans; ++s) {
        const int wanted = (s * waves + wave) * 64 + lane;
        in_row[s] = wanted * kChunkCodes < a.width;
        const int chunk = in_row[s] ? wanted : 0;
        code_offset[s] = static_cast<uint32_t>(chunk) * 16u;
        group_offset[s] = ((static_cast<uint32_t>(chunk) * kChunkCodes) / static_cast<uint32_t>(a.group)) * kSideBytes;
    }

    __syncthreads();  // aligns the workgroup's wavefronts before their first loads

    mk_u32x4 pieces[kSpans][MT][4];
#pragma unroll
    for (int s = 0; s < kSpans; ++s)
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
    SideRaw scale_raw[ROWS][kSpans], zero_raw[HAS_ZERO ? ROWS : 1][kSpans];
    CodeChunk<4> codes[ROWS][kSpans];
    // A row's two pieces of codes and the two scales (and offsets) that go with them.
    auto request_row = [&](int r) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < kSpans; ++s) {
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

    // Each lane's two chunks of every sample, through the wavefront's own LDS buffer.
    XChunk<XT> x[kSpans][MT];
    float x_sum[kSpans][MT], grid_term[kSpans][MT];
#pragma unroll
    for (int s = 0; s < kSpans; ++s)
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

    float sums[kSums];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        float value[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) value[m] = 0.0f;
#pragma unroll
        for (int s = 0; s < kSpans; ++s) {
            float dot[MT];
            if constexpr (kSubnormalCodes) chunk_dot_subnormal<MT>(codes[r][s], x[s], dot);
            else chunk_dot_bf16<MT>(codes[r][s], x[s], dot);
            const float scale = side_of(scale_raw[r][s]);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                value[m] = __builtin_fmaf(scale, __builtin_fmaf(code_step, dot[m], grid_term[s][m]), value[m]);
                if constexpr (HAS_ZERO) value[m] = __builtin_fmaf(side_of(zero_raw[r][s]), x_sum[s][m], value[m]);
            }
        }
        if (r + kAhead < ROWS) request_row(r + kAhead);
#pragma unroll
        for (int m = 0; m < MT; ++m) sums[r * MT + m] = value[m];
        __builtin_amdgcn_sched_barrier(0);  // rows in arrival order, temporaries short-lived
    }

    // All row sums over the lanes at once, then over the wavefronts.
    transposed_wave_sum<kSums, 0, 6>(sums, lane);
    if (lane < kSums) partials[transposed_value_of_lane<kSums>(lane) * 8 + wave] = sums[0];
    __syncthreads();
    if (tid < kSums) {
        float total = partials[tid * 8];
#pragma unroll
        for (int w = 1; w < 8; ++w) total += w < waves ? partials[tid * 8 + w] : 0.0f;
        const int j = tid / MT, m = tid - j * MT;
        const int row = row_base + j;
        const int sample = sample_base + m;
        if (sample < a.samples) {
            if (source.bias) total += mk_load_as_float(source.bias, row, a.bias_dtype);
            store_output<XT>(source.y, static_cast<size_t>(sample) * source.rows + row, total);
        }
    }
}

template <int MT, int ROWS>
int launch_rows_of(const Stream4Args &a, int tiles, hipStream_t stream) {
    if (tiles == 0) return 0;
    Stream4Group none;
    none.count = 0;
    none.widest_tiles = 0;
    const dim3 grid(tiles, mk_cdiv(a.samples, MT), 1), block(mk_cdiv(a.width, 2048 * kSpans) * 64);
    const size_t slices = static_cast<size_t>(block.x / 64) * kSliceWords * sizeof(uint32_t);
    auto launch = [&](auto kernel) -> int {
        hipLaunchKernelGGL(kernel, grid, block, slices, stream, a, none);
        return 0;
    };
    auto of = [&](auto has_zero, auto wide) -> int {
        constexpr bool Z = decltype(has_zero)::value, W = decltype(wide)::value;
        if (a.x_dtype == MK_F16) return launch(long_rows_kernel<MT, Z, ROWS, MK_F16, W>);
        return launch(long_rows_kernel<MT, Z, ROWS, MK_BF16, W>);
    };
    if (a.scale_dtype == MK_F32) {
        if (a.zeros) return of(std::true_type{}, std::true_type{});
        return of(std::false_type{}, std::true_type{});
    }
    if (a.zeros) return of(std::true_type{}, std::false_type{});
    return of(std::false_type{}, std::false_type{});
}

template <int ROWS>
int launch_tiles(const Stream4Args &a, hipStream_t stream) {
    const int tiles = a.rows / ROWS;
    const int status = a.samples == 1 ? launch_rows_of<1, ROWS>(a, tiles, stream) : launch_rows_of<2, ROWS>(a, tiles, stream);
    return status ? -1 : tiles * ROWS;
}

}  // namespace

bool long_accepts(int samples, int width, int group, int bits, int x_dtype, int scale_dtype, bool uniform) {
    (void)scale_dtype;   // 16-bit and fp32 scales both
    return bits == 4 && uniform && samples <= 2 && (x_dtype == MK_F16 || x_dtype == MK_BF16) && width > 16384 && width <= 32768 &&
           width % kChunkCodes == 0 && (group % kChunkCodes == 0 || group >= width);
}

// Multiplies the leading whole tiles of rows; returns the number of rows covered.
int long_launch(const Stream4Args &a, hipStream_t stream) {
    // A workgroup reads all of x (up to 128 KB for two samples) against 8 to 16 KB of codes per row: sixteen rows per
    // workgroup while that leaves half the compute units one each, eight rows where the second round of sixteen-row
    // tiles would be at most half full, fewer rows only for small layers.
    const int wide_tiles = a.rows / 16;
    if (wide_tiles > kComputeUnits && wide_tiles <= kComputeUnits + kComputeUnits / 2) return launch_tiles<8>(a, stream);
    if (wide_tiles >= kComputeUnits / 2) return launch_tiles<16>(a, stream);
    if (a.rows / 8 >= kComputeUnits / 2) return launch_tiles<8>(a, stream);
    return launch_tiles<4>(a, stream);
}

}  // namespace mk_matvec
