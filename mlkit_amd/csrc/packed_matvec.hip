// Packed scalar-codec matrix-vector product: planning, the word-at-a-time kernel for
// layouts the chunked kernel does not take, and the C entry points.
//
// Replaces the reference's `matrix_vector` wrapper and direct launch
// (kernels/packed_linear.py:181-226, inference/packed_linear.py:181-245 in
// /root/reference/src/mlkit).

#include <cstdlib>

#include "packed_matvec_impl.h"

#define MK_DECLARE_WIDTH(n)                                                                  \
    bool mk_matvec_launch_b##n(const mk_matvec::MatvecArgs &, const mk_matvec::Plan &, int, \
                               bool, hipStream_t);
MK_DECLARE_WIDTH(2) MK_DECLARE_WIDTH(3) MK_DECLARE_WIDTH(4) MK_DECLARE_WIDTH(5)
MK_DECLARE_WIDTH(6) MK_DECLARE_WIDTH(7) MK_DECLARE_WIDTH(8)
#undef MK_DECLARE_WIDTH

namespace {

using mk_matvec::kChunkCodes;
using mk_matvec::kMaxTableEntries;
using mk_matvec::MatvecArgs;
using mk_matvec::Plan;

int next_pow2(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

// ---------------------------------------------------------------------------------
// Word-at-a-time kernel for every layout the chunked kernel does not take: one
// wavefront per row, lanes stride over packing words assembled from bytes.
// ---------------------------------------------------------------------------------
struct WordArgs {
    const void *x;
    const uint8_t *packed;
    const void *scales;
    const void *zeros;
    const float *values;
    const void *bias;
    void *y;
    int samples, rows, width, group, groups;
    int first_row;  // rows [first_row, rows) are multiplied
    int x_dtype, scale_dtype, bias_dtype;
    int bits, bytes_per_word, codes_per_word, uniform;
    float grid_min, grid_step;
};

__global__ void packed_matvec_words_kernel(const WordArgs a) {
    const int lane = threadIdx.x & 63;
    const int row = a.first_row + blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int sample_base = blockIdx.y * 8;
    if (row >= a.rows) return;
    const int row_words = a.width / a.codes_per_word;
    const uint8_t *row_ptr = a.packed + static_cast<size_t>(row) * row_words * a.bytes_per_word;
    const uint64_t mask = (1ull << a.bits) - 1ull;
    float acc[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) acc[m] = 0.0f;
    for (int word = lane; word < row_words; word += 64) {
        uint64_t bits = 0;
        for (int b = 0; b < a.bytes_per_word; ++b)
            bits |= static_cast<uint64_t>(row_ptr[static_cast<size_t>(word) * a.bytes_per_word + b]) << (8 * b);
        for (int i = 0; i < a.codes_per_word; ++i) {
            const int k = word * a.codes_per_word + i;
            const uint32_t code = static_cast<uint32_t>((bits >> (i * a.bits)) & mask);
            const size_t slot = static_cast<size_t>(row) * a.groups + k / a.group;
            float weight = a.uniform ? a.grid_min + static_cast<float>(code) * a.grid_step
                                     : a.values[code];
            weight *= mk_load_as_float(a.scales, slot, a.scale_dtype);
            if (a.zeros) weight += mk_load_as_float(a.zeros, slot, a.scale_dtype);
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                const int sample = sample_base + m;
                if (sample < a.samples)
                    acc[m] = __builtin_fmaf(
                        weight, mk_load_as_float(a.x, static_cast<size_t>(sample) * a.width + k, a.x_dtype),
                        acc[m]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        const float total = mk_segment_sum<64>(acc[m]);
        const int sample = sample_base + m;
        if (lane == 0 && sample < a.samples) {
            float result = total;
            if (a.bias) result += mk_load_as_float(a.bias, row, a.bias_dtype);
            mk_store_from_float(a.y, static_cast<size_t>(sample) * a.rows + row, a.x_dtype, result);
        }
    }
}

// Dynamic LDS of one workgroup: value table, fp32 scale (and zero) tile, per-wave row sums.
size_t lds_bytes_for(const Plan &p, int groups, bool uniform, bool has_zero) {
    (void)has_zero;
    const size_t tile_rows = static_cast<size_t>(p.rows_parallel) * p.rows_per_thread;
    size_t tile_slots = tile_rows * groups;
    if (tile_slots < 4u * p.threads) tile_slots = 4u * p.threads;  // kStaged * threads
    size_t floats = (uniform ? 0 : kMaxTableEntries) + 2 * tile_slots;
    floats += tile_rows > static_cast<size_t>(p.threads) ? tile_rows : p.threads;  // bias tile
    const int group_rows = p.sample_tile >= 8 ? 1 : (p.sample_tile == 4 ? 2 : 4);
    floats += 2 * static_cast<size_t>(group_rows) * p.sample_tile * p.threads;  // per-lane sums, two buffers
    return floats * sizeof(float);
}

// Development switches, read from the environment once per process (not per launch).
struct Tuning {
    int no_stream4, no_pairs, workgroups, rows_parallel;  // rows_parallel 0: planned
};
const Tuning &tuning() {
    static const Tuning values = [] {
        auto read = [](const char *name, int fallback) {
            const char *text = std::getenv(name);
            return text && *text ? std::atoi(text) : fallback;
        };
        return Tuning{read("MK_MATVEC_NO_STREAM4", 0), read("MK_MATVEC_NO_PAIRS", 0), read("MK_MATVEC_WORKGROUPS", 512),
                      read("MK_MATVEC_ROWS_PARALLEL", 0)};
    }();
    return values;
}

// Chooses the lane/row decomposition of the chunked kernel; returns false when the
// layer needs the word kernel (widths or groups that are not multiples of 32 codes,
// or a scale tile that does not fit in LDS).
//
// A row's chunks are spread over `seg` lanes (a power of two up to 64, or whole
// wavefronts), one chunk per lane, two when a row has more than 512 chunks.  Every
// thread owns 2U rows, so a workgroup multiplies a tile of rows_parallel * 2U adjacent
// rows; rows_parallel grows (up to 256 threads) only while the grid keeps at least two
// workgroups per compute unit.
bool plan_chunked(int samples, int rows, int width, int group, int groups, int bits, int x_dtype,
                  bool uniform, bool has_zero, Plan &p) {
    if (bits < 2 || width % kChunkCodes != 0) return false;
    if (group % kChunkCodes != 0 && group < width) return false;
    const int chunks_per_row = width / kChunkCodes;
    int c = chunks_per_row > 512 ? 2 : 1;
    if (chunks_per_row > 1024) return false;
    const int max_tile = (x_dtype == MK_F32 ? 4 : 8) / c;
    int mt = 1;
    while (mt < samples && mt < max_tile) mt <<= 1;
    const int lanes = mk_cdiv(chunks_per_row, c);
    const int seg = lanes <= 64 ? next_pow2(lanes) : 64 * mk_cdiv(lanes, 64);
    const int rows_per_thread = mk_matvec::kThreadRows;
    int rows_parallel = seg < 64 ? 64 / seg : 1;
    const int wanted_workgroups = tuning().workgroups;
    while (seg * rows_parallel * 2 <= 256 &&
           rows / (rows_parallel * 2 * rows_per_thread) >= wanted_workgroups)
        rows_parallel *= 2;
    if (tuning().rows_parallel > 0) rows_parallel = tuning().rows_parallel;
    const int threads = seg * rows_parallel;
    if (threads % 64 != 0 || threads > 512) return false;
    p.sample_tile = mt;
    p.chunks = c;
    p.seg_lanes = seg;
    p.rows_parallel = rows_parallel;
    p.threads = threads;
    p.rows_per_thread = rows_per_thread;
    p.lds_bytes = lds_bytes_for(p, groups, uniform, has_zero);
    if (p.lds_bytes > 60 * 1024) return false;
    p.grid_x = 0;
    return true;
}

// Rows [first_row, output_width) through the word-at-a-time kernel.
int launch_words(const void *x, int x_dtype, const uint8_t *packed, const void *scales, int scale_dtype,
                 const float *values, const void *zeros, const void *bias, int bias_dtype, void *y, int samples,
                 int output_width, int input_width, int group, int bits, int uniform, float grid_min,
                 float grid_step, int first_row, hipStream_t stream) {
    const int divisor = mk_gcd(bits, 8);
    WordArgs w;
    w.x = x; w.packed = packed; w.scales = scales; w.zeros = zeros; w.values = values; w.bias = bias;
    w.y = y; w.samples = samples; w.rows = output_width; w.width = input_width; w.group = group;
    w.groups = mk_cdiv(input_width, group); w.first_row = first_row;
    w.x_dtype = x_dtype; w.scale_dtype = scale_dtype; w.bias_dtype = bias_dtype;
    w.bits = bits;
    w.bytes_per_word = bits / divisor; w.codes_per_word = 8 / divisor; w.uniform = uniform;
    w.grid_min = grid_min; w.grid_step = grid_step;
    dim3 grid(mk_cdiv(output_width - first_row, 4), mk_cdiv(samples, 8));
    hipLaunchKernelGGL(packed_matvec_words_kernel, grid, dim3(256), 0, stream, w);
    MK_LAUNCH_CHECK("mk_packed_matvec");
    return MK_OK;
}

}  // namespace

extern "C" int mk_packed_layout_supported(int bits, int input_width, int group) {
    if (bits < 1 || bits > 8 || input_width < 1 || group < 1) return 0;
    const int divisor = mk_gcd(bits, 8);
    const int codes_per_word = 8 / divisor;
    if (input_width % codes_per_word || group % codes_per_word) return 0;
    const int group_words = group / codes_per_word;
    int tile_words = group_words & -group_words;
    if (tile_words > 128 / codes_per_word) tile_words = 128 / codes_per_word;
    return tile_words * codes_per_word >= 16 ? 1 : 0;
}

extern "C" int mk_packed_matvec(const void *x, int x_dtype, const uint8_t *packed, const void *scales,
                                int scale_dtype, const float *values, int n_values, const void *zeros,
                                const void *bias, int bias_dtype, void *y, int samples,
                                int output_width, int input_width, int group, int bits, int uniform,
                                float grid_min, float grid_step, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(x && packed && scales && y, MK_ERR_INVALID, "mk_packed_matvec: null tensor pointer");
    MK_REQUIRE(mk_dtype_valid(x_dtype) && mk_dtype_valid(scale_dtype), MK_ERR_INVALID,
               "mk_packed_matvec: unknown dtype code");
    MK_REQUIRE(!bias || mk_dtype_valid(bias_dtype), MK_ERR_INVALID, "mk_packed_matvec: unknown bias dtype");
    MK_REQUIRE(samples >= 1 && output_width >= 1 && input_width >= 1 && group >= 1, MK_ERR_INVALID,
               "mk_packed_matvec: sizes must be positive");
    MK_REQUIRE(bits >= 1 && bits <= 8, MK_ERR_INVALID, "mk_packed_matvec: code width must be 1..8 bits");
    MK_REQUIRE(uniform || (values && n_values >= 1 && n_values <= (1 << bits)), MK_ERR_INVALID,
               "mk_packed_matvec: a value table of at most 2^bits entries is required");
    MK_REQUIRE(mk_packed_layout_supported(bits, input_width, group), MK_ERR_UNSUPPORTED,
               "mk_packed_matvec: rows or scale groups split a packing word (bits=%d width=%d group=%d)",
               bits, input_width, group);
    const int groups = mk_cdiv(input_width, group);
    const bool aligned = (reinterpret_cast<uintptr_t>(packed) & 3u) == 0 &&
                         (reinterpret_cast<uintptr_t>(scales) & 3u) == 0 &&
                         (reinterpret_cast<uintptr_t>(zeros) & 3u) == 0 &&
                         (reinterpret_cast<uintptr_t>(bias) & 3u) == 0 &&
                         (reinterpret_cast<uintptr_t>(x) & 15u) == 0 &&
                         (static_cast<size_t>(input_width) * mk_dtype_bytes(x_dtype)) % 16 == 0;
    int done_rows = 0;  // rows [0, done_rows) are covered by a chunked kernel
    Plan plan;
    if (aligned && !tuning().no_stream4 &&
        mk_matvec::long_accepts(samples, output_width, input_width, group, bits, x_dtype, scale_dtype, uniform != 0) &&
        (reinterpret_cast<uintptr_t>(scales) & 1u) == 0) {
        mk_matvec::Stream4Args s4;
        s4.x = x; s4.packed = packed; s4.scales = scales; s4.zeros = zeros; s4.bias = bias; s4.y = y;
        s4.samples = samples; s4.rows = output_width; s4.width = input_width; s4.group = group;
        s4.groups = groups; s4.bias_dtype = bias_dtype; s4.grid_min = grid_min; s4.grid_step = grid_step;
        s4.values = values; s4.n_values = n_values; s4.uniform = uniform; s4.bits = bits;
        s4.x_dtype = x_dtype; s4.scale_dtype = scale_dtype;
        done_rows = mk_matvec::long_launch(s4, stream);
        MK_REQUIRE(done_rows >= 0, MK_ERR_HIP, "mk_packed_matvec: the runtime refused the kernel's launch");
        if (input_width <= 16384 && output_width - done_rows >= 4) {   // (the grouped launch leaves the same rows % 4 to the word kernel)
            const int more = mk_matvec::stream4_launch_remainder(s4, done_rows, stream);
            MK_REQUIRE(more >= 0, MK_ERR_HIP, "mk_packed_matvec: the runtime refused the kernel's LDS size");
            done_rows += more;
        }
        if (done_rows > 0) MK_LAUNCH_CHECK("mk_packed_matvec");
    } else if (aligned && !tuning().no_stream4 &&
               mk_matvec::stream4_accepts(samples, input_width, group, bits, x_dtype, scale_dtype, uniform != 0) &&
        (reinterpret_cast<uintptr_t>(scales) & 1u) == 0) {
        mk_matvec::Stream4Args s4;
        s4.x = x; s4.packed = packed; s4.scales = scales; s4.zeros = zeros; s4.bias = bias; s4.y = y;
        s4.samples = samples; s4.rows = output_width; s4.width = input_width; s4.group = group;
        s4.groups = groups; s4.bias_dtype = bias_dtype; s4.grid_min = grid_min; s4.grid_step = grid_step;
        s4.values = values; s4.n_values = n_values; s4.uniform = uniform; s4.bits = bits;
        s4.x_dtype = x_dtype; s4.scale_dtype = scale_dtype;
        done_rows = mk_matvec::stream4_launch(s4, stream);
        MK_REQUIRE(done_rows >= 0, MK_ERR_HIP, "mk_packed_matvec: the runtime refused the kernel's LDS size");
        if (output_width - done_rows >= 4) {
            const int more = mk_matvec::stream4_launch_remainder(s4, done_rows, stream);
            MK_REQUIRE(more >= 0, MK_ERR_HIP, "mk_packed_matvec: the runtime refused the kernel's LDS size");
            done_rows += more;
        }
        if (done_rows > 0) MK_LAUNCH_CHECK("mk_packed_matvec");
    } else if (aligned && !tuning().no_pairs &&
               mk_matvec::pairs_accepts(input_width, group, bits, x_dtype, scale_dtype) &&
               (reinterpret_cast<uintptr_t>(scales) & 1u) == 0) {
        mk_matvec::Stream4Args s4;
        s4.x = x; s4.packed = packed; s4.scales = scales; s4.zeros = zeros; s4.bias = bias; s4.y = y;
        s4.samples = samples; s4.rows = output_width; s4.width = input_width; s4.group = group;
        s4.groups = groups; s4.bias_dtype = bias_dtype; s4.grid_min = grid_min; s4.grid_step = grid_step;
        s4.values = values; s4.n_values = n_values; s4.uniform = uniform; s4.bits = bits;
        s4.x_dtype = x_dtype; s4.scale_dtype = scale_dtype;
        done_rows = mk_matvec::pairs_launch(s4, stream);
        if (done_rows > 0) MK_LAUNCH_CHECK("mk_packed_matvec");
    } else if (aligned && plan_chunked(samples, output_width, input_width, group, groups, bits, x_dtype,
                                uniform != 0, zeros != nullptr, plan)) {
        const int tile_rows = plan.rows_parallel * plan.rows_per_thread;
        const int tiles = output_width / tile_rows;
        if (tiles > 0) {
            MatvecArgs a;
            a.x = x; a.packed = packed; a.scales = scales; a.zeros = zeros; a.values = values;
            a.bias = bias; a.y = y;
            a.scale_row_offset = 0;
            a.samples = samples; a.rows = output_width; a.width = input_width; a.group = group;
            a.groups = groups; a.n_values = n_values; a.scale_dtype = scale_dtype; a.bias_dtype = bias_dtype;
            a.seg_lanes = plan.seg_lanes; a.rows_parallel = plan.rows_parallel;
            a.chunks_per_row = input_width / kChunkCodes;
            a.grid_min = grid_min; a.grid_step = grid_step;
            plan.grid_x = tiles;
            bool launched = false;
            switch (bits) {
                case 2: launched = mk_matvec_launch_b2(a, plan, x_dtype, uniform != 0, stream); break;
                case 3: launched = mk_matvec_launch_b3(a, plan, x_dtype, uniform != 0, stream); break;
                case 4: launched = mk_matvec_launch_b4(a, plan, x_dtype, uniform != 0, stream); break;
                case 5: launched = mk_matvec_launch_b5(a, plan, x_dtype, uniform != 0, stream); break;
                case 6: launched = mk_matvec_launch_b6(a, plan, x_dtype, uniform != 0, stream); break;
                case 7: launched = mk_matvec_launch_b7(a, plan, x_dtype, uniform != 0, stream); break;
                case 8: launched = mk_matvec_launch_b8(a, plan, x_dtype, uniform != 0, stream); break;
            }
            if (launched) {
                MK_LAUNCH_CHECK("mk_packed_matvec");
                done_rows = tiles * tile_rows;
            }
        }
    }
    if (done_rows < output_width)
        return launch_words(x, x_dtype, packed, scales, scale_dtype, values, zeros, bias, bias_dtype, y, samples,
                            output_width, input_width, group, bits, uniform, grid_min, grid_step, done_rows, stream);
    return MK_OK;
}

extern "C" int mk_packed_matvec_group(const void *const *x, int x_dtype, int count, const uint8_t *const *packed,
                                      const void *const *scales, int scale_dtype, const float *values, int n_values,
                                      const void *const *zeros, const void *const *bias, int bias_dtype,
                                      void *const *y, const int *output_widths, int samples, int input_width,
                                      int group, int bits, int uniform, float grid_min, float grid_step,
                                      void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(count >= 1 && count <= mk_matvec::kMaxGroupMembers, MK_ERR_INVALID,
               "mk_packed_matvec_group: 1 to %d matrices per call", mk_matvec::kMaxGroupMembers);
    MK_REQUIRE(x && packed && scales && y && output_widths, MK_ERR_INVALID, "mk_packed_matvec_group: null argument");
    MK_REQUIRE(samples >= 1 && input_width >= 1 && group >= 1, MK_ERR_INVALID,
               "mk_packed_matvec_group: sizes must be positive");
    bool with_zeros = zeros && zeros[0];
    const bool dtypes_valid = mk_dtype_valid(x_dtype) && mk_dtype_valid(scale_dtype) && (!bias || mk_dtype_valid(bias_dtype)) &&
                              bits >= 1 && bits <= 8;
    // The kernels that take a group: the INT4 streaming kernels, else the table kernels.
    const bool streaming = dtypes_valid && !tuning().no_stream4 &&
                           mk_matvec::stream4_accepts(samples, input_width, group, bits, x_dtype, scale_dtype, uniform != 0);
    const bool tables = dtypes_valid && !streaming && !tuning().no_pairs && (uniform || (values && n_values >= 1 && n_values <= (1 << bits))) &&
                        mk_packed_layout_supported(bits, input_width, group) &&
                        input_width <= 16384 &&   // (longer rows: one launch per matrix)
                        mk_matvec::pairs_accepts(input_width, group, bits, x_dtype, scale_dtype);
    bool one_launch = (streaming || tables) && (static_cast<size_t>(input_width) * mk_dtype_bytes(x_dtype)) % 16 == 0;
    for (int i = 0; i < count; ++i) {
        MK_REQUIRE(x[i] && packed[i] && scales[i] && y[i] && output_widths[i] >= 1, MK_ERR_INVALID,
                   "mk_packed_matvec_group: matrix %d has a null pointer or no rows", i);
        MK_REQUIRE(((zeros && zeros[i]) != 0) == with_zeros, MK_ERR_INVALID,
                   "mk_packed_matvec_group: either every matrix has offsets or none has");
        const void *bias_i = bias ? bias[i] : nullptr;
        one_launch = one_launch && (reinterpret_cast<uintptr_t>(x[i]) & 15u) == 0 &&
                     (reinterpret_cast<uintptr_t>(packed[i]) & 3u) == 0 &&
                     (reinterpret_cast<uintptr_t>(scales[i]) & 3u) == 0 &&
                     (reinterpret_cast<uintptr_t>(with_zeros ? zeros[i] : nullptr) & 3u) == 0 &&
                     (reinterpret_cast<uintptr_t>(bias_i) & 3u) == 0;
    }
    if (!one_launch) {  // the same results, one launch per matrix
        for (int i = 0; i < count; ++i)
            if (int status = mk_packed_matvec(x[i], x_dtype, packed[i], scales[i], scale_dtype, values, n_values,
                                              with_zeros ? zeros[i] : nullptr, bias ? bias[i] : nullptr, bias_dtype,
                                              y[i], samples, output_widths[i], input_width, group, bits, uniform,
                                              grid_min, grid_step, stream_))
                return status;
        return MK_OK;
    }
    mk_matvec::Stream4Args shared{};
    shared.x = x[0]; shared.samples = samples; shared.width = input_width; shared.group = group;
    shared.groups = mk_cdiv(input_width, group); shared.bias_dtype = bias_dtype; shared.grid_min = grid_min;
    shared.grid_step = grid_step; shared.values = values; shared.n_values = n_values; shared.uniform = uniform;
    shared.bits = bits; shared.x_dtype = x_dtype; shared.scale_dtype = scale_dtype;
    mk_matvec::Stream4Group members{};
    members.count = count;
    for (int i = 0; i < count; ++i) {
        members.member[i].x = x[i];
        members.member[i].packed = packed[i];
        members.member[i].scales = scales[i];
        members.member[i].zeros = with_zeros ? zeros[i] : nullptr;
        members.member[i].bias = bias ? bias[i] : nullptr;
        members.member[i].y = y[i];
    }
    int rows_per_tile = 0;
    if (streaming)
        MK_REQUIRE(mk_matvec::stream4_launch_group(shared, members, output_widths, &rows_per_tile, stream) == 0, MK_ERR_HIP,
                   "mk_packed_matvec_group: the runtime refused the kernel's LDS size");
    else
        mk_matvec::pairs_launch_group(shared, members, output_widths, &rows_per_tile, stream);
    MK_LAUNCH_CHECK("mk_packed_matvec_group");
    for (int i = 0; i < count; ++i) {  // rows past a member's last whole tile
        int covered = output_widths[i] / rows_per_tile * rows_per_tile;
        if (streaming && output_widths[i] - covered >= 4) {   // their whole four-row tiles, as in the single call
            mk_matvec::Stream4Args own = shared;
            own.x = x[i]; own.packed = packed[i]; own.scales = scales[i]; own.zeros = members.member[i].zeros;
            own.bias = members.member[i].bias; own.y = y[i]; own.rows = output_widths[i];
            const int more = mk_matvec::stream4_launch_remainder(own, covered, stream);
            MK_REQUIRE(more >= 0, MK_ERR_HIP, "mk_packed_matvec_group: the runtime refused the kernel's LDS size");
            MK_LAUNCH_CHECK("mk_packed_matvec_group");
            covered += more;
        }
        if (covered < output_widths[i])
            if (int status = launch_words(x[i], x_dtype, packed[i], scales[i], scale_dtype, values, members.member[i].zeros,
                                          members.member[i].bias, bias_dtype, y[i], samples, output_widths[i],
                                          input_width, group, bits, uniform, grid_min, grid_step, covered, stream))
                return status;
    }
    return MK_OK;
}
