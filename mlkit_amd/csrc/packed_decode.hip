// Packed codes -> dense weight matrix on gfx950 (prefill path and `.weight`).
//
// out[n, k] = (uniform ? grid_min + code*grid_step : values[code]) * scale[n, k/group]
//             (+ zero[n, k/group]),  every operation a separate fp32 operation.
//
// One thread decodes one packing word (the fewest whole bytes holding whole codes), so
// consecutive threads read consecutive bytes and write consecutive elements.
//
// Replaces the reference's Triton kernel `decode_rows`
// (kernels/packed_linear.py:229-276 in /root/reference/src/mlkit).

#include "mk_common.h"

namespace {

struct DecodeArgs {
    const uint8_t *packed;
    const void *scales;
    const void *zeros;
    const float *values;
    void *out;
    int rows, width, group, groups;
    int scale_dtype, out_dtype;
    int bits, bytes_per_word, codes_per_word, uniform;
    float grid_min, grid_step;
};

__global__ void packed_decode_kernel(const DecodeArgs a) {
    const int row_words = a.width / a.codes_per_word;
    const size_t total = static_cast<size_t>(a.rows) * row_words;
    const uint64_t mask = (1ull << a.bits) - 1ull;
    for (size_t word = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; word < total;
         word += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t row = word / row_words;
        const int word_in_row = static_cast<int>(word - row * row_words);
        const uint8_t *source = a.packed + word * a.bytes_per_word;
        uint64_t bits = 0;
        for (int b = 0; b < a.bytes_per_word; ++b) bits |= static_cast<uint64_t>(source[b]) << (8 * b);
        for (int i = 0; i < a.codes_per_word; ++i) {
            const int k = word_in_row * a.codes_per_word + i;
            const uint32_t code = static_cast<uint32_t>((bits >> (i * a.bits)) & mask);
            const size_t slot = row * a.groups + k / a.group;
            float weight;
            if (a.uniform) {
                const float stepped = __fmul_rn(static_cast<float>(code), a.grid_step);
                weight = __fadd_rn(a.grid_min, stepped);
            } else {
                weight = a.values[code];
            }
            weight = __fmul_rn(weight, mk_load_as_float(a.scales, slot, a.scale_dtype));
            if (a.zeros) weight = __fadd_rn(weight, mk_load_as_float(a.zeros, slot, a.scale_dtype));
            mk_store_from_float(a.out, row * a.width + k, a.out_dtype, weight);
        }
    }
}

}  // namespace

extern "C" int mk_packed_decode(const uint8_t *packed, const void *scales, int scale_dtype,
                                const float *values, int n_values, const void *zeros, void *out,
                                int out_dtype, int output_width, int input_width, int group, int bits,
                                int uniform, float grid_min, float grid_step, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(packed && scales && out, MK_ERR_INVALID, "mk_packed_decode: null tensor pointer");
    MK_REQUIRE(mk_dtype_valid(scale_dtype) && mk_dtype_valid(out_dtype), MK_ERR_INVALID,
               "mk_packed_decode: unknown dtype code");
    MK_REQUIRE(output_width >= 1 && input_width >= 1 && group >= 1, MK_ERR_INVALID,
               "mk_packed_decode: sizes must be positive");
    MK_REQUIRE(bits >= 1 && bits <= 8, MK_ERR_INVALID, "mk_packed_decode: code width must be 1..8 bits");
    MK_REQUIRE(uniform || (values && n_values >= 1 && n_values <= (1 << bits)), MK_ERR_INVALID,
               "mk_packed_decode: a value table of at most 2^bits entries is required");
    MK_REQUIRE(mk_packed_layout_supported(bits, input_width, group), MK_ERR_UNSUPPORTED,
               "mk_packed_decode: rows or scale groups split a packing word (bits=%d width=%d group=%d)",
               bits, input_width, group);
    DecodeArgs a;
    a.packed = packed; a.scales = scales; a.zeros = zeros; a.values = values; a.out = out;
    a.rows = output_width; a.width = input_width; a.group = group; a.groups = mk_cdiv(input_width, group);
    a.scale_dtype = scale_dtype; a.out_dtype = out_dtype; a.bits = bits;
    const int divisor = mk_gcd(bits, 8);
    a.bytes_per_word = bits / divisor; a.codes_per_word = 8 / divisor; a.uniform = uniform;
    a.grid_min = grid_min; a.grid_step = grid_step;
    const size_t words = static_cast<size_t>(output_width) * (input_width / a.codes_per_word);
    size_t blocks = (words + 255) / 256;
    if (blocks > 256u * 32u) blocks = 256u * 32u;
    hipLaunchKernelGGL(packed_decode_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a);
    MK_LAUNCH_CHECK("mk_packed_decode");
    return MK_OK;
}
