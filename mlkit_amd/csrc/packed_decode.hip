// Packed codes -> dense weight matrix on gfx950 (prefill path and `.weight`).
//
// out[n, k] = (uniform ? grid_min + code*grid_step : values[code]) * scale[n, k/group]
//             (+ zero[n, k/group]),  every operation a separate fp32 operation.
//
// Rows that are whole multiples of 32 codes are decoded a chunk of 32 codes (BITS dwords)
// per thread: a few wide loads, 32 values from registers, wide stores.  Other layouts take
// the word kernel: one thread per packing word (the fewest whole bytes holding whole codes).
//
// Replaces the reference's Triton kernel `decode_rows`
// (kernels/packed_linear.py:229-276 in /root/reference/src/mlkit).

#include "packed_matvec_impl.h"

namespace {

struct DecodeArgs {
    const uint8_t *packed;
    const void *scales;
    const void *zeros;
    const float *values;
    void *out;
    int rows, width, group, groups;
    int scale_dtype, out_dtype;
    int bits, bytes_per_word, codes_per_word, uniform, n_values;
    float grid_min, grid_step;
    int chunks_per_group_shift;   // log2(group / 32) when that is a power of two (31: one group per row), else -1
    const long long *row_index;   // null, or the source row of every output row (a gather of rows)
    int source_rows;              // rows of the packed matrix; index i < 0 means source_rows + i; one still outside reads row 0
};

// The row of the packed matrix that output row `row` decodes.
__device__ __forceinline__ size_t source_row_of(const DecodeArgs &a, size_t row) {
    if (!a.row_index) return row;
    long long wanted = a.row_index[row];
    if (wanted < 0) wanted += a.source_rows;   // -1 is the last row, as in tensor indexing
    return wanted >= 0 && wanted < a.source_rows ? static_cast<size_t>(wanted) : 0;
}

__global__ void packed_decode_kernel(const DecodeArgs a) {
    const int row_words = a.width / a.codes_per_word;
    const size_t total = static_cast<size_t>(a.rows) * row_words;
    const uint64_t mask = (1ull << a.bits) - 1ull;
    for (size_t word = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; word < total;
         word += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t row = word / row_words;
        const int word_in_row = static_cast<int>(word - row * row_words);
        const size_t from = source_row_of(a, row);
        const uint8_t *source = a.packed + (from * row_words + word_in_row) * a.bytes_per_word;
        uint64_t bits = 0;
        for (int b = 0; b < a.bytes_per_word; ++b) bits |= static_cast<uint64_t>(source[b]) << (8 * b);
        for (int i = 0; i < a.codes_per_word; ++i) {
            const int k = word_in_row * a.codes_per_word + i;
            const uint32_t code = static_cast<uint32_t>((bits >> (i * a.bits)) & mask);
            const size_t slot = from * a.groups + k / a.group;
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


// One thread per chunk of 32 codes.  The value table is staged in LDS.
//
// A lane's 32 outputs are 64 bytes (128 of fp32): stored directly, a wavefront instruction
// would write 16 bytes at a stride of 64 and touch 64 cache lines.  The lanes of a
// wavefront therefore exchange their 16-byte pieces through LDS (each chunk's pieces one
// piece apart from the next chunk's, so both directions avoid bank conflicts) and every
// store instruction writes 1 KB of adjacent bytes.  A wavefront's 64 chunks are adjacent
// in the row-major output because rows are whole chunks.
//
// OUT is the output type (MK_F32: eight 16-byte pieces per chunk, else four).  MODE fixes the
// launch's uniform choices at compile time, because tested per element they cost more
// instructions than the decoding: 0 leaves them to run time (scale groups that are not whole
// chunks); 1 / 2: one scale per chunk, affine grid, without / with offsets; 3 / 4: the same
// for a value table.
template <int BITS, int OUT, int MODE>
__global__ void __launch_bounds__(256) packed_decode_chunks_kernel(const DecodeArgs a) {
    constexpr int PIECES = OUT == MK_F32 ? 8 : 4;
    constexpr bool kFixed = MODE != 0;
    const bool uniform = kFixed ? MODE <= 2 : a.uniform != 0;
    const bool has_zero = kFixed ? MODE % 2 == 0 : a.zeros != nullptr;
    __shared__ float table[1 << BITS];
    __shared__ mk_u32x4 exchange[4][64 * (PIECES + 1)];
    if (!uniform) {
        for (int i = threadIdx.x; i < (1 << BITS); i += blockDim.x) table[i] = i < a.n_values ? a.values[i] : 0.0f;
        __syncthreads();
    }
    const int lane = threadIdx.x & 63;
    mk_u32x4 *mine = exchange[threadIdx.x >> 6];
    // Chunk indices fit 32 bits (the launcher checks): a 64-bit division per lane and trip
    // would cost as much as decoding the chunk.
    const uint32_t row_chunks = static_cast<uint32_t>(a.width) / mk_matvec::kChunkCodes;
    const uint32_t total = static_cast<uint32_t>(a.rows) * row_chunks;
    const bool one_slot = kFixed || a.group % mk_matvec::kChunkCodes == 0 || a.group >= a.width;
    // The trip count is uniform within a wavefront: lanes past the end repeat the last chunk
    // and store nothing.
    for (uint32_t first_chunk = (blockIdx.x * blockDim.x + threadIdx.x) & ~63u; first_chunk < total;
         first_chunk += gridDim.x * blockDim.x) {
        const uint32_t wanted = first_chunk + lane;
        const uint32_t chunk = wanted < total ? wanted : total - 1;
        const uint32_t row = chunk / row_chunks;
        const uint32_t chunk_in_row = chunk - row * row_chunks;
        const int first = static_cast<int>(chunk_in_row) * mk_matvec::kChunkCodes;
        mk_matvec::CodeChunk<BITS> codes;
        const size_t from = source_row_of(a, row);
        mk_matvec::load_codes<BITS>(codes, a.packed + (from * row_chunks + chunk_in_row) * (4 * BITS));
        const uint32_t group_in_row = a.chunks_per_group_shift >= 0 ? chunk_in_row >> a.chunks_per_group_shift
                                                                    : static_cast<uint32_t>(first) / static_cast<uint32_t>(a.group);
        size_t slot = from * a.groups + group_in_row;
        float scale = mk_load_as_float(a.scales, slot, a.scale_dtype);
        float zero = has_zero ? mk_load_as_float(a.zeros, slot, a.scale_dtype) : 0.0f;
        float out[32];
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            if (!one_slot) {
                slot = from * a.groups + (first + k) / a.group;
                scale = mk_load_as_float(a.scales, slot, a.scale_dtype);
                if (has_zero) zero = mk_load_as_float(a.zeros, slot, a.scale_dtype);
            }
            const uint32_t code = mk_matvec::code_at<BITS>(codes, k);
            float weight = uniform ? __fadd_rn(a.grid_min, __fmul_rn(static_cast<float>(code), a.grid_step))
                                   : table[code];
            weight = __fmul_rn(weight, scale);
            if (has_zero) weight = __fadd_rn(weight, zero);
            out[k] = weight;
        }
#pragma unroll
        for (int q = 0; q < PIECES; ++q) {
            mk_u32x4 piece;
            if constexpr (PIECES == 8) {
#pragma unroll
                for (int h = 0; h < 4; ++h) piece[h] = __float_as_uint(out[4 * q + h]);
            } else {
#pragma unroll
                for (int h = 0; h < 4; ++h) {
                    const float low = out[8 * q + 2 * h], high = out[8 * q + 2 * h + 1];
                    if constexpr (OUT == MK_F16) {
                        const mk_h2 halves = {static_cast<_Float16>(low), static_cast<_Float16>(high)};
                        piece[h] = __builtin_bit_cast(uint32_t, halves);
                    } else {
                        piece[h] = static_cast<uint32_t>(mk_float_to_bf16(low)) | (static_cast<uint32_t>(mk_float_to_bf16(high)) << 16);
                    }
                }
            }
            mine[lane * (PIECES + 1) + q] = piece;
        }
        // The pieces cross lanes through LDS: the wavefront's writes are ordered before its reads
        // (the hardware completes a wavefront's LDS operations in order; the fence keeps the
        // compiler from moving a read above a write it cannot prove distinct).
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        mk_u32x4 *target = static_cast<mk_u32x4 *>(a.out) + static_cast<size_t>(first_chunk) * PIECES;
        const size_t pieces_left = static_cast<size_t>(total - first_chunk) * PIECES;
#pragma unroll
        for (int q = 0; q < PIECES; ++q) {
            const int index = q * 64 + lane;
            const mk_u32x4 piece = mine[(index / PIECES) * (PIECES + 1) + index % PIECES];
            if (static_cast<size_t>(index) < pieces_left) target[index] = piece;
        }
        // ... and this trip's reads before the next trip's writes.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

template <int BITS, int OUT>
void launch_chunks_as(const DecodeArgs &a, hipStream_t stream) {
    const size_t chunks = static_cast<size_t>(a.rows) * (a.width / mk_matvec::kChunkCodes);
    size_t blocks = (chunks + 255) / 256;
    if (blocks > 256u * 64u) blocks = 256u * 64u;
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    const bool one_slot = a.group % mk_matvec::kChunkCodes == 0 || a.group >= a.width;
    if (!one_slot) hipLaunchKernelGGL((packed_decode_chunks_kernel<BITS, OUT, 0>), grid, block, 0, stream, a);
    else if (a.uniform && !a.zeros) hipLaunchKernelGGL((packed_decode_chunks_kernel<BITS, OUT, 1>), grid, block, 0, stream, a);
    else if (a.uniform) hipLaunchKernelGGL((packed_decode_chunks_kernel<BITS, OUT, 2>), grid, block, 0, stream, a);
    else if (!a.zeros) hipLaunchKernelGGL((packed_decode_chunks_kernel<BITS, OUT, 3>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((packed_decode_chunks_kernel<BITS, OUT, 4>), grid, block, 0, stream, a);
}

template <int BITS>
void launch_chunks(const DecodeArgs &a, hipStream_t stream) {
    if (a.out_dtype == MK_F32) launch_chunks_as<BITS, MK_F32>(a, stream);
    else if (a.out_dtype == MK_F16) launch_chunks_as<BITS, MK_F16>(a, stream);
    else launch_chunks_as<BITS, MK_BF16>(a, stream);
}

}  // namespace

namespace {

int decode_rows(const uint8_t *packed, const void *scales, int scale_dtype, const float *values, int n_values,
                const void *zeros, void *out, int out_dtype, int output_rows, int input_width, int group, int bits,
                int uniform, float grid_min, float grid_step, const long long *row_index, int source_rows,
                const char *name, hipStream_t stream) {
    MK_REQUIRE(packed && scales && out, MK_ERR_INVALID, "%s: null tensor pointer", name);
    MK_REQUIRE(mk_dtype_valid(scale_dtype) && mk_dtype_valid(out_dtype), MK_ERR_INVALID, "%s: unknown dtype code", name);
    MK_REQUIRE(output_rows >= 1 && input_width >= 1 && group >= 1, MK_ERR_INVALID, "%s: sizes must be positive", name);
    MK_REQUIRE(bits >= 1 && bits <= 8, MK_ERR_INVALID, "%s: code width must be 1..8 bits", name);
    MK_REQUIRE(uniform || (values && n_values >= 1 && n_values <= (1 << bits)), MK_ERR_INVALID,
               "%s: a value table of at most 2^bits entries is required", name);
    MK_REQUIRE(mk_packed_layout_supported(bits, input_width, group), MK_ERR_UNSUPPORTED,
               "%s: rows or scale groups split a packing word (bits=%d width=%d group=%d)", name, bits, input_width,
               group);
    DecodeArgs a;
    a.packed = packed; a.scales = scales; a.zeros = zeros; a.values = values; a.out = out;
    a.rows = output_rows; a.width = input_width; a.group = group; a.groups = mk_cdiv(input_width, group);
    a.scale_dtype = scale_dtype; a.out_dtype = out_dtype; a.bits = bits;
    a.row_index = row_index; a.source_rows = source_rows;
    const int divisor = mk_gcd(bits, 8);
    a.bytes_per_word = bits / divisor; a.codes_per_word = 8 / divisor; a.uniform = uniform;
    a.grid_min = grid_min; a.grid_step = grid_step;
    a.n_values = n_values;
    a.chunks_per_group_shift = -1;
    if (group >= input_width) {
        a.chunks_per_group_shift = 31;
    } else if (group % mk_matvec::kChunkCodes == 0) {
        const int chunks_per_group = group / mk_matvec::kChunkCodes;
        if ((chunks_per_group & (chunks_per_group - 1)) == 0) {
            a.chunks_per_group_shift = 0;
            while ((1 << a.chunks_per_group_shift) < chunks_per_group) ++a.chunks_per_group_shift;
        }
    }
    const bool wide = input_width % mk_matvec::kChunkCodes == 0 && (reinterpret_cast<uintptr_t>(packed) & 3u) == 0 &&
                      (reinterpret_cast<uintptr_t>(out) & 15u) == 0 && bits >= 2 &&
                      static_cast<long long>(output_rows) * (input_width / mk_matvec::kChunkCodes) < (1ll << 31) - (1 << 24);
    if (wide) {
        switch (bits) {
            case 2: launch_chunks<2>(a, stream); break;
            case 3: launch_chunks<3>(a, stream); break;
            case 4: launch_chunks<4>(a, stream); break;
            case 5: launch_chunks<5>(a, stream); break;
            case 6: launch_chunks<6>(a, stream); break;
            case 7: launch_chunks<7>(a, stream); break;
            default: launch_chunks<8>(a, stream); break;
        }
        MK_LAUNCH_CHECK(name);
        return MK_OK;
    }
    const size_t words = static_cast<size_t>(output_rows) * (input_width / a.codes_per_word);
    size_t blocks = (words + 255) / 256;
    if (blocks > 256u * 32u) blocks = 256u * 32u;
    hipLaunchKernelGGL(packed_decode_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a);
    MK_LAUNCH_CHECK(name);
    return MK_OK;
}

}  // namespace

extern "C" int mk_packed_decode(const uint8_t *packed, const void *scales, int scale_dtype,
                                const float *values, int n_values, const void *zeros, void *out,
                                int out_dtype, int output_width, int input_width, int group, int bits,
                                int uniform, float grid_min, float grid_step, void *stream) {
    return decode_rows(packed, scales, scale_dtype, values, n_values, zeros, out, out_dtype, output_width, input_width,
                       group, bits, uniform, grid_min, grid_step, nullptr, output_width, "mk_packed_decode",
                       static_cast<hipStream_t>(stream));
}

extern "C" int mk_packed_decode_rows(const uint8_t *packed, const void *scales, int scale_dtype,
                                     const float *values, int n_values, const void *zeros, const long long *rows,
                                     int n_rows, void *out, int out_dtype, int output_width, int input_width,
                                     int group, int bits, int uniform, float grid_min, float grid_step,
                                     void *stream) {
    MK_REQUIRE(n_rows >= 0 && output_width >= 1, MK_ERR_INVALID, "mk_packed_decode_rows: sizes must be positive");
    if (n_rows == 0) return MK_OK;
    MK_REQUIRE(rows, MK_ERR_INVALID, "mk_packed_decode_rows: null row list");
    return decode_rows(packed, scales, scale_dtype, values, n_values, zeros, out, out_dtype, n_rows, input_width, group,
                       bits, uniform, grid_min, grid_step, rows, output_width, "mk_packed_decode_rows",
                       static_cast<hipStream_t>(stream));
}
