// Integer codes <-> little-endian bit stream on gfx950.
//
// Code i of width b occupies stream bits [i b, (i + 1) b); byte j holds stream bits
// [8 j, 8 j + 8), least significant first; the stream is ceil(count b / 8) bytes.  A thread
// owns 32 consecutive codes, which are exactly b dwords of the stream whatever b is, so no
// two threads share a byte: the codes pass through a 64-bit shift register and leave (or
// enter) as whole dwords.  The codes past the last whole run of 32 go byte by byte.
//
// Replaces the tensor operations of the reference's `pack` / `unpack`
// (quantization/operations/bit_packing.py:13-135 in /root/reference/src/mlkit).

#include <type_traits>

#include "mk_common.h"

namespace {

constexpr int kRun = 32;  // codes per thread

struct StreamArgs {
    const void *codes_in;   // pack: source codes
    void *codes_out;        // unpack: uint8 (bits <= 8) or int32 codes
    uint8_t *packed;        // pack: target stream
    const uint8_t *stream;  // unpack: source stream
    long long count;
    int bits;
    int *overflow;
};

// Code `index` as an unsigned value; `bad` collects what does not fit `bits` bits.
template <int CODE_BYTES>
__device__ __forceinline__ uint32_t code_at(const void *codes, long long index, int bits, uint32_t &bad) {
    if constexpr (CODE_BYTES == 1) {
        const uint32_t value = static_cast<const uint8_t *>(codes)[index];
        bad |= value >> bits;
        return value;
    } else if constexpr (CODE_BYTES == 2) {
        const int value = static_cast<const int16_t *>(codes)[index];
        bad |= static_cast<uint32_t>(value) >> bits;  // a negative value has high bits set
        return static_cast<uint32_t>(value);
    } else if constexpr (CODE_BYTES == 4) {
        const int value = static_cast<const int32_t *>(codes)[index];
        bad |= static_cast<uint32_t>(value) >> bits;
        return static_cast<uint32_t>(value);
    } else {
        const long long value = static_cast<const long long *>(codes)[index];
        bad |= (static_cast<unsigned long long>(value) >> bits) != 0 ? 1u : 0u;
        return static_cast<uint32_t>(value);
    }
}

// A whole run of 32 codes as unsigned values.  WIDE: the codes start on a 16-byte boundary (a run of one-byte
// codes is then two 16-byte loads, of four-byte codes eight, instead of 32 scalar ones at a stride that wastes
// most of every cache line a wavefront touches).
template <int CODE_BYTES, bool WIDE>
__device__ __forceinline__ void run_at(const void *codes, long long first, int bits, uint32_t (&value)[kRun], uint32_t &bad) {
    if constexpr (WIDE && CODE_BYTES == 1) {
        const uint4 *source = reinterpret_cast<const uint4 *>(static_cast<const uint8_t *>(codes) + first);
        const uint4 halves[2] = {source[0], source[1]};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t words[4] = {halves[h].x, halves[h].y, halves[h].z, halves[h].w};
#pragma unroll
            for (int w = 0; w < 4; ++w)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const uint32_t code = (words[w] >> (8 * b)) & 0xffu;
                    value[16 * h + 4 * w + b] = code;
                    bad |= code >> bits;
                }
        }
    } else if constexpr (WIDE && CODE_BYTES == 4) {
        const uint4 *source = reinterpret_cast<const uint4 *>(static_cast<const int32_t *>(codes) + first);
#pragma unroll
        for (int q = 0; q < kRun / 4; ++q) {
            const uint4 four = source[q];
            const uint32_t words[4] = {four.x, four.y, four.z, four.w};
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                value[4 * q + w] = words[w];
                bad |= words[w] >> bits;   // a negative value has high bits set
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < kRun; ++i) value[i] = code_at<CODE_BYTES>(codes, first + i, bits, bad);
    }
}

// ALIGNED: the stream starts on a 4-byte boundary and whole runs are stored as dwords.
// WIDE: see run_at.
// BITS: the code width when the launch knows it (the shift register then resolves at compile time and a run's
// dwords leave as one or two wide stores), or 0 for a.bits.
template <int CODE_BYTES, bool ALIGNED, bool WIDE = false, int BITS = 0>
__global__ void __launch_bounds__(256) pack_kernel(const StreamArgs a_) {
    StreamArgs a = a_;
    if constexpr (BITS != 0) a.bits = BITS;
    const long long whole_runs = a.count / kRun;
    const long long runs = whole_runs + (a.count % kRun ? 1 : 0);
    const uint32_t mask = (1u << a.bits) - 1u;
    uint32_t bad = 0;
    for (long long run = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; run < runs;
         run += static_cast<long long>(gridDim.x) * blockDim.x) {
        const long long first = run * kRun;
        uint8_t *target = a.packed + run * (4 * a.bits);
        if (run < whole_runs) {
            uint64_t window = 0;
            int filled = 0, word = 0;
            uint32_t value[kRun];
            run_at<CODE_BYTES, WIDE>(a.codes_in, first, a.bits, value, bad);
            if constexpr (BITS == 4 && ALIGNED) {   // 16-byte aligned: the stream is, and a run is 16 bytes
                uint32_t words[4];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    words[w] = 0;
#pragma unroll
                    for (int i = 0; i < 8; ++i) words[w] |= (value[8 * w + i] & 15u) << (4 * i);
                }
                typedef uint32_t u4 __attribute__((ext_vector_type(4), aligned(4)));
                *reinterpret_cast<u4 *>(target) = u4{words[0], words[1], words[2], words[3]};
                continue;
            }
#pragma unroll
            for (int i = 0; i < kRun; ++i) {
                window |= static_cast<uint64_t>(value[i] & mask) << filled;
                filled += a.bits;
                if (filled >= 32) {
                    const uint32_t out = static_cast<uint32_t>(window);
                    if constexpr (ALIGNED) {
                        reinterpret_cast<uint32_t *>(target)[word] = out;
                    } else {
                        for (int b = 0; b < 4; ++b) target[4 * word + b] = static_cast<uint8_t>(out >> (8 * b));
                    }
                    ++word;
                    window >>= 32;
                    filled -= 32;
                }
            }
        } else {  // the last, partial run: whole bytes, the final one zero padded
            const int left = static_cast<int>(a.count - first);
            uint64_t window = 0;
            int filled = 0, byte = 0;
            for (int i = 0; i < left; ++i) {
                window |= static_cast<uint64_t>(code_at<CODE_BYTES>(a.codes_in, first + i, a.bits, bad) & mask) << filled;
                filled += a.bits;
                while (filled >= 8) {
                    target[byte++] = static_cast<uint8_t>(window);
                    window >>= 8;
                    filled -= 8;
                }
            }
            if (filled > 0) target[byte] = static_cast<uint8_t>(window);
        }
    }
    if (bad && a.overflow) atomicOr(a.overflow, 1);
}

template <bool WIDE_CODES, bool ALIGNED, int BITS = 0>
__global__ void __launch_bounds__(256) unpack_kernel(const StreamArgs a_) {
    StreamArgs a = a_;
    if constexpr (BITS != 0) a.bits = BITS;   // known at the launch: the shift register resolves at compile time
    const long long whole_runs = a.count / kRun;
    const long long runs = whole_runs + (a.count % kRun ? 1 : 0);
    const long long stream_bytes = (a.count * a.bits + 7) / 8;
    const uint32_t mask = (1u << a.bits) - 1u;
    for (long long run = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; run < runs;
         run += static_cast<long long>(gridDim.x) * blockDim.x) {
        const long long first = run * kRun;
        const long long source_byte = run * (4 * a.bits);
        const uint8_t *source = a.stream + source_byte;
        const int left = run < whole_runs ? kRun : static_cast<int>(a.count - first);
        if constexpr (BITS != 0 && ALIGNED && !WIDE_CODES) {
            // A whole run of a known width onto an aligned target: the run's BITS dwords in one go, every code by a
            // constant shift, two 16-byte stores.
            uint8_t *target = static_cast<uint8_t *>(a.codes_out) + first;
            if (run < whole_runs && (reinterpret_cast<uintptr_t>(target) & 3u) == 0) {
                uint32_t words[BITS];
                typedef uint32_t chunk __attribute__((ext_vector_type(BITS == 3 ? 3 : (BITS >= 4 ? 4 : BITS)), aligned(4)));
                if constexpr (BITS <= 4) {
                    const chunk loaded = *reinterpret_cast<const chunk *>(source);
#pragma unroll
                    for (int w = 0; w < BITS; ++w) words[w] = loaded[w];
                } else {
#pragma unroll
                    for (int q = 0; q < BITS / 4; ++q) {
                        const chunk loaded = reinterpret_cast<const chunk *>(source)[q];
#pragma unroll
                        for (int w = 0; w < 4; ++w) words[4 * q + w] = loaded[w];
                    }
                }
                uint32_t packed[kRun / 4];
#pragma unroll
                for (int q = 0; q < kRun / 4; ++q) {
                    packed[q] = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        constexpr uint32_t kMask = (1u << BITS) - 1u;
                        const int position = (4 * q + j) * BITS, index = position >> 5, shift = position & 31;
                        uint32_t code = words[index] >> shift;
                        if (shift + BITS > 32) code |= words[(index + 1) % BITS] << (32 - shift);
                        packed[q] |= (code & kMask) << (8 * j);
                    }
                }
                typedef uint32_t u4 __attribute__((ext_vector_type(4), aligned(4)));
                reinterpret_cast<u4 *>(target)[0] = u4{packed[0], packed[1], packed[2], packed[3]};
                reinterpret_cast<u4 *>(target)[1] = u4{packed[4], packed[5], packed[6], packed[7]};
                continue;
            }
        }
        uint64_t window = 0;
        int filled = 0, word = 0;
        uint32_t out[kRun];
#pragma unroll
        for (int i = 0; i < kRun; ++i) {
            if (filled < a.bits && i < left) {
                uint32_t next = 0;
                if (ALIGNED && run < whole_runs) {
                    next = reinterpret_cast<const uint32_t *>(source)[word];
                } else {
                    for (int b = 0; b < 4; ++b)
                        if (source_byte + 4 * word + b < stream_bytes) next |= static_cast<uint32_t>(source[4 * word + b]) << (8 * b);
                }
                ++word;
                window |= static_cast<uint64_t>(next) << filled;
                filled += 32;
            }
            out[i] = static_cast<uint32_t>(window) & mask;
            window >>= a.bits;
            filled -= a.bits;
        }
        if constexpr (WIDE_CODES) {
            int32_t *target = static_cast<int32_t *>(a.codes_out) + first;
#pragma unroll
            for (int i = 0; i < kRun; ++i)  // constant indices keep `out` in registers
                if (i < left) target[i] = static_cast<int32_t>(out[i]);
        } else {
            uint8_t *target = static_cast<uint8_t *>(a.codes_out) + first;
            if (left == kRun && (reinterpret_cast<uintptr_t>(target) & 3u) == 0) {
                uint32_t words[kRun / 4];
#pragma unroll
                for (int q = 0; q < kRun / 4; ++q)
                    words[q] = out[4 * q] | (out[4 * q + 1] << 8) | (out[4 * q + 2] << 16) | (out[4 * q + 3] << 24);
                typedef uint32_t u4 __attribute__((ext_vector_type(4), aligned(4)));   // two wide stores per run
                reinterpret_cast<u4 *>(target)[0] = u4{words[0], words[1], words[2], words[3]};
                reinterpret_cast<u4 *>(target)[1] = u4{words[4], words[5], words[6], words[7]};
            } else {
#pragma unroll
                for (int i = 0; i < kRun; ++i)
                    if (i < left) target[i] = static_cast<uint8_t>(out[i]);
            }
        }
    }
}

unsigned grid_for(long long count) {
    const long long runs = (count + kRun - 1) / kRun;
    long long blocks = (runs + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    return static_cast<unsigned>(blocks < 1 ? 1 : blocks);
}

}  // namespace

extern "C" int mk_pack(const void *codes, int code_bytes, long long count, int bits, uint8_t *packed, int *overflow,
                       void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(bits >= 1 && bits <= 16, MK_ERR_INVALID, "mk_pack: packing supports one through sixteen bits");
    MK_REQUIRE(count >= 0, MK_ERR_INVALID, "mk_pack: negative count");
    MK_REQUIRE(code_bytes == 1 || code_bytes == 2 || code_bytes == 4 || code_bytes == 8, MK_ERR_INVALID,
               "mk_pack: codes are uint8, int16, int32 or int64");
    if (count == 0) return MK_OK;
    MK_REQUIRE(codes && packed, MK_ERR_INVALID, "mk_pack: null tensor pointer");
    StreamArgs a{};
    a.codes_in = codes; a.packed = packed; a.count = count; a.bits = bits; a.overflow = overflow;
    const bool aligned = (reinterpret_cast<uintptr_t>(packed) & 3u) == 0;
    const bool wide = aligned && (reinterpret_cast<uintptr_t>(codes) & 15u) == 0 && (code_bytes == 1 || code_bytes == 4);
    const dim3 grid(grid_for(count)), block(256);
    if (wide) {
        if (code_bytes == 1) {
            switch (bits) {
                case 2: hipLaunchKernelGGL((pack_kernel<1, true, true, 2>), grid, block, 0, stream, a); break;
                case 3: hipLaunchKernelGGL((pack_kernel<1, true, true, 3>), grid, block, 0, stream, a); break;
                case 4: hipLaunchKernelGGL((pack_kernel<1, true, true, 4>), grid, block, 0, stream, a); break;
                case 8: hipLaunchKernelGGL((pack_kernel<1, true, true, 8>), grid, block, 0, stream, a); break;
                default: hipLaunchKernelGGL((pack_kernel<1, true, true>), grid, block, 0, stream, a); break;
            }
        } else {
            hipLaunchKernelGGL((pack_kernel<4, true, true>), grid, block, 0, stream, a);
        }
        MK_LAUNCH_CHECK("mk_pack");
        return MK_OK;
    }
    auto launch = [&](auto aligned_tag) {
        constexpr bool A = decltype(aligned_tag)::value;
        switch (code_bytes) {
            case 1: hipLaunchKernelGGL((pack_kernel<1, A>), grid, block, 0, stream, a); break;
            case 2: hipLaunchKernelGGL((pack_kernel<2, A>), grid, block, 0, stream, a); break;
            case 4: hipLaunchKernelGGL((pack_kernel<4, A>), grid, block, 0, stream, a); break;
            default: hipLaunchKernelGGL((pack_kernel<8, A>), grid, block, 0, stream, a); break;
        }
    };
    if (aligned) launch(std::true_type{});
    else launch(std::false_type{});
    MK_LAUNCH_CHECK("mk_pack");
    return MK_OK;
}

extern "C" int mk_unpack(const uint8_t *packed, long long count, int bits, void *codes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(bits >= 1 && bits <= 16, MK_ERR_INVALID, "mk_unpack: one through sixteen bits");
    MK_REQUIRE(count >= 0, MK_ERR_INVALID, "mk_unpack: negative count");
    if (count == 0) return MK_OK;
    MK_REQUIRE(packed && codes, MK_ERR_INVALID, "mk_unpack: null tensor pointer");
    StreamArgs a{};
    a.stream = packed; a.codes_out = codes; a.count = count; a.bits = bits;
    const bool aligned = (reinterpret_cast<uintptr_t>(packed) & 3u) == 0;
    const dim3 grid(grid_for(count)), block(256);
    if (bits > 8) {
        if (aligned) hipLaunchKernelGGL((unpack_kernel<true, true>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((unpack_kernel<true, false>), grid, block, 0, stream, a);
    } else {
        if (aligned) {
            switch (bits) {
                case 2: hipLaunchKernelGGL((unpack_kernel<false, true, 2>), grid, block, 0, stream, a); break;
                case 3: hipLaunchKernelGGL((unpack_kernel<false, true, 3>), grid, block, 0, stream, a); break;
                case 4: hipLaunchKernelGGL((unpack_kernel<false, true, 4>), grid, block, 0, stream, a); break;
                case 8: hipLaunchKernelGGL((unpack_kernel<false, true, 8>), grid, block, 0, stream, a); break;
                default: hipLaunchKernelGGL((unpack_kernel<false, true>), grid, block, 0, stream, a); break;
            }
        } else {
            hipLaunchKernelGGL((unpack_kernel<false, false>), grid, block, 0, stream, a);
        }
    }
    MK_LAUNCH_CHECK("mk_unpack");
    return MK_OK;
}
