// Shared host/device helpers of libmlkit_amd (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/mlkit_amd.h"

// Records the message returned by mk_last_error() and returns `code`.
int mk_fail(int code, const char *format, ...);

#define MK_REQUIRE(condition, code, ...)                 \
    do {                                                 \
        if (!(condition)) return mk_fail((code), __VA_ARGS__); \
    } while (0)

// Launch errors surface here: nothing is synchronised, only the launch status is read.
#define MK_LAUNCH_CHECK(name)                                                        \
    do {                                                                             \
        hipError_t status_ = hipGetLastError();                                      \
        if (status_ != hipSuccess)                                                   \
            return mk_fail(MK_ERR_HIP, "%s: %s", (name), hipGetErrorString(status_)); \
    } while (0)

static inline int mk_dtype_bytes(int dtype) { return dtype == MK_F32 ? 4 : 2; }
static inline bool mk_dtype_valid(int dtype) { return dtype >= MK_F32 && dtype <= MK_BF16; }
static inline int mk_cdiv(int a, int b) { return (a + b - 1) / b; }
static inline int mk_gcd(int a, int b) {
    while (b) {
        int t = a % b;
        a = b;
        b = t;
    }
    return a;
}

// Defined in scalar_codec.hip, also used by the error-feedback sweep (error_feedback.hip).
int mk_fit_scales_strided(const float *value, long long row_stride, float *scales, float *zeros,
                          long long out_row_stride, int rows, int span, int group, int asym, float reciprocal,
                          float value_minimum, int scale_format, int store_zero, hipStream_t stream);

#ifdef __HIPCC__

typedef uint32_t mk_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t mk_u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t mk_u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 mk_h2 __attribute__((ext_vector_type(2)));
typedef __bf16 mk_bf2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float mk_bf16_to_float(uint16_t bits) {
    return __uint_as_float(static_cast<uint32_t>(bits) << 16);
}

// Round-to-nearest-even fp32 -> bf16 bit pattern (NaN kept quiet).
__device__ __forceinline__ uint16_t mk_float_to_bf16(float value) {
    uint32_t bits = __float_as_uint(value);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((bits >> 16) | 0x40u);
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return static_cast<uint16_t>(bits >> 16);
}

// Element `index` of a buffer of MK_F32 / MK_F16 / MK_BF16 values, as fp32.
__device__ __forceinline__ float mk_load_as_float(const void *base, size_t index, int dtype) {
    if (dtype == MK_F32) return static_cast<const float *>(base)[index];
    const uint16_t raw = static_cast<const uint16_t *>(base)[index];
    if (dtype == MK_F16) return static_cast<float>(__builtin_bit_cast(_Float16, raw));
    return mk_bf16_to_float(raw);
}

// The same load split in two, branch-free, so that many can be in flight before any is
// used: the aligned dword holding the element is fetched from a 4-byte aligned buffer
// and the element is shifted out of it only when it is converted.
struct MkRaw {
    uint32_t word;
    uint32_t shift;
};

__device__ __forceinline__ MkRaw mk_load_raw(const void *aligned_base, size_t index, int dtype) {
    const size_t byte = index << (dtype == MK_F32 ? 2 : 1);
    MkRaw raw;
    raw.word = static_cast<const uint32_t *>(aligned_base)[byte >> 2];
    raw.shift = (static_cast<uint32_t>(byte) & 3u) * 8u;
    return raw;
}

__device__ __forceinline__ float mk_raw_to_float(MkRaw raw, int dtype) {
    const uint32_t bits = raw.word >> raw.shift;
    const float from_half = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits)));
    const float from_bits = __uint_as_float(dtype == MK_F32 ? bits : bits << 16);
    return dtype == MK_F16 ? from_half : from_bits;
}

__device__ __forceinline__ void mk_store_from_float(void *base, size_t index, int dtype, float value) {
    if (dtype == MK_F32) {
        static_cast<float *>(base)[index] = value;
    } else if (dtype == MK_F16) {
        static_cast<uint16_t *>(base)[index] =
            __builtin_bit_cast(uint16_t, static_cast<_Float16>(value));
    } else {
        static_cast<uint16_t *>(base)[index] = mk_float_to_bf16(value);
    }
}

// Sum over aligned groups of `SEG` lanes (a power of two up to 64); every lane of a
// group receives the group's sum.  Lanes of a 64-wide wavefront exchange values with
// DPP inside rows of 16 and with ds_bpermute across rows.
template <int SEG>
__device__ __forceinline__ float mk_segment_sum(float value) {
    if (SEG >= 2) value += __shfl_xor(value, 1, 64);
    if (SEG >= 4) value += __shfl_xor(value, 2, 64);
    if (SEG >= 8) value += __shfl_xor(value, 4, 64);
    if (SEG >= 16) value += __shfl_xor(value, 8, 64);
    if (SEG >= 32) value += __shfl_xor(value, 16, 64);
    if (SEG >= 64) value += __shfl_xor(value, 32, 64);
    return value;
}

// Storage rounding of a positive scale; format codes: 0 fp32, 1 fp16, 2 bf16, 3 fp8 e4m3,
// 4 e8m0 (power of two).
__device__ __forceinline__ float mk_rounded_scale(float value, int format) {
    if (format == 1) {
        const float clamped = fminf(fmaxf(value, 0x1p-24f), 65504.0f);
        return static_cast<float>(static_cast<_Float16>(clamped));
    }
    if (format == 2) return mk_bf16_to_float(mk_float_to_bf16(value));
    if (format == 3) {
        const float clamped = fminf(fmaxf(value, 0x1p-9f), 448.0f);
        const int exponent = static_cast<int>((__float_as_uint(clamped) >> 23) & 255u) - 127;
        const int quantum_exponent = (exponent > -6 ? exponent : -6) - 3;
        const float quantum = __uint_as_float(static_cast<uint32_t>(quantum_exponent + 127) << 23);
        const float reciprocal = __uint_as_float(static_cast<uint32_t>(127 - quantum_exponent) << 23);
        return __fmul_rn(rintf(__fmul_rn(clamped, reciprocal)), quantum);
    }
    if (format == 4) {
        // 2^round(log2 v) exactly: the mantissa m in [1, 2) rounds up iff m^2 > 2.
        const float clamped = fmaxf(value, 0x1p-126f);
        const uint32_t bits = __float_as_uint(clamped);
        int exponent = static_cast<int>((bits >> 23) & 255u) - 127;
        const uint64_t mantissa = (bits & 0x7fffffu) | 0x800000u;
        if (mantissa * mantissa > (2ull << 46)) ++exponent;
        if (value < 0x1p-126f) exponent = value > 0x1.6a09e6p-127f ? -126 : -127;
        exponent = exponent > 127 ? 127 : exponent;
        return ldexpf(1.0f, exponent);
    }
    return value;
}

#endif  // __HIPCC__
