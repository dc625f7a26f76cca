// Packed scalar-codec matrix-vector product for 1..8 input rows on gfx950: kernel templates.
//
// y[m, n] = sum_k dequant(code[n, k]) * x[m, k] (+ bias[n]),  fp32 accumulate.
//
// Streaming kernel (HBM bound, no matrix cores).  A lane owns up to C chunks of 32
// consecutive codes of a row (BITS dwords each, one coalesced 4*BITS-byte load); the
// matching 32 activations of every sample stay in registers for the life of the
// workgroup, so the only per-row traffic is the code stream itself plus one scale per
// chunk read from LDS, where the workgroup's scale tile is staged once as fp32.
// A row's lanes form a segment of the workgroup: a power of two up to 64 lanes, or a
// whole number of wavefronts.  Partial sums meet by a segment reduction inside the
// wavefront and, when a row spans several wavefronts, by a fixed-order sum through LDS,
// so results do not depend on scheduling.
//
// Rows of the weight whose width or scale groups are not multiples of 32 codes take
// the word-at-a-time kernel at the end of this file.
//
// Replaces the reference's Triton kernel `packed_matrix_vector`
// (kernels/packed_linear.py:107-173 in /root/reference/src/mlkit).

#pragma once
#include <cstddef>

#include <atomic>

#include "mk_common.h"

namespace mk_matvec {

constexpr int kChunkCodes = 32;
constexpr int kMaxTableEntries = 256;
#ifndef MK_MATVEC_AHEAD
#define MK_MATVEC_AHEAD 8
#endif

struct MatvecArgs {
    const void *x;
    const uint8_t *packed;
    const void *scales;
    const void *zeros;
    const float *values;
    const void *bias;
    void *y;
    int samples;
    int rows;
    int width;
    int group;
    int groups;
    int n_values;
    int scale_dtype;
    int bias_dtype;
    int seg_lanes;        // lanes (incl. idle ones) that share one row
    int rows_parallel;    // rows in flight per workgroup pass
    int chunks_per_row;   // width / 32
    int scale_row_offset; // row of `scales`/`zeros` that row 0 of this launch uses
    float grid_min;
    float grid_step;
};

// Arguments of the 4-bit streaming kernel (packed_matvec_stream4.hip).
struct Stream4Args {
    const void *x;        // fp16 [samples, width]
    const uint8_t *packed;
    const void *scales;   // fp16 [rows, groups]
    const void *zeros;    // fp16 [rows, groups] or null
    const void *bias;     // [rows] of bias_dtype, or null
    void *y;              // fp16 [samples, rows]
    int samples, rows, width, group, groups, bias_dtype;
    float grid_min, grid_step;
    const float *values;  // fp32 table (pair-table kernel, when uniform == 0)
    int n_values, uniform, bits;
    int x_dtype, scale_dtype;  // pair-table kernel: MK_F16 or MK_BF16 each
    // stream4_launch_rotating only: the activations are multiplied by rotate_signs (or not, when
    // null), Walsh-Hadamard transformed over the whole row and multiplied by rotate_scale inside
    // the kernel, before they meet the codes.
    const float *rotate_signs = nullptr;
    float rotate_scale = 1.0f;
    int rotate_log_block = 0;  // the transform spans blocks of 1 << rotate_log_block values (the whole row, or equal parts of it)
};
// Several weight matrices that share the activations, the row width and the codec, multiplied
// by one launch: the grid's z index selects the member, x walks that member's tiles of rows
// (workgroups past a shorter member's last tile leave at once).  count == 0: the single
// matrix described by Stream4Args.  The member is known from the workgroup's index alone, so
// its table entry is fetched together with the other arguments, not behind them.
constexpr int kMaxGroupMembers = 8;
struct Stream4Member {
    const void *x;  // this member's activations (members may share them)
    const uint8_t *packed;
    const void *scales, *zeros, *bias;
    void *y;
    int rows;   // output width of this member (row stride of y)
    int tiles;  // whole tiles of rows this launch multiplies
};
struct Stream4Group {
    int count, widest_tiles;
    Stream4Member member[kMaxGroupMembers];
};

// What a workgroup's matrix is: pointers, row count and number of tiles (wavefront-uniform).
struct TileSource {
    const void *x;
    const uint8_t *packed;
    const uint8_t *scales, *zeros;
    const void *bias;
    void *y;
    int rows, tiles;
};

// The kernels take (Stream4Args, Stream4Group) by value, i.e. in the kernel-argument segment,
// which is constant memory: member `member` of the table is read from there with one scalar
// load at a computed offset.  (Indexing the by-value parameter itself with a run-time index
// makes the compiler copy the whole table to scratch memory first.)
constexpr size_t kGroupTableOffset = (sizeof(Stream4Args) + alignof(Stream4Group) - 1) / alignof(Stream4Group) *
                                     alignof(Stream4Group);

template <int ROWS>
__device__ __forceinline__ TileSource tile_source(const Stream4Args &a, const Stream4Group &g, int member) {
    TileSource s{a.x, a.packed, static_cast<const uint8_t *>(a.scales), static_cast<const uint8_t *>(a.zeros), a.bias,
                 a.y, a.rows, a.rows / ROWS};
    if (g.count > 0) {
        typedef const Stream4Member __attribute__((address_space(4))) *ConstantMember;
        typedef const char __attribute__((address_space(4))) *ConstantBytes;
        const ConstantBytes segment = (ConstantBytes)__builtin_amdgcn_kernarg_segment_ptr();
        const ConstantMember chosen =
            reinterpret_cast<ConstantMember>(segment + kGroupTableOffset + offsetof(Stream4Group, member)) + member;
        s.x = chosen->x;
        s.packed = chosen->packed;
        s.scales = static_cast<const uint8_t *>(chosen->scales);
        s.zeros = static_cast<const uint8_t *>(chosen->zeros);
        s.bias = chosen->bias;
        s.y = chosen->y;
        s.rows = chosen->rows;
        s.tiles = chosen->tiles;
    }
    return s;
}

// The number of workgroups of `kernel` the GPU holds at once, asked of the runtime the first
// time and remembered per kernel (`known`).
template <typename Kernel>
inline int resident_workgroups(Kernel kernel, int threads, size_t dynamic_lds, std::atomic<int> &known) {
    int value = known.load(std::memory_order_relaxed);
    if (value == 0) {  // two threads asking at once both get the same answer
        int per_cu = 0, device = 0, units = 256;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, dynamic_lds) != hipSuccess || per_cu < 1)
            per_cu = 4;
        if (hipGetDevice(&device) == hipSuccess)
            (void)hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device);
        value = per_cu * units;
        known.store(value, std::memory_order_relaxed);
    }
    return value;
}

// Pair-table kernel (packed_matvec_pairs.hip): 2-, 3- and 4-bit codes of any scalar grid.
bool pairs_accepts(int width, int group, int bits, int x_dtype, int scale_dtype);
int pairs_launch(const Stream4Args &a, hipStream_t stream);
int pairs_launch_group(const Stream4Args &shared, Stream4Group &group, const int *member_rows, int *rows_per_tile,
                       hipStream_t stream);
bool stream4_accepts(int samples, int width, int group, int bits, int x_dtype, int scale_dtype, bool uniform);
int stream4_launch(const Stream4Args &a, hipStream_t stream);
// The whole four-row tiles of rows [first_row, rows) after a launch of taller tiles; returns the rows covered, or -1.
int stream4_launch_remainder(const Stream4Args &a, int first_row, hipStream_t stream);
// 4-bit uniform-grid codes in rows of 16416 to 32768 codes, and one or two samples of some shorter rows, fp16 or bf16
// activations (packed_matvec_long.hip: a wavefront owns two spans of 2048 codes):
// multiplies the leading whole tiles of rows and returns the number of rows covered, or -1.
bool long_accepts(int samples, int rows, int width, int group, int bits, int x_dtype, int scale_dtype, bool uniform);
int long_launch(const Stream4Args &a, hipStream_t stream);
bool long_group_accepts(const Stream4Args &shared, const Stream4Group &group, const int *member_rows);
int long_launch_group(const Stream4Args &shared, Stream4Group &group, const int *member_rows, int *rows_per_tile, hipStream_t stream);
// Three to eight samples of fp32 activations against 4-bit uniform-grid codes as integer matrix-core blocks
// (packed_matvec_digits.hip): `tiles` tiles of `rows_per_tile` rows of the single matrix or of every member.
bool digits_accepts(const Stream4Args &a, int rows_per_tile);
int digits_launch(const Stream4Args &a, const Stream4Group &members, int tiles, int rows_per_tile, hipStream_t stream);
// One sample of fp16 activations, a row of whole 2048-code slices made of power-of-two blocks
// (one block: a power-of-two row) and whole tiles of rows only: the kernel rotates the
// activations itself (see Stream4Args).  Returns 0 when
// launched, -1 when the runtime refused a launch attribute, -2 when the shape is not one of these.
int stream4_launch_rotating(const Stream4Args &a, hipStream_t stream);
// The same for a group (Stream4Args carries what the members share; its packed / scales /
// zeros / bias / y / rows are ignored).  `rows_per_tile` receives the tile height chosen for
// all members: rows beyond the last whole tile of a member are left to the caller.
int stream4_launch_group(const Stream4Args &shared, Stream4Group &group, const int *member_rows, int *rows_per_tile,
                         hipStream_t stream);

// ---------------------------------------------------------------------------------
// Activation registers.  XT: MK_F32 keeps 32 floats per chunk; MK_F16 / MK_BF16 keep
// 16 packed pairs.  `kPairs48` stores fp16 pairs as (x[i], x[i+4]) inside every group
// of eight codes, the order in which the 4-bit extraction below produces its pairs.
// ---------------------------------------------------------------------------------
template <int XT>
struct XChunk {
    uint32_t r[XT == MK_F32 ? 32 : 16];
};

template <int XT>
__device__ __forceinline__ float x_element(const XChunk<XT> &x, int k) {
    if constexpr (XT == MK_F32) {
        return __uint_as_float(x.r[k]);
    } else if constexpr (XT == MK_F16) {
        const mk_h2 pair = __builtin_bit_cast(mk_h2, x.r[k >> 1]);
        return static_cast<float>(pair[k & 1]);
    } else {
        const uint32_t word = x.r[k >> 1];
        return __uint_as_float((k & 1) ? (word & 0xffff0000u) : (word << 16));
    }
}

template <int XT>
__device__ __forceinline__ void load_x_chunk(XChunk<XT> &x, const void *base, size_t element) {
    constexpr int kWords = XT == MK_F32 ? 32 : 16;
    const mk_u32x4 *src = reinterpret_cast<const mk_u32x4 *>(
        static_cast<const uint8_t *>(base) + element * (XT == MK_F32 ? 4 : 2));
#pragma unroll
    for (int i = 0; i < kWords / 4; ++i) {
        const mk_u32x4 v = src[i];
        x.r[4 * i + 0] = v.x;
        x.r[4 * i + 1] = v.y;
        x.r[4 * i + 2] = v.z;
        x.r[4 * i + 3] = v.w;
    }
}

// Sum of the 32 activations of a chunk in fp32.
template <int XT>
__device__ __forceinline__ float chunk_sum(const XChunk<XT> &x) {
    float total = 0.0f;
    if constexpr (XT == MK_F16) {
        const mk_h2 ones = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
#pragma unroll
        for (int j = 0; j < 16; ++j)
            total = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(mk_h2, x.r[j]), total, false);
    } else {
#pragma unroll
        for (int k = 0; k < 32; ++k) total += x_element<XT>(x, k);
    }
    return total;
}

// (x0,x1)(x2,x3)(x4,x5)(x6,x7) -> (x0,x4) (x1,x5)/16 (x2,x6) (x3,x7)/16 for every eight
// codes: the pair order and scaling the 4-bit extraction of chunk_dot expects.  Returns
// what that extraction accumulates for all-zero codes, 1024 * sum(stored values); with
// `stored_sum`, also the sum of the activations as the dot products see them.
__device__ __forceinline__ float pair_for_nibbles(XChunk<MK_F16> &x, float *stored_sum = nullptr) {
    const mk_h2 sixteenth = {static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
    const mk_h2 ones = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
    auto scaled = [&](uint32_t pair) __attribute__((always_inline)) {
        return __builtin_bit_cast(uint32_t, __builtin_bit_cast(mk_h2, pair) * sixteenth);
    };
    // plain: sum of the activations kept as they are; reduced: sum of those kept at 1/16.
    float plain = 0.0f, reduced = 0.0f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t p0 = x.r[4 * g + 0], p1 = x.r[4 * g + 1];
        const uint32_t p2 = x.r[4 * g + 2], p3 = x.r[4 * g + 3];
        x.r[4 * g + 0] = __builtin_amdgcn_perm(p2, p0, 0x05040100u);
        x.r[4 * g + 1] = scaled(__builtin_amdgcn_perm(p2, p0, 0x07060302u));
        x.r[4 * g + 2] = __builtin_amdgcn_perm(p3, p1, 0x05040100u);
        x.r[4 * g + 3] = scaled(__builtin_amdgcn_perm(p3, p1, 0x07060302u));
        plain = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(mk_h2, x.r[4 * g + 0]), plain, false);
        reduced = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(mk_h2, x.r[4 * g + 1]), reduced, false);
        plain = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(mk_h2, x.r[4 * g + 2]), plain, false);
        reduced = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(mk_h2, x.r[4 * g + 3]), reduced, false);
    }
    // The sum the dot products effectively see: the 1/16 activations count sixteen-fold.
    if (stored_sum) *stored_sum = __builtin_fmaf(16.0f, reduced, plain);
    return 1024.0f * (plain + reduced);
}

// The same pairing without the factor 1/16: (x0,x4) (x1,x5) (x2,x6) (x3,x7) for every eight codes, for codes
// that enter as fp16 subnormals (chunk_dot_subnormal).  Returns the sum of the chunk's activations.
__device__ __forceinline__ float pair_for_subnormal_nibbles(XChunk<MK_F16> &x) {
    const mk_h2 ones = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
    float total = 0.0f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t p0 = x.r[4 * g + 0], p1 = x.r[4 * g + 1];
        const uint32_t p2 = x.r[4 * g + 2], p3 = x.r[4 * g + 3];
        x.r[4 * g + 0] = __builtin_amdgcn_perm(p2, p0, 0x05040100u);
        x.r[4 * g + 1] = __builtin_amdgcn_perm(p2, p0, 0x07060302u);
        x.r[4 * g + 2] = __builtin_amdgcn_perm(p3, p1, 0x05040100u);
        x.r[4 * g + 3] = __builtin_amdgcn_perm(p3, p1, 0x07060302u);
#pragma unroll
        for (int i = 0; i < 4; ++i) total = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(mk_h2, x.r[4 * g + i]), total, false);
    }
    return total;
}

// ---- activations: coalesced loads, then each lane's chunk out of LDS ------------------------
//
// A lane needs the 32 activations (64 bytes) of a chunk.  Sixty-four lanes reading 16 bytes
// at a stride of 64 touch 64 cache lines per instruction, and the compute unit's vector
// memory path takes them one line per cycle, ahead of the code stream.  Instead a wavefront
// reads the 4 KB of one sample's 2048-code slice as four 1 KB instructions (lane l: bytes
// 16 l), parks them in its own LDS buffer and reads chunks back.  Chunks are 80 bytes apart
// in LDS so that sixteen lanes reading 16 bytes of sixteen chunks hit different banks.

// The value of the lane whose index differs in bit 0 (XOR = 1) or bit 1 (XOR = 2): DPP quad permutations.
template <int XOR>
__device__ __forceinline__ float quad_value_of_lane(float value) {
    constexpr int control = XOR == 1 ? 0xB1 : 0x4E;   // quad_perm [1,0,3,2] / [2,3,0,1]
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, value), control, 0xf, 0xf, true));
}

constexpr int kChunkStrideWords = 20;
constexpr int kSliceWords = 64 * kChunkStrideWords;  // one wavefront's buffer: 5 KB

// Piece i of the slice that starts at element `slice_start` of x's row `sample`: 16 bytes per
// lane.  Pieces past the end of the row read the start of the row instead (their chunks are
// zeroed later).
__device__ __forceinline__ mk_u32x4 request_piece(const void *x, int width, int sample, int slice_start, int i, int lane) {
    const int element = slice_start + (16 * i + (lane >> 2)) * kChunkCodes + (lane & 3) * 8;
    const size_t offset = static_cast<size_t>(sample) * width + (element < width ? element : (lane & 3) * 8);
    return *reinterpret_cast<const mk_u32x4 *>(static_cast<const uint8_t *>(x) + offset * 2);
}

// The same eight elements of an fp32 row as two loads of four floats (`second`: elements 4 - 7).
__device__ __forceinline__ mk_u32x4 request_wide_piece(const void *x, int width, int sample, int slice_start, int i, int lane, int second) {
    const int element = slice_start + (16 * i + (lane >> 2)) * kChunkCodes + (lane & 3) * 8;
    const size_t offset = static_cast<size_t>(sample) * width + (element < width ? element : (lane & 3) * 8) + 4 * second;
    return *reinterpret_cast<const mk_u32x4 *>(static_cast<const uint8_t *>(x) + offset * 4);
}

// fp32 activations enter the dot products as integers: a chunk's 32 values are scaled by a power of two 2^k of
// the chunk's own (largest magnitude into [2^21, 2^22)), rounded to integers X and cut into six signed 4-bit
// digits, X = sum_d t_d 16^d with t_d in [-8, 7].  Plane d of a chunk is four words that hold digit d of its 32
// values in the nibble order of the packed codes, so that one v_dot8_i32_i4 multiplies eight codes (as c - 8, one
// XOR away from the packed word) by eight digits, exactly.  Six such instructions per eight codes replace eight
// v_dot2 and four masks of a split into two fp16 halves, and the only roundings left are the one to X (half a
// unit in 2^22 of the chunk's largest value) and those of the fp32 sums over the chunks.
constexpr int kPlaneDigits = 6;
constexpr int kPlaneStrideWords = 28;   // 24 plane words, 2^-k, the sum of the X; 112 bytes apart: eight lanes reading
                                        // 16 bytes of eight adjacent chunks touch every LDS bank once
constexpr int kPlaneSliceWords = 64 * kPlaneStrideWords;  // one wavefront's buffer: 7 KB

// Eight fp32 activations of a chunk (this lane's quarter of it; the four lanes of a quad hold the chunk): digit d
// of the eight in plane[d], their sum (of the integers X) in `total`; returns 2^-k.  Chunks of zeros keep k = 0,
// chunks below 2^-106 the largest usable k; a chunk with a value that is not finite returns NaN.
__device__ __forceinline__ float planes_of_piece(mk_u32x4 first, mk_u32x4 second, uint32_t (&plane)[kPlaneDigits], int &total) {
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
    // x 2^k + 1.5 * 2^23 holds X + 2^22 in its low 23 bits (rounded to nearest even); adding 8 to every digit makes
    // them unsigned nibbles, and flipping each nibble's top bit afterwards makes those two's complement again.
    constexpr uint32_t kEights = 0x888888u;
    uint32_t y[8];
    int sum = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        y[k] = __float_as_uint(__builtin_fmaf(__uint_as_float(bits[k]), factor, 12582912.0f)) + (kEights - 0x4B400000u);
        sum += static_cast<int>(y[k]);
    }
    total = sum - 8 * static_cast<int>(kEights);
    uint32_t even[4], odd[4];   // byte b of even[p]: digit 2 b of value 2 p (low nibble) and of value 2 p + 1 (high nibble)
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t a = y[2 * p], b = y[2 * p + 1];
        even[p] = (a & 0x0f0f0fu) | ((b & 0x0f0f0fu) << 4);
        odd[p] = ((a >> 4) & 0x0f0f0fu) | (b & 0xf0f0f0u);
    }
    auto gather = [](const uint32_t (&w)[4], uint32_t &d0, uint32_t &d1, uint32_t &d2) __attribute__((always_inline)) {
        const uint32_t t01 = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u);   // w0.b0 w1.b0 w0.b1 w1.b1
        const uint32_t t23 = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u);
        d0 = __builtin_amdgcn_perm(t23, t01, 0x05040100u) ^ 0x88888888u;
        d1 = __builtin_amdgcn_perm(t23, t01, 0x07060302u) ^ 0x88888888u;
        const uint32_t u01 = __builtin_amdgcn_perm(w[1], w[0], 0x0c0c0602u);   // w0.b2 w1.b2 0 0
        const uint32_t u23 = __builtin_amdgcn_perm(w[3], w[2], 0x0c0c0602u);
        d2 = __builtin_amdgcn_perm(u23, u01, 0x05040100u) ^ 0x88888888u;
    };
    gather(even, plane[0], plane[2], plane[4]);
    gather(odd, plane[1], plane[3], plane[5]);
    return inverse;
}

// Parks a piece's planes (and, from the quad's first lane, 2^-k and the chunk's sum) in the wavefront's buffer.
__device__ __forceinline__ void park_planes(uint32_t *slice, int i, int lane, const uint32_t (&plane)[kPlaneDigits], float inverse, int total) {
    uint32_t *const slot = slice + (16 * i + (lane >> 2)) * kPlaneStrideWords;
#pragma unroll
    for (int d = 0; d < kPlaneDigits; ++d) slot[4 * d + (lane & 3)] = plane[d];
    total += __builtin_amdgcn_mov_dpp(total, 0xB1, 0xf, 0xf, true);
    total += __builtin_amdgcn_mov_dpp(total, 0x4E, 0xf, 0xf, true);
    if ((lane & 3) == 0) {
        slot[24] = __float_as_uint(inverse);
        slot[25] = static_cast<uint32_t>(total);
    }
}

// A lane's chunk out of the buffer: planes[4 d + j] is digit d of code word j; masked by `keep`.
__device__ __forceinline__ void planes_from_slice(uint32_t (&planes)[4 * kPlaneDigits], float &inverse, float &sum,
                                                  const uint32_t *slice, int chunk_in_slice, uint32_t keep) {
    const uint32_t *const slot = slice + chunk_in_slice * kPlaneStrideWords;
#pragma unroll
    for (int d = 0; d < kPlaneDigits; ++d) {
        const mk_u32x4 v = *reinterpret_cast<const mk_u32x4 *>(slot + 4 * d);
        planes[4 * d + 0] = v.x & keep;
        planes[4 * d + 1] = v.y & keep;
        planes[4 * d + 2] = v.z & keep;
        planes[4 * d + 3] = v.w & keep;
    }
    const mk_u32x2 tail = *reinterpret_cast<const mk_u32x2 *>(slot + 24);
    inverse = __uint_as_float(tail.x);
    sum = static_cast<float>(static_cast<int>(tail.y & keep));
}

__device__ __forceinline__ void park_piece(uint32_t *slice, int i, int lane, mk_u32x4 piece) {
    *reinterpret_cast<mk_u32x4 *>(slice + (16 * i + (lane >> 2)) * kChunkStrideWords + (lane & 3) * 4) = piece;
}

// Between a wavefront's parking of pieces in its own LDS buffer and its lanes' reads of what OTHER lanes
// parked: the hardware completes a wavefront's LDS operations in order, and this pins the compiler to the
// same order (writes before the barrier, reads after it; wavefront scope, no wait beyond the LDS counter).
__device__ __forceinline__ void wave_exchange_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int XT>
__device__ __forceinline__ void chunk_from_slice(XChunk<XT> &x, const uint32_t *slice, int chunk_in_slice) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const mk_u32x4 v = *reinterpret_cast<const mk_u32x4 *>(slice + chunk_in_slice * kChunkStrideWords + 4 * i);
        x.r[4 * i + 0] = v.x;
        x.r[4 * i + 1] = v.y;
        x.r[4 * i + 2] = v.z;
        x.r[4 * i + 3] = v.w;
    }
}

// The matrix-core kernels park the slices of four samples side by side, unpadded: quarter q
// of chunk c sits at 16-byte granule 4 c + (q ^ ((c >> 2) & 3)), so that sixteen lanes reading
// one quarter of sixteen adjacent chunks still spread over all banks, and a sample's buffer
// is four words longer than its slices, which staggers the four samples.
constexpr int blocks_sample_words(int slices) {
    return slices * 16 * 16 + 4;
}

__device__ __forceinline__ void park_piece_swizzled(uint32_t *slice, int i, int lane, mk_u32x4 piece) {
    const int chunk = 16 * i + (lane >> 2), quarter = (lane & 3) ^ ((lane >> 4) & 3);
    *reinterpret_cast<mk_u32x4 *>(slice + chunk * 16 + quarter * 4) = piece;
}

template <int XT>
__device__ __forceinline__ void chunk_from_swizzled_slice(XChunk<XT> &x, const uint32_t *slice, int chunk_in_slice) {
    const int turn = (chunk_in_slice >> 2) & 3;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const mk_u32x4 v = *reinterpret_cast<const mk_u32x4 *>(slice + chunk_in_slice * 16 + (i ^ turn) * 4);
        x.r[4 * i + 0] = v.x;
        x.r[4 * i + 1] = v.y;
        x.r[4 * i + 2] = v.z;
        x.r[4 * i + 3] = v.w;
    }
}

// A 16-bit scale or offset as fp32; `dtype` (MK_F16 or MK_BF16) is uniform per launch.
__device__ __forceinline__ float side_as_float(uint16_t raw, int dtype) {
    const float from_half = static_cast<float>(__builtin_bit_cast(_Float16, raw));
    const float from_brain = __uint_as_float(static_cast<uint32_t>(raw) << 16);
    return dtype == MK_F16 ? from_half : from_brain;
}

template <int XT>
__device__ __forceinline__ void store_output(void *y, size_t index, float value) {
    if constexpr (XT == MK_F16) static_cast<_Float16 *>(y)[index] = static_cast<_Float16>(value);
    else static_cast<uint16_t *>(y)[index] = mk_float_to_bf16(value);
}

typedef _Float16 mk_h4 __attribute__((ext_vector_type(4)));
typedef short mk_s4 __attribute__((ext_vector_type(4)));
typedef float mk_f4 __attribute__((ext_vector_type(4)));

// The value lane R of this lane's quad holds (a DPP quad broadcast).
template <int R>
__device__ __forceinline__ float quad_value(float value) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, value), R * 0x55, 0xf, 0xf, true));
}

// ---------------------------------------------------------------------------------
// Code chunks: BITS dwords hold 32 codes.
// ---------------------------------------------------------------------------------
template <int BITS>
struct CodeChunk {
    uint32_t w[BITS];
};

template <int BITS>
__device__ __forceinline__ void load_codes(CodeChunk<BITS> &c, const uint8_t *address) {
    // `address` is 4-byte aligned; wide loads need no more than that on gfx9.
    typedef uint32_t u1 __attribute__((aligned(4)));
    typedef mk_u32x2 u2 __attribute__((aligned(4)));
    typedef mk_u32x3 u3 __attribute__((aligned(4)));
    typedef mk_u32x4 u4 __attribute__((aligned(4)));
    if constexpr (BITS == 1) {
        c.w[0] = __builtin_nontemporal_load(reinterpret_cast<const u1 *>(address));
    } else if constexpr (BITS == 2) {
        const mk_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u2 *>(address));
        c.w[0] = v.x; c.w[1] = v.y;
    } else if constexpr (BITS == 3) {
        const mk_u32x3 v = __builtin_nontemporal_load(reinterpret_cast<const u3 *>(address));
        c.w[0] = v.x; c.w[1] = v.y; c.w[2] = v.z;
    } else {
        const mk_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(address));
        c.w[0] = v.x; c.w[1] = v.y; c.w[2] = v.z; c.w[3] = v.w;
        if constexpr (BITS == 5) {
            c.w[4] = __builtin_nontemporal_load(reinterpret_cast<const u1 *>(address + 16));
        } else if constexpr (BITS == 6) {
            const mk_u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u2 *>(address + 16));
            c.w[4] = t.x; c.w[5] = t.y;
        } else if constexpr (BITS == 7) {
            const mk_u32x3 t = __builtin_nontemporal_load(reinterpret_cast<const u3 *>(address + 16));
            c.w[4] = t.x; c.w[5] = t.y; c.w[6] = t.z;
        } else if constexpr (BITS == 8) {
            const mk_u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(address + 16));
            c.w[4] = t.x; c.w[5] = t.y; c.w[6] = t.z; c.w[7] = t.w;
        }
    }
}

// Code k (0..31) of a chunk; k is a compile-time constant after unrolling, so this is
// one bit-field extract, or a funnel shift and a mask when the code crosses a dword.
template <int BITS>
__device__ __forceinline__ uint32_t code_at(const CodeChunk<BITS> &c, int k) {
    const int bit = k * BITS;
    const int word = bit >> 5, shift = bit & 31;
    constexpr uint32_t mask = (1u << BITS) - 1u;
    if (shift + BITS <= 32) return (c.w[word] >> shift) & mask;
    return __builtin_amdgcn_alignbit(c.w[(word + 1) % BITS], c.w[word], shift) & mask;
}

// sum_k T[code_k] * x_k for one chunk and MT samples; T = identity (uniform grids,
// the affine map is applied once per chunk by the caller) or the LDS table.
template <int BITS, int XT, int MT, bool UNIFORM>
__device__ __forceinline__ void chunk_dot(const CodeChunk<BITS> &codes, const XChunk<XT> (&x)[MT],
                                          const float *table, float (&dot)[MT]) {
#pragma unroll
    for (int m = 0; m < MT; ++m) dot[m] = 0.0f;
    if constexpr (BITS == 4 && XT == MK_F16 && UNIFORM) {
        // Two codes at a time.  v_bfi_b32 drops a nibble into the mantissa of both halves
        // of the fp16 pair (1024, 1024): bits 0..3 give 1024 + c, bits 4..7 give
        // 1024 + 16 c (those activations were pre-scaled by 1/16).  Each product is exact
        // in fp32 and v_dot2_f32_f16 accumulates in fp32; the caller subtracts the
        // code-independent part, 1024 * sum(stored activations), once per chunk.
        // (word & mask) | (magic & ~mask) is one v_bfi_b32; `magic` is kept opaque so the
        // second term is not folded into a constant.
        uint32_t magic = 0x64006400u;
        asm volatile("" : "+v"(magic));
        auto insert = [&](uint32_t mask, uint32_t word) __attribute__((always_inline)) {
            return __builtin_bit_cast(mk_h2, (word & mask) | (magic & ~mask));
        };
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = codes.w[i];
            const uint32_t w8 = w >> 8;
            const mk_h2 h0 = insert(0x000f000fu, w);   // codes 0 and 4
            const mk_h2 h1 = insert(0x00f000f0u, w);   // codes 1 and 5 (x16)
            const mk_h2 h2 = insert(0x000f000fu, w8);  // codes 2 and 6
            const mk_h2 h3 = insert(0x00f000f0u, w8);  // codes 3 and 7 (x16)
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float d = dot[m];
                d = __builtin_amdgcn_fdot2(h0, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 0]), d, false);
                d = __builtin_amdgcn_fdot2(h1, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 1]), d, false);
                d = __builtin_amdgcn_fdot2(h2, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 2]), d, false);
                d = __builtin_amdgcn_fdot2(h3, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 3]), d, false);
                dot[m] = d;
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const uint32_t code = code_at<BITS>(codes, k);
            float value;
            if constexpr (UNIFORM) {
                value = static_cast<float>(code);
            } else {
                value = table[code];
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) dot[m] = __builtin_fmaf(value, x_element<XT>(x[m], k), dot[m]);
        }
    }
}

// sum_k code_k x_k of a chunk of 4-bit codes for MT samples, times 2^-24.  A nibble left where it is in the low
// bits of a half word is the fp16 subnormal c * 2^-24 (16 c * 2^-24 for the upper nibble of a byte), which
// v_dot2_f32_f16 multiplies exactly: no exponent is inserted, nothing code-free has to be removed afterwards and
// the activations are used as they are.  The upper nibbles have their own sum, divided by 16 at the end.
template <int MT>
__device__ __forceinline__ void chunk_dot_subnormal(const CodeChunk<4> &codes, const XChunk<MK_F16> (&x)[MT], float (&dot)[MT]) {
    float lower[MT], upper[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) lower[m] = upper[m] = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w = codes.w[i], w8 = w >> 8;
        const mk_h2 h0 = __builtin_bit_cast(mk_h2, w & 0x000f000fu), h1 = __builtin_bit_cast(mk_h2, w & 0x00f000f0u);
        const mk_h2 h2 = __builtin_bit_cast(mk_h2, w8 & 0x000f000fu), h3 = __builtin_bit_cast(mk_h2, w8 & 0x00f000f0u);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            lower[m] = __builtin_amdgcn_fdot2(h0, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 0]), lower[m], false);
            upper[m] = __builtin_amdgcn_fdot2(h1, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 1]), upper[m], false);
            lower[m] = __builtin_amdgcn_fdot2(h2, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 2]), lower[m], false);
            upper[m] = __builtin_amdgcn_fdot2(h3, __builtin_bit_cast(mk_h2, x[m].r[4 * i + 3]), upper[m], false);
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) dot[m] = __builtin_fmaf(upper[m], 0.0625f, lower[m]);
}

// ---- bf16 activations ----------------------------------------------------------------------
//
// bf16 has seven mantissa bits, so only the low nibble of each half fits the magic-number
// insertion (128 + c); every pair of codes needs its own shift: 3 shifts, 4 v_bfi and 4
// v_dot2_f32_bf16 per eight codes, against 1 + 4 + 4 for fp16.  Pairs are (x0,x4) (x1,x5)
// (x2,x6) (x3,x7) of every eight codes, unscaled.

// Re-pairs a chunk in place; returns the sum of its activations.
__device__ __forceinline__ float pair_for_nibbles_bf16(XChunk<MK_BF16> &x) {
    const uint32_t ones = 0x3f803f80u;
    float total = 0.0f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t p0 = x.r[4 * g + 0], p1 = x.r[4 * g + 1];
        const uint32_t p2 = x.r[4 * g + 2], p3 = x.r[4 * g + 3];
        x.r[4 * g + 0] = __builtin_amdgcn_perm(p2, p0, 0x05040100u);
        x.r[4 * g + 1] = __builtin_amdgcn_perm(p2, p0, 0x07060302u);
        x.r[4 * g + 2] = __builtin_amdgcn_perm(p3, p1, 0x05040100u);
        x.r[4 * g + 3] = __builtin_amdgcn_perm(p3, p1, 0x07060302u);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            total = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(mk_bf2, ones), __builtin_bit_cast(mk_bf2, x.r[4 * g + i]), total, false);
    }
    return total;
}

// sum over the chunk of (128 + code_k) x_k for MT samples.
template <int MT>
__device__ __forceinline__ void chunk_dot_bf16(const CodeChunk<4> &codes, const XChunk<MK_BF16> (&x)[MT], float (&dot)[MT]) {
#pragma unroll
    for (int m = 0; m < MT; ++m) dot[m] = 0.0f;
    uint32_t magic = 0x43004300u;
    asm volatile("" : "+v"(magic));
    auto insert = [&](uint32_t word) __attribute__((always_inline)) {
        return __builtin_bit_cast(mk_bf2, (word & 0x000f000fu) | (magic & ~0x000f000fu));
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w = codes.w[i];
        const mk_bf2 h0 = insert(w), h1 = insert(w >> 4), h2 = insert(w >> 8), h3 = insert(w >> 12);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float d = dot[m];
            d = __builtin_amdgcn_fdot2_f32_bf16(h0, __builtin_bit_cast(mk_bf2, x[m].r[4 * i + 0]), d, false);
            d = __builtin_amdgcn_fdot2_f32_bf16(h1, __builtin_bit_cast(mk_bf2, x[m].r[4 * i + 1]), d, false);
            d = __builtin_amdgcn_fdot2_f32_bf16(h2, __builtin_bit_cast(mk_bf2, x[m].r[4 * i + 2]), d, false);
            d = __builtin_amdgcn_fdot2_f32_bf16(h3, __builtin_bit_cast(mk_bf2, x[m].r[4 * i + 3]), d, false);
            dot[m] = d;
        }
    }
}

// A chunk of 32 codes against the digit planes of MT fp32 samples (planes_of_piece): sum_k (c_k - 8) X_k, exact
// in integers and rounded once on its way to fp32.  (Codes as fp16 subnormals would not do for fp32 outputs:
// v_dot2_f32_f16 aligns its terms by the exponent FIELDS of its inputs and keeps about 24 bits below the largest,
// so a subnormal code, whose value lies far below its field's 2^-14, costs the running sum up to ten low bits.)
template <int MT>
__device__ __forceinline__ void chunk_dot_planes(const CodeChunk<4> &codes, const uint32_t (&planes)[MT][4 * kPlaneDigits], float (&dot)[MT]) {
    int signed_codes[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) signed_codes[j] = static_cast<int>(codes.w[j] ^ 0x88888888u);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        int digit_sum[kPlaneDigits];
#pragma unroll
        for (int d = 0; d < kPlaneDigits; ++d) {
            // the first of a chain in the three-operand form with a literal zero (the builtin's two-operand form
            // wants its accumulator cleared by a move of its own)
            asm("v_dot8_i32_i4 %0, %1, %2, 0" : "=v"(digit_sum[d]) : "v"(signed_codes[0]), "v"(planes[m][4 * d]));
#pragma unroll
            for (int j = 1; j < 4; ++j)
                digit_sum[d] = __builtin_amdgcn_sdot8(signed_codes[j], static_cast<int>(planes[m][4 * d + j]), digit_sum[d], false);
        }
        // |digit sum| <= 32 * 64: three of them combine within 20 bits (two shift-and-adds each)
        auto sixteen_times_plus = [](int upper, int lower) __attribute__((always_inline)) {
            int result;   // (spelled out: the compiler turns the two-step form into three shifts and a three-way add)
            asm("v_lshl_add_u32 %0, %1, 4, %2" : "=v"(result) : "v"(upper), "v"(lower));
            return result;
        };
        const int low = sixteen_times_plus(sixteen_times_plus(digit_sum[2], digit_sum[1]), digit_sum[0]);
        const int high = sixteen_times_plus(sixteen_times_plus(digit_sum[5], digit_sum[4]), digit_sum[3]);
        dot[m] = __builtin_fmaf(static_cast<float>(high), 4096.0f, static_cast<float>(low));
    }
}

// A thread owns kThreadRows rows of its workgroup's tile; they are finished in groups of
// group_rows<MT>() rows (at most 8 row sums per thread and group) while the code stream
// runs rows_ahead() rows in front.
constexpr int kThreadRows = 16;

template <int MT>
constexpr int group_rows() {
    return MT >= 8 ? 1 : (MT == 4 ? 2 : 4);
}

template <int BITS, int C>
constexpr int rows_ahead() {
    return 64 / (C * BITS) >= 8 ? 8 : 4;
}

// Element `index` (counted from `base`, a uniform address) of a 2- or 4-byte typed
// buffer, fetched as the aligned dword that holds it; convert with mk_raw_to_float.
__device__ __forceinline__ MkRaw load_raw_near(const uint8_t *base, uint32_t index, int dtype) {
    const uint32_t misalignment = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(base)) & 3u;
    const uint32_t byte = misalignment + (index << (dtype == MK_F32 ? 2 : 1));
    MkRaw raw;
    raw.word = reinterpret_cast<const uint32_t *>(base - misalignment)[byte >> 2];
    raw.shift = (byte & 3u) * 8u;
    return raw;
}

// The value lane `lane ^ (1 << STAGE)` holds, by vector-ALU lane moves only (DPP inside
// rows of 16 lanes, v_permlane16_swap / v_permlane32_swap across rows).
template <int STAGE>
__device__ __forceinline__ float lane_exchange(float value, int lane) {
    const int bits = __builtin_bit_cast(int, value);
    int moved;
    if constexpr (STAGE == 0) {
        moved = __builtin_amdgcn_mov_dpp(bits, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
    } else if constexpr (STAGE == 1) {
        moved = __builtin_amdgcn_mov_dpp(bits, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
    } else if constexpr (STAGE == 2) {
        // lanes 0-3 and 8-11 of a row read four lanes up, lanes 4-7 and 12-15 four lanes down
        moved = __builtin_amdgcn_update_dpp(bits, bits, 0x104, 0xf, 0x5, false);   // row_shl:4
        moved = __builtin_amdgcn_update_dpp(moved, bits, 0x114, 0xf, 0xa, false);  // row_shr:4
    } else if constexpr (STAGE == 3) {
        moved = __builtin_amdgcn_mov_dpp(bits, 0x128, 0xf, 0xf, true);  // row_ror:8
    } else if constexpr (STAGE == 4) {
        const auto swapped = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
        moved = (lane & 16) ? swapped[0] : swapped[1];
    } else {
        const auto swapped = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
        moved = (lane & 32) ? swapped[0] : swapped[1];
    }
    return __builtin_bit_cast(float, moved);
}

// Sums each of V per-lane values over the 64 lanes of a wavefront.  While more than one
// value is left, every stage halves them: the lane whose bit STAGE is clear keeps the
// lower half and receives its partner's lower half, the other lane the upper half.  On
// return v[0] of lane L is the total of value number
//     sum over s < log2(V) of bit_s(L) * (V >> (s + 1)).
// END < 6 sums over groups of 2^END lanes only (lane bits END and above keep apart).
template <int V, int STAGE = 0, int END = 6>
__device__ __forceinline__ void transposed_wave_sum(float (&v)[V], int lane) {
    if constexpr (STAGE < END) {
        if constexpr (V > 1) {
            constexpr int H = V / 2;
            const bool upper = (lane >> STAGE) & 1;
            float next[H];
#pragma unroll
            for (int j = 0; j < H; ++j) {
                const float keep = upper ? v[j + H] : v[j];
                const float send = upper ? v[j] : v[j + H];
                next[j] = keep + lane_exchange<STAGE>(send, lane);
            }
            transposed_wave_sum<H, STAGE + 1, END>(next, lane);
            v[0] = next[0];
        } else {
            v[0] += lane_exchange<STAGE>(v[0], lane);
            transposed_wave_sum<1, STAGE + 1, END>(v, lane);
        }
    }
}

template <int V>
__device__ __forceinline__ int transposed_value_of_lane(int lane) {
    int value = 0;
#pragma unroll
    for (int s = 0; (V >> (s + 1)) > 0; ++s) value += ((lane >> s) & 1) * (V >> (s + 1));
    return value;
}

// Sum over aligned groups of 32 lanes by DPP adds; valid in the LAST lane of each group
// (for `lanes` < 32, a power of two: in the last lane of each group of `lanes`).
__device__ __forceinline__ float dpp_group_sum(float v, int lanes) {
#define MK_DPP_ADD(ctrl, row_mask)                                                               \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, \
                                                               row_mask, 0xf, true))
    if (lanes >= 2) MK_DPP_ADD(0xB1, 0xf);    // quad_perm [1,0,3,2]
    if (lanes >= 4) MK_DPP_ADD(0x4E, 0xf);    // quad_perm [2,3,0,1]
    if (lanes >= 8) MK_DPP_ADD(0x141, 0xf);   // row_half_mirror
    if (lanes >= 16) MK_DPP_ADD(0x140, 0xf);  // row_mirror
    if (lanes >= 32) MK_DPP_ADD(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
#undef MK_DPP_ADD
    return v;
}

// One workgroup multiplies a tile of rows_parallel * kThreadRows adjacent rows.  The grid
// covers whole tiles only (rows left over go to the word kernel), so a row's address is a
// uniform base plus a per-lane constant and the streaming part has no branches at all.
//
// Timeline of a wavefront: align with the workgroup; request activations, scales and the
// first rows_ahead() rows of codes; then, for each group of rows: wait for a row,
// accumulate its unscaled dot products, request the row rows_ahead() further on; apply
// the scales and put the per-lane sums in LDS.  After a barrier a few threads add up the
// lanes of each row and store the outputs while the other wavefronts are already summing
// the next rows.  Only the last group's sums are not hidden behind the stream.
template <int BITS, int XT, int MT, int C, bool UNIFORM>
__global__ void __launch_bounds__(512) packed_matvec_kernel(const MatvecArgs a) {
    extern __shared__ float lds[];
    constexpr int kRows = kThreadRows;
    constexpr int kGroupRows = group_rows<MT>();
    constexpr int kGroups = kRows / kGroupRows;
    constexpr int kSums = kGroupRows * MT;  // row sums per thread and group
    constexpr int kAhead = rows_ahead<BITS, C>();
    constexpr bool kNibblePairs = (BITS == 4 && XT == MK_F16 && UNIFORM);

    const int tid = threadIdx.x;
    const int threads = blockDim.x;
    const int seg = a.seg_lanes;
    const int row_phase = a.rows_parallel == 1 ? 0 : tid / seg;
    const int lane_in_row = a.rows_parallel == 1 ? tid : tid - row_phase * seg;
    const int tile_rows = a.rows_parallel * kRows;
    const int row_base = blockIdx.x * tile_rows;
    const int sample_base = blockIdx.y * MT;
    const bool has_zero = a.zeros != nullptr;
    const uint32_t row_bytes = static_cast<uint32_t>(a.chunks_per_row) * (4 * BITS);
    const uint8_t *tile_codes = a.packed + static_cast<size_t>(row_base) * row_bytes;
    const uint32_t pass_stride = static_cast<uint32_t>(a.rows_parallel) * row_bytes;

    // Lanes past the end of a row read chunk 0 and multiply it by zero activations.
    bool chunk_active[C];
    uint32_t lane_offset[C];
    int slot_of[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int chunk = lane_in_row + c * seg;
        chunk_active[c] = chunk < a.chunks_per_row;
        const int safe_chunk = chunk_active[c] ? chunk : 0;
        lane_offset[c] = static_cast<uint32_t>(row_phase) * row_bytes + static_cast<uint32_t>(safe_chunk) * (4 * BITS);
        slot_of[c] = row_phase * a.groups + (safe_chunk * kChunkCodes) / a.group;
    }

    // LDS: [value table][scale tile][zero tile][bias tile][two buffers of per-lane row
    // sums, sums[value][thread]]; the tiles are padded so staging needs no bounds checks.
    constexpr int kStaged = 4;
    const int slot_count = tile_rows * a.groups;
    const int tile_slots = slot_count > kStaged * threads ? slot_count : kStaged * threads;
    float *table = lds;
    float *scale_tile = table + (UNIFORM ? 0 : kMaxTableEntries);
    float *zero_tile = scale_tile + tile_slots;
    float *bias_tile = zero_tile + tile_slots;  // [max(tile_rows, threads)]
    float *lane_sums = bias_tile + (tile_rows > threads ? tile_rows : threads);

    // A compute unit serves its wavefronts' loads first come, first served, and a
    // wavefront receives its loads in issue order.  So the workgroup is aligned first,
    // then every wavefront issues its few small loads and only then the code stream.
    // Everything up to the stream is unconditional straight-line code: a load whose only
    // use sits in a branch would be moved into that branch, behind the stream.
    __syncthreads();

    // Activations of this lane's chunks, resident for the whole workgroup (L2 hits).
    XChunk<XT> x[C][MT];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int chunk = lane_in_row + c * seg;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int sample = sample_base + m;
            const int safe_sample = sample < a.samples ? sample : a.samples - 1;
            load_x_chunk<XT>(x[c][m], a.x,
                             static_cast<size_t>(safe_sample) * a.width +
                                 static_cast<size_t>(chunk_active[c] ? chunk : 0) * kChunkCodes);
        }
    }
    // Scales, offsets, bias and table entries (first touch, from HBM): only needed once
    // the first group of rows is summed, so they queue behind the activations.
    const int scale_bytes = a.scale_dtype == MK_F32 ? 4 : 2;
    const size_t first_slot_byte = static_cast<size_t>(a.scale_row_offset + row_base) * a.groups * scale_bytes;
    const uint8_t *scale_base = static_cast<const uint8_t *>(a.scales) + first_slot_byte;
    const uint8_t *zero_base = has_zero ? static_cast<const uint8_t *>(a.zeros) + first_slot_byte : scale_base;
    MkRaw staged_scale[kStaged], staged_zero[kStaged];
#pragma unroll
    for (int j = 0; j < kStaged; ++j) {
        const int i = tid + j * threads;
        const uint32_t slot = i < slot_count ? i : 0;
        staged_scale[j] = load_raw_near(scale_base, slot, a.scale_dtype);
        staged_zero[j] = load_raw_near(zero_base, slot, a.scale_dtype);
    }
    const int bias_dtype = a.bias ? a.bias_dtype : a.scale_dtype;
    const uint8_t *bias_base =
        a.bias ? static_cast<const uint8_t *>(a.bias) +
                     static_cast<size_t>(a.scale_row_offset + row_base) * (bias_dtype == MK_F32 ? 4 : 2)
               : scale_base;
    const MkRaw staged_bias = load_raw_near(bias_base, a.bias && tid < tile_rows ? tid : 0, bias_dtype);
    float staged_table[UNIFORM ? 1 : kStaged];
    if constexpr (!UNIFORM) {
#pragma unroll
        for (int j = 0; j < kStaged; ++j) {
            const int i = tid + j * threads;
            staged_table[j] = a.values[i < a.n_values ? i : a.n_values - 1];
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // The code stream starts kAhead rows deep; each row summed below requests the next.
    CodeChunk<BITS> codes[kRows][C];
    auto issue_row = [&](int r) __attribute__((always_inline)) {
        const uint8_t *pass_codes = tile_codes + static_cast<size_t>(r) * pass_stride;
#pragma unroll
        for (int c = 0; c < C; ++c) load_codes<BITS>(codes[r][c], pass_codes + lane_offset[c]);
    };
#pragma unroll
    for (int r = 0; r < kAhead; ++r) {
        issue_row(r);
        __builtin_amdgcn_sched_barrier(0);  // in row order
    }

    // Per-chunk constants of the affine grid map: sum_k (min + step c_k) x_k
    //   = step * dot + min * sum(x)   (minus step * the code-free part of dot on the nibble path).
    float x_sum[C][MT];
    float grid_term[C][MT];
#pragma unroll
    for (int c = 0; c < C; ++c) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const uint32_t keep = (chunk_active[c] && sample_base + m < a.samples) ? 0xffffffffu : 0u;
#pragma unroll
            for (int i = 0; i < (XT == MK_F32 ? 32 : 16); ++i) x[c][m].r[i] &= keep;
            x_sum[c][m] = chunk_sum<XT>(x[c][m]);
            if constexpr (kNibblePairs) {
                const float code_free = pair_for_nibbles(x[c][m]);
                grid_term[c][m] = a.grid_min * x_sum[c][m] - a.grid_step * code_free;
            } else {
                grid_term[c][m] = a.grid_min * x_sum[c][m];
            }
        }
    }
    if constexpr (!UNIFORM) {
        // The table is needed by the stream itself (a short wait: requested before the codes).
#pragma unroll
        for (int j = 0; j < kStaged; ++j) {
            const int i = tid + j * threads;
            table[i < kMaxTableEntries ? i : kMaxTableEntries - 1] = staged_table[j];
        }
        for (int i = tid + kStaged * threads; i < kMaxTableEntries; i += threads)
            table[i] = a.values[i < a.n_values ? i : a.n_values - 1];
        __syncthreads();
    }

    // Who adds up the lanes of a row: `team` consecutive threads per output, each summing
    // every team-th lane of the row, then a DPP sum inside the team.
    const int team = seg < 32 ? seg : 32;                    // a power of two
    const int team_shift = 31 - __builtin_clz(team);
    const int phase_shift = 31 - __builtin_clz(a.rows_parallel);  // rows_parallel is a power of two
    const int group_outputs = a.rows_parallel * kSums;  // (row in group, phase, sample)
    const int pass_slots = a.rows_parallel * a.groups;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) {
        // The stream: unscaled dot products, row by row as the codes arrive.
        float dots[kGroupRows][C][MT];
#pragma unroll
        for (int j = 0; j < kGroupRows; ++j) {
            const int r = g * kGroupRows + j;
#pragma unroll
            for (int c = 0; c < C; ++c) chunk_dot<BITS, XT, MT, UNIFORM>(codes[r][c], x[c], table, dots[j][c]);
            if (r + kAhead < kRows) issue_row(r + kAhead);
            // Keeps the rows in arrival order and their temporaries short-lived.
            __builtin_amdgcn_sched_barrier(0);
        }

        if (g == 0) {
            // Scales, offsets and bias go through LDS as fp32 (they arrived long ago).  The
            // empty asm pins their first use here, so no wait for them moves above the stream.
#pragma unroll
            for (int j = 0; j < kStaged; ++j) {
                asm volatile("" : "+v"(staged_scale[j].word), "+v"(staged_zero[j].word));
                const int i = tid + j * threads;
                scale_tile[i] = mk_raw_to_float(staged_scale[j], a.scale_dtype);
                zero_tile[i] = has_zero ? mk_raw_to_float(staged_zero[j], a.scale_dtype) : 0.0f;
            }
            for (int i = tid + kStaged * threads; i < slot_count; i += threads) {
                scale_tile[i] = mk_load_as_float(scale_base, i, a.scale_dtype);
                zero_tile[i] = has_zero ? mk_load_as_float(zero_base, i, a.scale_dtype) : 0.0f;
            }
            bias_tile[tid] = a.bias ? mk_raw_to_float(staged_bias, bias_dtype) : 0.0f;
            for (int i = tid + threads; i < tile_rows; i += threads)
                bias_tile[i] = a.bias ? mk_load_as_float(bias_base, i, bias_dtype) : 0.0f;
            __syncthreads();
        }

        // Scaled per-lane sums into LDS: buffer[(j * MT + m) * threads + tid].
        float *buffer = lane_sums + (g & 1) * (kSums * threads);
#pragma unroll
        for (int j = 0; j < kGroupRows; ++j) {
            const int r = g * kGroupRows + j;
            float acc[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[m] = 0.0f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float scale = scale_tile[r * pass_slots + slot_of[c]];
                const float zero = zero_tile[r * pass_slots + slot_of[c]];
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    float value = dots[j][c][m];
                    if constexpr (UNIFORM) value = __builtin_fmaf(a.grid_step, value, grid_term[c][m]);
                    acc[m] = __builtin_fmaf(scale, value, acc[m]);
                    acc[m] = __builtin_fmaf(zero, x_sum[c][m], acc[m]);
                }
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) buffer[(j * MT + m) * threads + tid] = acc[m];
        }
        // After this barrier the group's sums are complete; the buffer is written again
        // two groups later, behind the next barrier, so its readers below are done by then.
        __syncthreads();

        // Output o = (j * MT + m) * rows_parallel + phase: its lanes are threads
        // phase * seg .. phase * seg + seg - 1 of value (j * MT + m).
        for (int t = tid; t < group_outputs * team; t += threads) {
            const int output = t >> team_shift, part = t & (team - 1);
            const int value = output >> phase_shift, phase = output & (a.rows_parallel - 1);
            const float *in = buffer + value * threads + phase * seg;
            float total = 0.0f;
#pragma unroll
            for (int k = 0; k < 16; ++k) {  // seg <= 512 = 16 * 32
                const int lane_k = part + k * team;
                const float term = in[lane_k < seg ? lane_k : seg - 1];
                total += lane_k < seg ? term : 0.0f;
            }
            total = dpp_group_sum(total, team);
            if (part == team - 1) {
                const int j = value / MT, m = value - j * MT;
                const int local = (g * kGroupRows + j) * a.rows_parallel + phase;
                const int sample = sample_base + m;
                if (sample < a.samples)
                    mk_store_from_float(a.y, static_cast<size_t>(sample) * a.rows + row_base + local, XT,
                                        total + bias_tile[local]);
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// Launch of one instantiation chosen by the host-side plan.
// ---------------------------------------------------------------------------------
struct Plan {
    int sample_tile;  // MT
    int chunks;       // C
    int seg_lanes;
    int rows_parallel;
    int rows_per_thread;
    int threads;
    int grid_x;
    size_t lds_bytes;
};

template <int BITS, int XT, int MT, int C, bool UNIFORM>
void launch_chunked(const MatvecArgs &a, const Plan &p, hipStream_t stream) {
    dim3 grid(p.grid_x, mk_cdiv(a.samples, MT));
    hipLaunchKernelGGL((packed_matvec_kernel<BITS, XT, MT, C, UNIFORM>), grid, dim3(p.threads),
                       p.lds_bytes, stream, a);
}

template <int BITS, int XT, bool UNIFORM>
bool dispatch_tile(const MatvecArgs &a, const Plan &p, hipStream_t stream) {
#define MK_CASE(MT_, C_)                                              \
    if (p.sample_tile == MT_ && p.chunks == C_) {                     \
        launch_chunked<BITS, XT, MT_, C_, UNIFORM>(a, p, stream);     \
        return true;                                                  \
    }
    MK_CASE(1, 1) MK_CASE(2, 1) MK_CASE(4, 1)
    MK_CASE(1, 2) MK_CASE(2, 2)
    if constexpr (XT != MK_F32) { MK_CASE(8, 1) MK_CASE(4, 2) }
#undef MK_CASE
    return false;
}

template <int BITS>
bool dispatch_bits(const MatvecArgs &a, const Plan &p, int x_dtype, bool uniform, hipStream_t stream) {
    if (uniform) {
        if (x_dtype == MK_F16) return dispatch_tile<BITS, MK_F16, true>(a, p, stream);
        if (x_dtype == MK_BF16) return dispatch_tile<BITS, MK_BF16, true>(a, p, stream);
        return dispatch_tile<BITS, MK_F32, true>(a, p, stream);
    }
    if (x_dtype == MK_F16) return dispatch_tile<BITS, MK_F16, false>(a, p, stream);
    if (x_dtype == MK_BF16) return dispatch_tile<BITS, MK_BF16, false>(a, p, stream);
    return dispatch_tile<BITS, MK_F32, false>(a, p, stream);
}

}  // namespace mk_matvec
