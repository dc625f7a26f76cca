// LDL-form error feedback (GPTQ / LDLQ) on gfx950: the sequential column sweep of a tile,
// the triangular solve that predicts a region's targets, and the trailing block update.
//
// Sweep and solve.  One wavefront owns one weight row; lane l keeps columns l, l + 64, ...
// of the tile in registers.  Step j takes one value from the lane that owns column j
// (v_readlane) and every lane adds its multiple of coefficient row j to its columns.
// Each column therefore receives exactly the sequence of separately rounded multiplies
// and adds that a scalar loop over j gives it.  Coefficient rows reach the wavefronts of
// a workgroup through LDS, a chunk of rows at a time, with the next chunk's global loads
// in flight while the current one is used; entries at or left of the diagonal are stored
// as zero, which makes the update of finished columns a no-op.
//
// Trailing update.  feedback[:, stop:] += (original - output)[:, tile] @ coeff[tile, stop:]
// runs on the fp32 matrix cores (v_mfma_f32_32x32x2_f32).  Each product sum starts from
// zero and accumulates over ascending k, which on this hardware equals a chain of fused
// multiply-adds in the same order; the sum is then added to feedback once.
//
// Replaces, in /root/reference/src/mlkit:
//   kernels/error_feedback.py:22-143                    round_feedback_tile / round_tile
//   quantization/algorithms/error_feedback.py:373-393   _pending_continuation (solve_triangular)
//   quantization/algorithms/error_feedback.py:366-370   trailing addmm_

#include "mk_common.h"

#include <type_traits>

namespace {

constexpr int kSweepThreads = 256;  // four wavefronts = four rows
constexpr int kModeInteger = 0, kModeCodebook = 1, kModeSolve = 2, kModeRegion = 3;

struct SweepArgs {
    const float *original;
    const float *feedback;
    const float *coeff;
    const float *scales;
    const float *zeros;
    const float *values;
    float *output;     // reconstruction [rows, width]; solve: [rows, span]
    uint8_t *encoded;  // [rows, width]
    float *deviation_t;  // null, or [width, rows]: original - reconstruction, column-major
    int rows, width;
    int region_start, tile_start, tile_width;
    int group, groups_per_row, n_values;
    float code_min, code_max;
    // kModeRegion only: the region's scales (and offsets) are fitted inside the kernel and
    // written to fit_scales / fit_zeros (same indexing as scales / zeros).
    float *fit_scales, *fit_zeros;
    int solve_first, asym, scale_format;
    float reciprocal, value_minimum;
};

// 16 bytes per lane from global memory straight into LDS: lane l's bytes land at
// `target` + 16 l (`target` is wavefront-uniform).  Completion counts as a vector memory load.
__device__ __forceinline__ void rows_to_lds(const float *source, float *target) {
    __builtin_amdgcn_global_load_lds(source, target, 16, 0, 0);
}

// Waits until this wavefront's vector memory loads, LDS transfers included, are complete.
__device__ __forceinline__ void wait_for_loads() {
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), other counters untouched
}

template <int S>
struct SweepShape {
    static constexpr int kWidth = 64 * S;                      // padded tile width
    static constexpr int kChunk = S <= 4 ? 16 : 4;             // coefficient rows per LDS chunk
    static constexpr int kPerThread = kChunk * kWidth / kSweepThreads;
};

// Coefficients outside the strict upper triangle of the tile count as zero.  fetch_chunk
// only issues the loads; keep_chunk, a chunk of steps later, is the first to look at them.
template <int S>
__device__ __forceinline__ bool chunk_wanted(const SweepArgs &a, int first, int p, int *j, int *c) {
    const int flat = p * kSweepThreads + threadIdx.x;
    *j = first + flat / SweepShape<S>::kWidth;
    *c = flat % SweepShape<S>::kWidth;
    return *j < a.tile_width && *c > *j && *c < a.tile_width;
}

template <int S>
__device__ __forceinline__ void fetch_chunk(const SweepArgs &a, int first, float (&held)[SweepShape<S>::kPerThread]) {
#pragma unroll
    for (int p = 0; p < SweepShape<S>::kPerThread; ++p) {
        int j, c;
        const bool wanted = chunk_wanted<S>(a, first, p, &j, &c);
        held[p] = a.coeff[static_cast<size_t>(a.tile_start + (wanted ? j : 0)) * a.width + a.tile_start + (wanted ? c : 0)];
    }
}

template <int S>
__device__ __forceinline__ void keep_chunk(const SweepArgs &a, int first, float *buffer,
                                           const float (&held)[SweepShape<S>::kPerThread]) {
#pragma unroll
    for (int p = 0; p < SweepShape<S>::kPerThread; ++p) {
        int j, c;
        const bool wanted = chunk_wanted<S>(a, first, p, &j, &c);
        buffer[p * kSweepThreads + threadIdx.x] = wanted ? held[p] : 0.0f;
    }
}

__device__ __forceinline__ float lane_value(float value, int lane) {
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(value), lane));
}

// Smallest (distance, index) over the table for one wavefront-uniform x: lane e scans
// entries e, e + 64, ...; keys order by distance first, then by index.
__device__ __forceinline__ int nearest_by_scan(float x, const float *table, int count, int lane) {
    unsigned long long best = ~0ull;
    for (int e = lane; e < count; e += 64) {
        const float distance = fabsf(__fsub_rn(x, table[e]));
        const unsigned long long key = (static_cast<unsigned long long>(__float_as_uint(distance)) << 32) | static_cast<unsigned>(e);
        best = key < best ? key : best;
    }
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const unsigned long long other = __shfl_xor(best, offset, 64);
        best = other < best ? other : best;
    }
    const int index = static_cast<int>(best & 0xffffffffu);
    return index < count ? index : count - 1;
}

template <int S, int MODE>
__global__ void __launch_bounds__(kSweepThreads) sweep_kernel(const SweepArgs a) {
    using Shape = SweepShape<S>;
    __shared__ float chunks[2][Shape::kChunk * Shape::kWidth];
    __shared__ float table[MODE == kModeCodebook ? 256 : 1];
    const int lane = threadIdx.x & 63;
    const int wanted_row = blockIdx.x * (kSweepThreads / 64) + (threadIdx.x >> 6);
    const bool active = wanted_row < a.rows;
    const int row = active ? wanted_row : a.rows - 1;
    const size_t row_base = static_cast<size_t>(row) * a.width;

    if constexpr (MODE == kModeCodebook)
        for (int i = threadIdx.x; i < a.n_values; i += kSweepThreads) table[i] = a.values[i];

    float held[Shape::kPerThread];
    fetch_chunk<S>(a, 0, held);

    // This lane's columns: weight, running correction, and the scale and offset of each.
    float weight[S], running[S], scale[S], zero[S], finished[S];
    uint32_t code[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const int c = 64 * s + lane;
        const bool inside = c < a.tile_width;
        const int position = a.tile_start + (inside ? c : 0);
        running[s] = inside ? a.feedback[row_base + position] : 0.0f;
        weight[s] = 0.0f; scale[s] = 1.0f; zero[s] = 0.0f; finished[s] = 0.0f; code[s] = 0;
        if constexpr (MODE != kModeSolve) {
            weight[s] = inside ? a.original[row_base + position] : 0.0f;
            const int slot = row * a.groups_per_row + (position - a.region_start) / a.group;
            scale[s] = inside ? a.scales[slot] : 1.0f;
            if (a.zeros) zero[s] = inside ? a.zeros[slot] : 0.0f;
        }
    }
    keep_chunk<S>(a, 0, chunks[0], held);
    __syncthreads();

    int chunk_index = 0;
#pragma unroll
    for (int s = 0; s < S; ++s) {
        for (int first = 64 * s; first < 64 * (s + 1) && first < a.tile_width; first += Shape::kChunk) {
            const bool more = first + Shape::kChunk < a.tile_width;
            if (more) fetch_chunk<S>(a, first + Shape::kChunk, held);
            const float *rows_of_chunk = chunks[chunk_index & 1];
            for (int i = 0; i < Shape::kChunk; ++i) {
                const int j = first + i;
                if (j >= a.tile_width) break;
                const int owner = j & 63;
                float pushed;
                if constexpr (MODE == kModeSolve) {
                    pushed = -lane_value(running[s], owner);
                } else {
                    const float target = __fadd_rn(weight[s], running[s]);
                    const float normalized = __fdiv_rn(__fsub_rn(target, zero[s]), scale[s]);
                    float chosen;
                    uint32_t index;
                    if constexpr (MODE == kModeInteger) {
                        chosen = fminf(fmaxf(rintf(normalized), a.code_min), a.code_max);
                        index = static_cast<uint32_t>(static_cast<int>(__fsub_rn(chosen, a.code_min)));
                    } else {
                        index = nearest_by_scan(lane_value(normalized, owner), table, a.n_values, lane);
                        chosen = table[index];
                    }
                    const float reconstruction = __fadd_rn(__fmul_rn(chosen, scale[s]), zero[s]);
                    const bool mine = lane == owner;
                    finished[s] = mine ? reconstruction : finished[s];
                    code[s] = mine ? index : code[s];
                    pushed = lane_value(__fsub_rn(weight[s], reconstruction), owner);
                }
                const float *coefficient_row = rows_of_chunk + i * Shape::kWidth + lane;
#pragma unroll
                for (int later = s; later < S; ++later)
                    running[later] = __fadd_rn(running[later], __fmul_rn(pushed, coefficient_row[64 * later]));
            }
            if (more) keep_chunk<S>(a, first + Shape::kChunk, chunks[(chunk_index + 1) & 1], held);
            __syncthreads();
            ++chunk_index;
        }
    }

    if (!active) return;
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const int c = 64 * s + lane;
        if (c >= a.tile_width) continue;
        if constexpr (MODE == kModeSolve) {
            // a.output is [rows, tile_width]; with `original` given the solved adjustment is
            // added to the region's weights (the targets a region's scales are fitted to).
            float value = running[s];
            if (a.original) value = __fadd_rn(a.original[row_base + a.tile_start + c], value);
            a.output[static_cast<size_t>(row) * a.tile_width + c] = value;
        } else {
            a.output[row_base + a.tile_start + c] = finished[s];
            a.encoded[row_base + a.tile_start + c] = static_cast<uint8_t>(code[s]);
            if (a.deviation_t)
                a.deviation_t[static_cast<size_t>(a.tile_start + c) * a.rows + row] = __fsub_rn(weight[s], finished[s]);
        }
    }
}

// ---- tiles of at most 128 columns: sixteen lanes per row ----------------------------------
//
// The sweep is one dependent chain per row (round column j, push its deviation into the
// later columns), so its time is (instructions per step) x (steps) x (wavefronts per SIMD).
// Here a wavefront sweeps four rows at once: lane 16 g + p owns columns p, 16 + p, ... ,
// 112 + p of row g (eight slots).  A step rounds one column in every lane's current slot,
// hands the owner's deviation to the sixteen lanes of its row (four `v_readlane` and a
// select) and updates at most eight columns per lane.  4096 rows are 1024 wavefronts, one
// per SIMD, each with a quarter of the per-step work of the one-row-per-wavefront kernel.
//
// Coefficient rows reach LDS sixteen at a time, which is one slot of steps; the layout
// [row in chunk][p][slot] lets a lane read its eight coefficients as two float4.

constexpr int kRowLanes = 16, kSlots = 8, kNarrowTile = kRowLanes * kSlots;  // 128 columns
constexpr int kNarrowRows = kSweepThreads / kRowLanes;                       // 16 rows per workgroup
constexpr int kNarrowHeld = kRowLanes * kNarrowTile / kSweepThreads;         // 8 coefficients per thread and chunk

// Coefficients outside the strict upper triangle of the tile count as zero.  The loads are
// issued here and first looked at in keep_slot, a slot of steps later.
__device__ __forceinline__ bool slot_wanted(const SweepArgs &a, int slot, int q, int *j, int *c) {
    const int flat = q * kSweepThreads + threadIdx.x;
    *j = slot * kRowLanes + flat / kNarrowTile;
    *c = flat % kNarrowTile;
    return *j < a.tile_width && *c > *j && *c < a.tile_width;
}

__device__ __forceinline__ void fetch_slot(const SweepArgs &a, int slot, float (&held)[kNarrowHeld]) {
#pragma unroll
    for (int q = 0; q < kNarrowHeld; ++q) {
        int j, c;
        const bool wanted = slot_wanted(a, slot, q, &j, &c);
        held[q] = a.coeff[static_cast<size_t>(a.tile_start + (wanted ? j : 0)) * a.width + a.tile_start + (wanted ? c : 0)];
    }
}

__device__ __forceinline__ void keep_slot(const SweepArgs &a, int slot, float *buffer, const float (&held)[kNarrowHeld]) {
#pragma unroll
    for (int q = 0; q < kNarrowHeld; ++q) {
        int j, c;
        const bool wanted = slot_wanted(a, slot, q, &j, &c);
        const int i = j - slot * kRowLanes;
        buffer[i * kNarrowTile + (c % kRowLanes) * kSlots + c / kRowLanes] = wanted ? held[q] : 0.0f;
    }
}

// The value lane 16 g + owner holds, in all sixteen lanes of row g.
__device__ __forceinline__ float row_value(float value, int owner, int row_in_wave) {
    const uint32_t bits = __float_as_uint(value);
    const uint32_t v0 = __builtin_amdgcn_readlane(bits, owner);
    const uint32_t v1 = __builtin_amdgcn_readlane(bits, owner + 16);
    const uint32_t v2 = __builtin_amdgcn_readlane(bits, owner + 32);
    const uint32_t v3 = __builtin_amdgcn_readlane(bits, owner + 48);
    uint32_t chosen = v3;
    chosen = row_in_wave == 2 ? v2 : chosen;
    chosen = row_in_wave == 1 ? v1 : chosen;
    chosen = row_in_wave == 0 ? v0 : chosen;
    return __uint_as_float(chosen);
}

// The same for an owner known at compile time: a DPP row broadcast, which the compiler
// folds into the multiplications that use the value.
template <int OWNER>
__device__ __forceinline__ float row_value(float value, std::integral_constant<int, OWNER>, int) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(value), 0x150 + OWNER, 0xf, 0xf, false));
}

// WHOLE: the tile is exactly 128 columns.  All 128 steps are unrolled, so owners, register
// slots and LDS offsets are constants, and the tile's 128 x 128 coefficients go from global
// memory straight into LDS before the first step (row-major; one memory latency for the
// whole kernel instead of one per slot).  Otherwise the sixteen steps of a slot are a loop
// over coefficient rows staged slot by slot.
// The nearest of up to sixteen table values by (distance, index): every lane compares its own
// value with all sixteen at once -- differences, then a tournament in which the entry with the
// higher index wins only on a strictly smaller distance.  Entries beyond the table are NaN and
// never win.  The same answer as a scan in ascending index order that keeps the first minimum.
constexpr int kSmallTable = 16;

struct Nearest {
    float difference, value;
    uint32_t index;
};

template <int COUNT>
__device__ __forceinline__ Nearest nearest_of(const Nearest (&entries)[COUNT]) {
    if constexpr (COUNT == 1) {
        return entries[0];
    } else {
        Nearest winners[COUNT / 2];
#pragma unroll
        for (int i = 0; i < COUNT / 2; ++i) {
            const Nearest &low = entries[2 * i], &high = entries[2 * i + 1];
            const bool take = fabsf(high.difference) < fabsf(low.difference);
            winners[i].difference = take ? high.difference : low.difference;
            winners[i].value = take ? high.value : low.value;
            winners[i].index = take ? high.index : low.index;
        }
        return nearest_of<COUNT / 2>(winners);
    }
}

// Tables of 17 to 256 values: the sixteen lanes of a row search for the value of the column that is being rounded
// (the step's owner) together.  Lane p holds entries p, 16 + p, 32 + p, ... (entries beyond the table are NaN and
// never win: every lane holds at least one real entry), finds the nearest of its own by the tournament above
// and the sixteen winners meet in four DPP exchanges (lane ^ 1, lane ^ 2, mirrored halves of eight, mirrored
// row), in each of which the other lane's entry wins on a strictly smaller distance, or on an equal distance and
// a lower index: the smallest (distance, index) of the table, in every lane of the row.
constexpr int kLargeTable = 256;

// (Distances compare as the bit patterns of their magnitudes: the same order for numbers, and a NaN -- an entry
// beyond the table -- is larger than every number, so it loses to any real entry.)
template <int CONTROL>
__device__ __forceinline__ Nearest nearer_of_lane_pair(const Nearest &mine) {
    Nearest other;
    other.difference = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(mine.difference), CONTROL, 0xf, 0xf, true));
    other.value = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(mine.value), CONTROL, 0xf, 0xf, true));
    other.index = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(mine.index), CONTROL, 0xf, 0xf, true));
    const uint32_t own_distance = __float_as_uint(mine.difference) & 0x7fffffffu;
    const uint32_t other_distance = __float_as_uint(other.difference) & 0x7fffffffu;
    const bool take = other_distance < own_distance || (other_distance == own_distance && other.index < mine.index);
    Nearest winner;
    winner.difference = take ? other.difference : mine.difference;
    winner.value = take ? other.value : mine.value;
    winner.index = take ? other.index : mine.index;
    return winner;
}

__device__ __forceinline__ Nearest nearest_over_row(float wanted, const float (&table)[kLargeTable / 16], int p) {
    constexpr int kOwn = kLargeTable / 16;
    // This lane's entries in ascending index order, keeping the first minimum (a scan rather than the tournament:
    // one comparison result alive at a time; the fully unrolled sweep around it has no registers to spare).
    __builtin_amdgcn_sched_barrier(0);
    float best_difference = __fsub_rn(wanted, table[0]), best_value = table[0];
    int best_slot = 0;
#pragma unroll
    for (int i = 1; i < kOwn; ++i) {
        const float difference = __fsub_rn(wanted, table[i]);
        const bool take = fabsf(difference) < fabsf(best_difference);
        best_difference = take ? difference : best_difference;
        best_value = take ? table[i] : best_value;
        best_slot = take ? i : best_slot;
    }
    Nearest best;
    best.difference = best_difference;
    best.value = best_value;
    best.index = static_cast<uint32_t>(16 * best_slot + p);
    best = nearer_of_lane_pair<0xB1>(best);    // quad_perm [1,0,3,2]
    best = nearer_of_lane_pair<0x4E>(best);    // quad_perm [2,3,0,1]
    best = nearer_of_lane_pair<0x141>(best);   // row_half_mirror: lane i <-> 7 - i of each eight
    best = nearer_of_lane_pair<0x140>(best);   // row_mirror: lane i <-> 15 - i of the row
    __builtin_amdgcn_sched_barrier(0);
    return best;
}

// Up to sixteen values with a compile-time owner (the unrolled whole-tile kernels): lane p holds entry p alone and
// the sixteen lanes meet as above; the owner's value arrives as a DPP row broadcast folded into the subtraction.
__device__ __forceinline__ Nearest nearest_one_per_lane(float wanted, float entry, int p) {
    Nearest best;
    best.difference = __fsub_rn(wanted, entry);
    best.value = entry;
    best.index = static_cast<uint32_t>(p);
    best = nearer_of_lane_pair<0xB1>(best);
    best = nearer_of_lane_pair<0x4E>(best);
    best = nearer_of_lane_pair<0x141>(best);
    best = nearer_of_lane_pair<0x140>(best);
    return best;
}

// TABLE: 0 rounds to an integer grid; kSmallTable rounds to a table of at most sixteen values, kLargeTable to one of
// at most 256.
template <int MODE, bool WHOLE, int TABLE = 0>
__global__ void __launch_bounds__(kSweepThreads) narrow_sweep_kernel(const SweepArgs a) {
    static_assert(MODE == kModeInteger || MODE == kModeSolve || (MODE == kModeRegion && WHOLE),
                  "larger tables use the one-row-per-wavefront kernel; a fused region is one whole tile");
    static_assert(TABLE == 0 || ((TABLE == kSmallTable || TABLE == kLargeTable) && MODE != kModeSolve),
                  "a table of at most sixteen or at most 256 values, or none");
    constexpr int kHeldEntries = TABLE == kLargeTable ? kLargeTable / 16 : TABLE;
    constexpr int kStaged = WHOLE ? kNarrowTile * kNarrowTile : 2 * kRowLanes * kNarrowTile;
    __shared__ __attribute__((aligned(16))) float staged[kStaged];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int row_in_wave = lane >> 4, p = lane & (kRowLanes - 1);
    const int wanted_row = blockIdx.x * kNarrowRows + wave * 4 + row_in_wave;
    const bool active = wanted_row < a.rows;
    const int row = active ? wanted_row : a.rows - 1;
    const size_t row_base = static_cast<size_t>(row) * a.width;

    float table[TABLE > 0 ? kHeldEntries : 1];
    if constexpr (TABLE == kLargeTable) {
#pragma unroll
        for (int i = 0; i < kHeldEntries; ++i) {
            const int entry = 16 * i + p;
            table[i] = entry < a.n_values ? a.values[entry < a.n_values ? entry : 0] : __builtin_nanf("");
        }
    } else if constexpr (TABLE > 0 && WHOLE) {
        table[0] = p < a.n_values ? a.values[p < a.n_values ? p : 0] : __builtin_nanf("");   // this lane's entry
    } else if constexpr (TABLE > 0) {
#pragma unroll
        for (int i = 0; i < TABLE; ++i) table[i] = i < a.n_values ? a.values[i < a.n_values ? i : 0] : __builtin_nanf("");
    }

    float held[kNarrowHeld];
    if constexpr (WHOLE) {
        // One wavefront instruction moves two coefficient rows of the tile (2 x 128 floats,
        // lane l's 16 bytes at 16 l from the uniform LDS address); a wavefront moves rows
        // 32 wave ... 32 wave + 31.
        const float *corner = a.coeff + static_cast<size_t>(a.tile_start) * a.width + a.tile_start;
        const uint32_t lane_offset = static_cast<uint32_t>(lane >> 5) * a.width + (lane & 31) * 4;
#pragma unroll
        for (int pair = 0; pair < 16; ++pair) {
            const int j = wave * 32 + 2 * pair;
            rows_to_lds(corner + static_cast<size_t>(j) * a.width + lane_offset, &staged[j * kNarrowTile]);
        }
    } else {
        fetch_slot(a, 0, held);
    }

    float weight[kSlots], running[kSlots], scale[kSlots], zero[kSlots], finished[kSlots], base[kSlots];
    uint32_t code[kSlots];
#pragma unroll
    for (int t = 0; t < kSlots; ++t) {
        const int c = kRowLanes * t + p;
        const bool inside = c < a.tile_width;
        const int position = a.tile_start + (inside ? c : 0);
        running[t] = inside ? a.feedback[row_base + position] : 0.0f;
        weight[t] = 0.0f; scale[t] = 1.0f; zero[t] = 0.0f; finished[t] = 0.0f; code[t] = 0; base[t] = 0.0f;
        if constexpr (MODE == kModeRegion) {
            weight[t] = a.original[row_base + position];
        } else if constexpr (MODE != kModeSolve) {
            weight[t] = inside ? a.original[row_base + position] : 0.0f;
            const int slot = row * a.groups_per_row + (position - a.region_start) / a.group;
            scale[t] = inside ? a.scales[slot] : 1.0f;
            if (a.zeros) zero[t] = inside ? a.zeros[slot] : 0.0f;
        } else {
            if (a.original) base[t] = a.original[row_base + position];  // added to the solved adjustment at the end
        }
    }
    if constexpr (WHOLE) {
        wait_for_loads();
    } else {
        keep_slot(a, 0, staged, held);
    }
    __syncthreads();

    // One step: round column 16 t + owner of every row, push its deviation into the later
    // columns.  `owner` is an int or a std::integral_constant.  `coefficients` is row
    // 16 t + owner of the tile as this lane reads it.
    // WHOLE: the coefficient row of a step is read from LDS during the step before it (the
    // addresses are known in advance; read inside the step, every step waited for LDS at the
    // head of its dependent chain).  Even steps use one set of registers, odd steps the other.
    float row_even[kSlots], row_odd[kSlots];
    auto load_row = [&](auto slot, auto owner, float (&row)[kSlots]) __attribute__((always_inline)) {
        constexpr int t = decltype(slot)::value;
        const float *coefficients = staged + (kRowLanes * t + decltype(owner)::value) * kNarrowTile + p;
#pragma unroll
        for (int later = t; later < kSlots; ++later) row[later] = coefficients[kRowLanes * later];
    };
    auto advance = [&](auto slot, auto owner, const float *coefficients, auto solving, const float (&row_ready)[kSlots]) __attribute__((always_inline)) {
        constexpr int t = decltype(slot)::value;
        constexpr bool kSolving = decltype(solving)::value;
        float pushed;
        if constexpr (kSolving) {
            pushed = -row_value(running[t], owner, row_in_wave);
        } else {
            const float target = __fadd_rn(weight[t], running[t]);
            const float normalized = __fdiv_rn(__fsub_rn(target, zero[t]), scale[t]);
            float chosen;
            uint32_t index;
            if constexpr (TABLE == kLargeTable) {
                const Nearest nearest = nearest_over_row(row_value(normalized, owner, row_in_wave), table, p);
                chosen = nearest.value;
                index = nearest.index;
            } else if constexpr (TABLE > 0 && WHOLE) {
                const Nearest nearest = nearest_one_per_lane(row_value(normalized, owner, row_in_wave), table[0], p);
                chosen = nearest.value;
                index = nearest.index;
            } else if constexpr (TABLE > 0) {
                Nearest entries[TABLE];
#pragma unroll
                for (int i = 0; i < TABLE; ++i) {
                    entries[i].difference = __fsub_rn(normalized, table[i]);
                    entries[i].value = table[i];
                    entries[i].index = i;
                }
                const Nearest nearest = nearest_of<TABLE>(entries);
                chosen = nearest.value;
                index = nearest.index;
            } else {
                chosen = fminf(fmaxf(rintf(normalized), a.code_min), a.code_max);
                index = static_cast<uint32_t>(static_cast<int>(__fsub_rn(chosen, a.code_min)));
            }
            const float reconstruction = __fadd_rn(__fmul_rn(chosen, scale[t]), zero[t]);
            const bool mine = p == static_cast<int>(owner);
            finished[t] = mine ? reconstruction : finished[t];
            code[t] = mine ? index : code[t];
            pushed = row_value(__fsub_rn(weight[t], reconstruction), owner, row_in_wave);
        }
        float row_of[kSlots];
        if constexpr (WHOLE) {
            // Row-major row: this lane's columns are 16 floats apart.  Columns up to the
            // owner's hold whatever the matrix has there; only the solve still reads its
            // running values of such columns afterwards, so it masks them.
#pragma unroll
            for (int later = t; later < kSlots; ++later) row_of[later] = row_ready[later];
            if constexpr (kSolving) row_of[t] = p > static_cast<int>(owner) ? row_of[t] : 0.0f;
        } else {
            float4 low = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (t < 4) low = *reinterpret_cast<const float4 *>(coefficients);
            const float4 high = *reinterpret_cast<const float4 *>(coefficients + 4);
            row_of[0] = low.x, row_of[1] = low.y, row_of[2] = low.z, row_of[3] = low.w;
            row_of[4] = high.x, row_of[5] = high.y, row_of[6] = high.z, row_of[7] = high.w;
        }
#pragma unroll
        for (int later = t; later < kSlots; ++later)
            running[later] = __fadd_rn(running[later], __fmul_rn(pushed, row_of[later]));
    };
    auto step_of_whole = [&](auto slot, auto owner, auto solving) __attribute__((always_inline)) {
        constexpr int t = decltype(slot)::value, o = decltype(owner)::value;
        constexpr bool kLast = t == kSlots - 1 && o == kRowLanes - 1;
        using NextSlot = std::integral_constant<int, (o == kRowLanes - 1 && !kLast) ? t + 1 : t>;
        using NextOwner = std::integral_constant<int, o == kRowLanes - 1 ? 0 : o + 1>;
        if constexpr (o & 1) {
            if constexpr (!kLast) load_row(NextSlot{}, NextOwner{}, row_even);
            __builtin_amdgcn_sched_barrier(0);  // the reads stay ahead of this step's arithmetic
            advance(slot, owner, nullptr, solving, row_odd);
        } else {
            load_row(NextSlot{}, NextOwner{}, row_odd);
            __builtin_amdgcn_sched_barrier(0);
            advance(slot, owner, nullptr, solving, row_even);
        }
    };
    auto slot_of_steps = [&](auto slot, auto solving) __attribute__((always_inline)) {
        constexpr int t = decltype(slot)::value;
        if constexpr (WHOLE && TABLE == kLargeTable) {
            // The search of a large table is some 150 instructions per step: unrolled 128 times it neither fits the
            // registers nor the instruction cache.  The sixteen steps of a slot are a loop; the owner's value
            // comes through v_readlane and the next step's coefficient row is read from LDS a step ahead.
            float row_now[kSlots], row_next[kSlots];
            auto read_row = [&](int index, float (&row)[kSlots]) __attribute__((always_inline)) {
                const float *coefficients = staged + index * kNarrowTile + p;
#pragma unroll
                for (int later = t; later < kSlots; ++later) row[later] = coefficients[kRowLanes * later];
            };
            read_row(kRowLanes * t, row_now);
            for (int owner = 0; owner < kRowLanes; ++owner) {
                const int following = kRowLanes * t + owner + 1;
                read_row(following < kNarrowTile ? following : kNarrowTile - 1, row_next);
                advance(slot, owner, nullptr, solving, row_now);
#pragma unroll
                for (int later = t; later < kSlots; ++later) row_now[later] = row_next[later];
            }
        } else if constexpr (WHOLE) {
            step_of_whole(slot, std::integral_constant<int, 0>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 1>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 2>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 3>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 4>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 5>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 6>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 7>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 8>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 9>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 10>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 11>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 12>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 13>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 14>{}, solving);
            step_of_whole(slot, std::integral_constant<int, 15>{}, solving);
        } else if (kRowLanes * t < a.tile_width) {  // uniform
            const bool more = kRowLanes * (t + 1) < a.tile_width;
            if (more) fetch_slot(a, t + 1, held);
            const float *mine_in_chunk = staged + (t & 1) * kRowLanes * kNarrowTile + p * kSlots;
            const int owners = min(kRowLanes, a.tile_width - kRowLanes * t);
            for (int owner = 0; owner < owners; ++owner) advance(slot, owner, mine_in_chunk + owner * kNarrowTile, solving, row_even);
            if (more) keep_slot(a, t + 1, staged + ((t + 1) & 1) * kRowLanes * kNarrowTile, held);
            __syncthreads();
        }
    };
    auto all_slots = [&](auto solving) __attribute__((always_inline)) {
        if constexpr (WHOLE && TABLE != kLargeTable) load_row(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, row_even);
        slot_of_steps(std::integral_constant<int, 0>{}, solving);
        slot_of_steps(std::integral_constant<int, 1>{}, solving);
        slot_of_steps(std::integral_constant<int, 2>{}, solving);
        slot_of_steps(std::integral_constant<int, 3>{}, solving);
        slot_of_steps(std::integral_constant<int, 4>{}, solving);
        slot_of_steps(std::integral_constant<int, 5>{}, solving);
        slot_of_steps(std::integral_constant<int, 6>{}, solving);
        slot_of_steps(std::integral_constant<int, 7>{}, solving);
    };
    if constexpr (MODE == kModeRegion) {
        // The region's scales are fitted to original + x, where x U = feedback over the
        // region's own columns (U: the unit upper coefficient tile); then the same columns
        // are rounded with those scales.  Both passes read the coefficient tile from LDS.
        float fed[kSlots];
#pragma unroll
        for (int t = 0; t < kSlots; ++t) fed[t] = running[t];
        if (a.solve_first) all_slots(std::true_type{});   // uniform
        float fitted[kSlots];
#pragma unroll
        for (int t = 0; t < kSlots; ++t) {
            fitted[t] = a.solve_first ? __fadd_rn(weight[t], running[t]) : weight[t];
            running[t] = fed[t];
        }
        // A scale group is `a.group` columns: group / 16 adjacent slots of all sixteen lanes.
        const int slots_per_group = a.group / kRowLanes;
        auto fit_groups = [&](auto span) __attribute__((always_inline)) {
            constexpr int kSpan = decltype(span)::value;
#pragma unroll
            for (int first = 0; first < kSlots; first += kSpan) {
                float low = fitted[first], high = fitted[first];
                bool all_finite = true;
#pragma unroll
                for (int t = first; t < first + kSpan; ++t) {
                    low = fminf(low, fitted[t]);
                    high = fmaxf(high, fitted[t]);
                    all_finite = all_finite && (fitted[t] - fitted[t] == 0.0f);
                }
#pragma unroll
                for (int offset = 1; offset < kRowLanes; offset <<= 1) {
                    low = fminf(low, __shfl_xor(low, offset, 64));
                    high = fmaxf(high, __shfl_xor(high, offset, 64));
                    all_finite = __shfl_xor(static_cast<int>(all_finite), offset, 64) && all_finite;
                }
                float group_scale, group_zero = 0.0f;
                if (a.asym) {
                    group_scale = __fmul_rn(fmaxf(__fsub_rn(high, low), 1e-12f), a.reciprocal);
                    group_zero = __fsub_rn(low, __fmul_rn(a.value_minimum, group_scale));
                    const float magnitude = mk_rounded_scale(fmaxf(fabsf(group_zero), 1e-12f), a.scale_format);
                    group_zero = group_zero > 0.0f ? magnitude : (group_zero < 0.0f ? -magnitude : 0.0f);
                } else {
                    group_scale = __fmul_rn(fmaxf(fmaxf(high, -low), 1e-12f), a.reciprocal);
                }
                group_scale = mk_rounded_scale(group_scale, a.scale_format);
                if (!all_finite) {  // fminf / fmaxf drop NaNs: report them as the tensor reductions would
                    group_scale = __builtin_nanf("");
                    group_zero = __builtin_nanf("");
                }
#pragma unroll
                for (int t = first; t < first + kSpan; ++t) {
                    scale[t] = group_scale;
                    zero[t] = group_zero;
                }
                if (active && p == 0) {
                    const int slot = row * a.groups_per_row + first / kSpan;
                    a.fit_scales[slot] = group_scale;
                    if (a.fit_zeros) a.fit_zeros[slot] = group_zero;
                }
            }
        };
        if (slots_per_group == 8) fit_groups(std::integral_constant<int, 8>{});
        else if (slots_per_group == 4) fit_groups(std::integral_constant<int, 4>{});
        else if (slots_per_group == 2) fit_groups(std::integral_constant<int, 2>{});
        else fit_groups(std::integral_constant<int, 1>{});
        all_slots(std::false_type{});
    } else {
        all_slots(std::bool_constant<MODE == kModeSolve>{});
    }

    if (!active) return;
#pragma unroll
    for (int t = 0; t < kSlots; ++t) {
        const int c = kRowLanes * t + p;
        if (c >= a.tile_width) continue;
        if constexpr (MODE == kModeSolve) {
            // a.output is [rows, tile_width]; with `original` given the solved adjustment is
            // added to the region's weights (the targets a region's scales are fitted to).
            a.output[static_cast<size_t>(row) * a.tile_width + c] = a.original ? __fadd_rn(base[t], running[t]) : running[t];
        } else {
            a.output[row_base + a.tile_start + c] = finished[t];
            a.encoded[row_base + a.tile_start + c] = static_cast<uint8_t>(code[t]);
            if (a.deviation_t)
                a.deviation_t[static_cast<size_t>(a.tile_start + c) * a.rows + row] = __fsub_rn(weight[t], finished[t]);
        }
    }
}

// One kernel for a region that is a single whole tile of an integer grid: pending solve,
// scale fit and column sweep.
bool region_fusable(int span, int block, int fitted_group, bool integer_grid, int n_values) {
    return (integer_grid || n_values <= kLargeTable) && span == kNarrowTile && block >= kNarrowTile &&
           fitted_group % kRowLanes == 0 && kNarrowTile % fitted_group == 0;
}

int launch_region(const SweepArgs &a, bool integer_grid, hipStream_t stream) {
    const dim3 grid(mk_cdiv(a.rows, kNarrowRows)), block(kSweepThreads);
    if (integer_grid) hipLaunchKernelGGL((narrow_sweep_kernel<kModeRegion, true>), grid, block, 0, stream, a);
    else if (a.n_values <= kSmallTable) hipLaunchKernelGGL((narrow_sweep_kernel<kModeRegion, true, kSmallTable>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((narrow_sweep_kernel<kModeRegion, true, kLargeTable>), grid, block, 0, stream, a);
    return MK_OK;
}

template <int MODE>
int launch_sweep(const SweepArgs &a, hipStream_t stream) {
    const dim3 grid(mk_cdiv(a.rows, kSweepThreads / 64)), block(kSweepThreads);
    if constexpr (MODE != kModeCodebook) {
        if (a.tile_width <= kNarrowTile) {
            const dim3 narrow_grid(mk_cdiv(a.rows, kNarrowRows));
            if (a.tile_width == kNarrowTile)
                hipLaunchKernelGGL((narrow_sweep_kernel<MODE, true>), narrow_grid, block, 0, stream, a);
            else
                hipLaunchKernelGGL((narrow_sweep_kernel<MODE, false>), narrow_grid, block, 0, stream, a);
            return MK_OK;
        }
    } else if (a.tile_width <= kNarrowTile && a.n_values <= kSmallTable) {
        // small tables (NF4, FP4, ...): sixteen lanes per row, every lane searching the table for itself
        const dim3 narrow_grid(mk_cdiv(a.rows, kNarrowRows));
        if (a.tile_width == kNarrowTile)
            hipLaunchKernelGGL((narrow_sweep_kernel<kModeInteger, true, kSmallTable>), narrow_grid, block, 0, stream, a);
        else
            hipLaunchKernelGGL((narrow_sweep_kernel<kModeInteger, false, kSmallTable>), narrow_grid, block, 0, stream, a);
        return MK_OK;
    } else if (a.tile_width <= kNarrowTile && a.n_values <= kLargeTable) {
        // larger tables (minifloat grids, codebooks): the sixteen lanes of a row search the table together
        const dim3 narrow_grid(mk_cdiv(a.rows, kNarrowRows));
        if (a.tile_width == kNarrowTile)
            hipLaunchKernelGGL((narrow_sweep_kernel<kModeInteger, true, kLargeTable>), narrow_grid, block, 0, stream, a);
        else
            hipLaunchKernelGGL((narrow_sweep_kernel<kModeInteger, false, kLargeTable>), narrow_grid, block, 0, stream, a);
        return MK_OK;
    }
    if (a.tile_width <= 128)
        hipLaunchKernelGGL((sweep_kernel<2, MODE>), grid, block, 0, stream, a);
    else if (a.tile_width <= 256)
        hipLaunchKernelGGL((sweep_kernel<4, MODE>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((sweep_kernel<16, MODE>), grid, block, 0, stream, a);
    return MK_OK;
}

// ---- trailing block update on the fp32 matrix cores ------------------------------------
//
// feedback[:, c0:c1] receives, chain after chain, the product of one tile's deviations with
// its coefficient rows:  f = (...((f + S_0) + S_1)...) , S_i = sum over the k of chain i,
// started from zero.  Several deferred tiles (chains) can therefore be applied in one pass
// over feedback with exactly the roundings of applying them one launch at a time.
//
// A workgroup of four wavefronts owns a 128 x 128 tile of feedback; each wavefront keeps a
// 64 x 64 quarter as 2 x 2 MFMA tiles.  k advances in chunks of 32: the next chunk's global
// loads are issued before the current chunk's 64 MFMAs and land in the other LDS buffer
// afterwards, so one barrier per chunk suffices.

typedef float mk_f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTileRows = 128, kTileColumns = 128, kDepthChunk = 32, kUpdateThreads = 256;
constexpr int kDeviationLoads = kTileRows * kDepthChunk / 4 / kUpdateThreads;      // float4 per thread
constexpr int kCoefficientLoads = kDepthChunk * kTileColumns / 4 / kUpdateThreads;

struct UpdateArgs {
    float *feedback;
    const float *original;
    const float *output;
    const float *coeff;
    int rows, width;
    int first_column;   // first column of chain 0
    int chain_width;    // columns (= k) per chain
    int chains;
    int column_begin, column_end;  // columns of feedback that are updated
    const float *deviation_t;      // null, or [width, rows] deviations written by the sweep
    // The kernels that read `deviation_t` take a linear range of tiles (column tile fastest):
    // workgroup b owns tile `tile_first + b` of a grid `column_tiles` wide.
    int tile_first, column_tiles;
};

struct UpdateStage {
    float4 deviation[kDeviationLoads];
    float4 coefficient[kCoefficientLoads];
};

// VEC: rows and tiles start on 16-byte boundaries, so operands load as float4.
template <bool VEC>
__device__ __forceinline__ void fetch_stage(const UpdateArgs &a, int row0, int column0, int k_base, int k_limit,
                                            UpdateStage &stage) {
#pragma unroll
    for (int p = 0; p < kDeviationLoads; ++p) {
        const int flat = p * kUpdateThreads + threadIdx.x;
        const int r = flat / (kDepthChunk / 4), k = (flat % (kDepthChunk / 4)) * 4;
        const bool row_ok = row0 + r < a.rows;
        const size_t base = static_cast<size_t>(row_ok ? row0 + r : 0) * a.width + k_base;
        float values[4];
        if (VEC && k + 4 <= k_limit) {
            const float4 w = *reinterpret_cast<const float4 *>(a.original + base + k);
            const float4 q = *reinterpret_cast<const float4 *>(a.output + base + k);
            values[0] = __fsub_rn(w.x, q.x); values[1] = __fsub_rn(w.y, q.y);
            values[2] = __fsub_rn(w.z, q.z); values[3] = __fsub_rn(w.w, q.w);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool ok = k + i < k_limit;
                const size_t index = base + (ok ? k + i : 0);
                const float difference = __fsub_rn(a.original[index], a.output[index]);
                values[i] = ok ? difference : 0.0f;
            }
        }
        stage.deviation[p] = row_ok ? make_float4(values[0], values[1], values[2], values[3])
                                    : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
#pragma unroll
    for (int p = 0; p < kCoefficientLoads; ++p) {
        const int flat = p * kUpdateThreads + threadIdx.x;
        const int k = flat / (kTileColumns / 4), c = (flat % (kTileColumns / 4)) * 4;
        const bool k_ok = k < k_limit;
        const size_t base = static_cast<size_t>(k_base + (k_ok ? k : 0)) * a.width;
        float values[4];
        if (VEC && column0 + c + 4 <= a.column_end) {
            const float4 v = *reinterpret_cast<const float4 *>(a.coeff + base + column0 + c);
            values[0] = v.x; values[1] = v.y; values[2] = v.z; values[3] = v.w;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool ok = column0 + c + i < a.column_end;
                const float loaded = a.coeff[base + (ok ? column0 + c + i : 0)];
                values[i] = ok ? loaded : 0.0f;
            }
        }
        stage.coefficient[p] = k_ok ? make_float4(values[0], values[1], values[2], values[3])
                                    : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
}

__device__ __forceinline__ void keep_stage(float (*deviation_t)[kTileRows + 1], float (*coefficient)[kTileColumns],
                                           const UpdateStage &stage) {
#pragma unroll
    for (int p = 0; p < kDeviationLoads; ++p) {
        const int flat = p * kUpdateThreads + threadIdx.x;
        const int r = flat / (kDepthChunk / 4), k = (flat % (kDepthChunk / 4)) * 4;
        deviation_t[k + 0][r] = stage.deviation[p].x;
        deviation_t[k + 1][r] = stage.deviation[p].y;
        deviation_t[k + 2][r] = stage.deviation[p].z;
        deviation_t[k + 3][r] = stage.deviation[p].w;
    }
#pragma unroll
    for (int p = 0; p < kCoefficientLoads; ++p) {
        const int flat = p * kUpdateThreads + threadIdx.x;
        const int k = flat / (kTileColumns / 4), c = (flat % (kTileColumns / 4)) * 4;
        *reinterpret_cast<float4 *>(&coefficient[k][c]) = stage.coefficient[p];
    }
}

template <bool VEC>
__global__ void __launch_bounds__(kUpdateThreads, 2) block_update_kernel(const UpdateArgs a) {
    __shared__ float deviation_t[2][kDepthChunk][kTileRows + 1];  // [buffer][k][row]
    __shared__ __attribute__((aligned(16))) float coefficient[2][kDepthChunk][kTileColumns];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row0 = blockIdx.y * kTileRows;
    const int column0 = a.column_begin + blockIdx.x * kTileColumns;
    const int wave_row = (wave >> 1) * 64, wave_column = (wave & 1) * 64;
    const int chunks_per_chain = (a.chain_width + kDepthChunk - 1) / kDepthChunk;
    const int steps = a.chains * chunks_per_chain;

    // Running totals start from feedback itself.
    mk_f32x16 totals[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = row0 + wave_row + mi * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                const int column = column0 + wave_column + ni * 32 + (lane & 31);
                const bool inside = row < a.rows && column < a.column_end;
                totals[mi][ni][r] = inside ? a.feedback[static_cast<size_t>(row) * a.width + column] : 0.0f;
            }

    auto k_of = [&](int step, int &k_base, int &k_limit) __attribute__((always_inline)) {
        const int chain = step / chunks_per_chain, chunk = step - chain * chunks_per_chain;
        k_base = a.first_column + chain * a.chain_width + chunk * kDepthChunk;
        k_limit = a.chain_width - chunk * kDepthChunk;
        if (k_limit > kDepthChunk) k_limit = kDepthChunk;
    };

    UpdateStage stage;
    int k_base, k_limit;
    k_of(0, k_base, k_limit);
    fetch_stage<VEC>(a, row0, column0, k_base, k_limit, stage);
    keep_stage(deviation_t[0], coefficient[0], stage);
    __syncthreads();

    mk_f32x16 sums[2][2];
    for (int step = 0; step < steps; ++step) {
        const int buffer = step & 1;
        const int chunk = step % chunks_per_chain;
        if (chunk == 0) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sums[mi][ni][r] = 0.0f;
        }
        const bool more = step + 1 < steps;
        if (more) {
            k_of(step + 1, k_base, k_limit);
            fetch_stage<VEC>(a, row0, column0, k_base, k_limit, stage);
        }
#pragma unroll 4
        for (int kk = 0; kk < kDepthChunk; kk += 2) {
            const int k = kk + (lane >> 5);
            float left[2], right[2];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) left[mi] = deviation_t[buffer][k][wave_row + mi * 32 + (lane & 31)];
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) right[ni] = coefficient[buffer][k][wave_column + ni * 32 + (lane & 31)];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    sums[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(left[mi], right[ni], sums[mi][ni], 0, 0, 0);
        }
        if (chunk == chunks_per_chain - 1) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r) totals[mi][ni][r] = __fadd_rn(totals[mi][ni][r], sums[mi][ni][r]);
        }
        if (more) keep_stage(deviation_t[buffer ^ 1], coefficient[buffer ^ 1], stage);
        __syncthreads();
    }

#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = row0 + wave_row + mi * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                const int column = column0 + wave_column + ni * 32 + (lane & 31);
                if (row < a.rows && column < a.column_end)
                    a.feedback[static_cast<size_t>(row) * a.width + column] = totals[mi][ni][r];
            }
}

// The same update with the deviations read from the column-major buffer the sweep kernel
// fills, for launches made of whole tiles only (rows and updated columns in multiples of
// 128, chains in multiples of 32 columns): the left operand loads and lands in LDS as whole
// float4s along the rows (no subtraction, no transposing stores), nothing is masked, and
// every address that does not depend on k is computed once.
constexpr int kDeviationStride = kTileRows;  // floats per k row in LDS

__global__ void __launch_bounds__(kUpdateThreads, 2) block_update_from_deviations_kernel(const UpdateArgs a) {
    // Two buffers per operand, each a variable of its own: the compiler then sees that the
    // transfer into one buffer cannot touch the buffer being read, and does not wait for it.
    __shared__ __attribute__((aligned(16))) float deviation_even[kDepthChunk][kDeviationStride];  // [k][row]
    __shared__ __attribute__((aligned(16))) float deviation_odd[kDepthChunk][kDeviationStride];
    __shared__ __attribute__((aligned(16))) float coefficient_even[kDepthChunk][kTileColumns];    // [k][column]
    __shared__ __attribute__((aligned(16))) float coefficient_odd[kDepthChunk][kTileColumns];
    // Addresses are a wavefront-uniform 64-bit base plus a 32-bit per-lane offset, so that
    // the compiler keeps the bases in scalar registers.
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = a.tile_first + blockIdx.x;
    const int tile_row = tile / a.column_tiles;
    const int row0 = tile_row * kTileRows;
    const int column0 = a.column_begin + (tile - tile_row * a.column_tiles) * kTileColumns;
    const int wave_row = (wave >> 1) * 64, wave_column = (wave & 1) * 64;
    const int chunks_per_chain = a.chain_width / kDepthChunk;
    const int steps = a.chains * chunks_per_chain;

    // Operands go from global memory straight into LDS: one wavefront instruction moves two
    // consecutive k rows of a tile (2 x 128 floats = 64 lanes x 16 bytes, lane l's bytes at
    // 16 l from the wavefront-uniform LDS address). Per chunk a wavefront moves k rows
    // 8 wave ... 8 wave + 7 of both tiles.
    const uint32_t left_lane = static_cast<uint32_t>(lane >> 5) * a.rows + (lane & 31) * 4;
    const uint32_t right_lane = static_cast<uint32_t>(lane >> 5) * a.width + (lane & 31) * 4;
    const float *left_tile = a.deviation_t + row0;     // + k * rows
    const float *right_tile = a.coeff + column0;       // + k * width

    // This lane's cell of every 32 x 32 MFMA tile: rows (lane / 32) * 4 + ..., column lane % 32.
    const uint32_t cell_lane = static_cast<uint32_t>((lane >> 5) * 4) * a.width + (lane & 31);
    float *quarter = a.feedback + static_cast<size_t>(row0 + wave_row) * a.width + column0 + wave_column;
    auto cell = [&](int mi, int ni, int r) __attribute__((always_inline)) -> float * {
        return quarter + static_cast<size_t>(mi * 32 + (r >> 2) * 8 + (r & 3)) * a.width + ni * 32 + cell_lane;
    };
    // feedback's own values: one 32 x 32 quarter is requested in each of the first four steps,
    // behind that step's operand loads, so that no step waits for the whole tile.
    mk_f32x16 totals[2][2];

    auto fetch = [&](int step, auto odd) __attribute__((always_inline)) {
        const int chain = step / chunks_per_chain, chunk = step - chain * chunks_per_chain;
        const size_t k_base = static_cast<size_t>(a.first_column + chain * a.chain_width + chunk * kDepthChunk + wave * 8);
        const float *left = left_tile + k_base * a.rows;
        const float *right = right_tile + k_base * a.width;
#pragma unroll
        for (int pair = 0; pair < 4; ++pair) {
            const float *left_source = left + static_cast<size_t>(2 * pair) * a.rows + left_lane;
            const float *right_source = right + static_cast<size_t>(2 * pair) * a.width + right_lane;
            const int k = wave * 8 + 2 * pair;
            if constexpr (odd.value) {
                rows_to_lds(left_source, &deviation_odd[k][0]);
                rows_to_lds(right_source, &coefficient_odd[k][0]);
            } else {
                rows_to_lds(left_source, &deviation_even[k][0]);
                rows_to_lds(right_source, &coefficient_even[k][0]);
            }
        }
    };
    // A wavefront's own transfers have landed once its vector memory counter reads zero; the
    // barrier that follows extends that to the whole workgroup.
    auto landed = [&]() __attribute__((always_inline)) {
        wait_for_loads();
        __syncthreads();
    };

    fetch(0, std::false_type{});
    landed();

    const uint32_t left_read = (lane >> 5) * kDeviationStride + wave_row + (lane & 31);
    const uint32_t right_read = (lane >> 5) * kTileColumns + wave_column + (lane & 31);
    mk_f32x16 sums[2][2];
    auto advance = [&](int step, auto quarter, auto odd) __attribute__((always_inline)) {
        const int chunk = step % chunks_per_chain;
        if (chunk == 0) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sums[mi][ni][r] = 0.0f;
        }
        const bool more = step + 1 < steps;
        if (more) fetch(step + 1, std::bool_constant<!odd.value>{});
        if constexpr (quarter.value >= 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                totals[quarter.value >> 1][quarter.value & 1][r] = *cell(quarter.value >> 1, quarter.value & 1, r);
        }
        const float *left_rows = (odd.value ? &deviation_odd[0][0] : &deviation_even[0][0]) + left_read;
        const float *right_rows = (odd.value ? &coefficient_odd[0][0] : &coefficient_even[0][0]) + right_read;
        // The operands of the next pair of depth steps are read from LDS before this pair's
        // MFMAs are issued: both waves of a SIMD otherwise wait for LDS at the same time.
        float left0 = left_rows[0], left1 = left_rows[32];
        float right0 = right_rows[0], right1 = right_rows[32];
#pragma unroll
        for (int kk = 0; kk < kDepthChunk; kk += 2) {
            float next_left0 = 0.0f, next_left1 = 0.0f, next_right0 = 0.0f, next_right1 = 0.0f;
            if (kk + 2 < kDepthChunk) {
                next_left0 = left_rows[(kk + 2) * kDeviationStride];
                next_left1 = left_rows[(kk + 2) * kDeviationStride + 32];
                next_right0 = right_rows[(kk + 2) * kTileColumns];
                next_right1 = right_rows[(kk + 2) * kTileColumns + 32];
            }
            __builtin_amdgcn_sched_barrier(0);
            sums[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(left0, right0, sums[0][0], 0, 0, 0);
            sums[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(left0, right1, sums[0][1], 0, 0, 0);
            sums[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(left1, right0, sums[1][0], 0, 0, 0);
            sums[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(left1, right1, sums[1][1], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            left0 = next_left0, left1 = next_left1, right0 = next_right0, right1 = next_right1;
        }
        if ((quarter.value < 0 || quarter.value == 3) && chunk == chunks_per_chain - 1) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r) totals[mi][ni][r] = __fadd_rn(totals[mi][ni][r], sums[mi][ni][r]);
        }
        landed();
    };
    using None = std::integral_constant<int, -1>;
    advance(0, std::integral_constant<int, 0>{}, std::false_type{});   // the launcher guarantees chains of four steps or more
    advance(1, std::integral_constant<int, 1>{}, std::true_type{});
    advance(2, std::integral_constant<int, 2>{}, std::false_type{});
    advance(3, std::integral_constant<int, 3>{}, std::true_type{});
    int step = 4;
    for (; step + 1 < steps; step += 2) {
        advance(step, None{}, std::false_type{});
        advance(step + 1, None{}, std::true_type{});
    }
    if (step < steps) advance(step, None{}, std::false_type{});

#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) *cell(mi, ni, r) = totals[mi][ni][r];
}

// Chains of exactly 128 columns on 64 x 64 tiles.  Two uses: the update of a super-block's own
// later tiles right after a tile's sweep (one chain over at most 96 of the 128 x 128 tiles
// above, each a wavefront-serial chain of 256 MFMAs, on a GPU with 1024 SIMDs), and the last,
// partly filled round of a wide launch (a few 128 x 128 tiles would hold the whole GPU for a
// full round; as quarter tiles they spread over four times as many SIMDs).  A workgroup owns
// a 64 x 64 tile and a wavefront one 32 x 32 accumulator (64 MFMAs per chain); operands arrive
// half a chain at a time in two LDS buffers, the next half on its way while the current one is
// multiplied.  Sums are formed exactly as above (per chain: ascending k from zero, then added
// to the running total).
constexpr int kWholeChain = 128;
constexpr int kSmallTile = 64;

constexpr int kSmallDepth = 64;  // k rows per step: half a chain, two LDS buffers of 2 x 16 KB

__global__ void __launch_bounds__(kUpdateThreads) block_update_small_tile_kernel(const UpdateArgs a) {
    __shared__ __attribute__((aligned(16))) float deviation_even[kSmallDepth][kSmallTile];     // [k][row]
    __shared__ __attribute__((aligned(16))) float deviation_odd[kSmallDepth][kSmallTile];
    __shared__ __attribute__((aligned(16))) float coefficient_even[kSmallDepth][kSmallTile];   // [k][column]
    __shared__ __attribute__((aligned(16))) float coefficient_odd[kSmallDepth][kSmallTile];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Quarter q of 128 x 128 tile `tile_first + b / 4` (the same linear order as the large kernel).
    const int large = a.tile_first + (blockIdx.x >> 2), quarter = blockIdx.x & 3;
    const int large_row = large / a.column_tiles;
    const int row0 = large_row * kTileRows + (quarter >> 1) * kSmallTile;
    const int column0 = a.column_begin + (large - large_row * a.column_tiles) * kTileColumns + (quarter & 1) * kSmallTile;
    const int wave_row = (wave >> 1) * 32, wave_column = (wave & 1) * 32;

    // One instruction moves four k rows of a tile (4 x 64 floats; lane l's 16 bytes land at
    // 16 l from the uniform LDS address); per step a wavefront moves k rows 16 wave ... 16 wave + 15.
    const uint32_t left_lane = static_cast<uint32_t>(lane >> 4) * a.rows + (lane & 15) * 4;
    const uint32_t right_lane = static_cast<uint32_t>(lane >> 4) * a.width + (lane & 15) * 4;
    auto fetch = [&](int step, auto odd) __attribute__((always_inline)) {
        const size_t k_base = static_cast<size_t>(a.first_column + step * kSmallDepth + wave * 16);  // chains are adjacent
        const float *left = a.deviation_t + row0 + k_base * a.rows;
        const float *right = a.coeff + column0 + k_base * a.width;
#pragma unroll
        for (int four = 0; four < 4; ++four) {
            const int k = wave * 16 + 4 * four;
            rows_to_lds(left + static_cast<size_t>(4 * four) * a.rows + left_lane,
                        odd.value ? &deviation_odd[k][0] : &deviation_even[k][0]);
            rows_to_lds(right + static_cast<size_t>(4 * four) * a.width + right_lane,
                        odd.value ? &coefficient_odd[k][0] : &coefficient_even[k][0]);
        }
    };
    const int steps = a.chains * (kWholeChain / kSmallDepth);
    fetch(0, std::false_type{});

    // This lane's cells of the 32 x 32 tile: rows (lane / 32) * 4 + ..., column lane % 32.
    float *cells = a.feedback + static_cast<size_t>(row0 + wave_row + (lane >> 5) * 4) * a.width + column0 + wave_column + (lane & 31);
    mk_f32x16 totals, sums;
#pragma unroll
    for (int r = 0; r < 16; ++r) totals[r] = cells[static_cast<size_t>((r >> 2) * 8 + (r & 3)) * a.width];

    const uint32_t left_read = (lane >> 5) * kSmallTile + wave_row + (lane & 31);
    const uint32_t right_read = (lane >> 5) * kSmallTile + wave_column + (lane & 31);
    auto advance = [&](int step, auto odd) __attribute__((always_inline)) {
        // The step's operands have landed for every wavefront, and every wavefront is done
        // reading the other buffer (the step before): the next step's operands may overwrite it.
        wait_for_loads();
        __syncthreads();
        if (step + 1 < steps) fetch(step + 1, std::bool_constant<!odd.value>{});
        if ((step & 1) == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sums[r] = 0.0f;
        }
        const float *left_rows = (odd.value ? &deviation_odd[0][0] : &deviation_even[0][0]) + left_read;
        const float *right_rows = (odd.value ? &coefficient_odd[0][0] : &coefficient_even[0][0]) + right_read;
#pragma unroll 16
        for (int kk = 0; kk < kSmallDepth; kk += 2)
            sums = __builtin_amdgcn_mfma_f32_32x32x2f32(left_rows[kk * kSmallTile], right_rows[kk * kSmallTile], sums, 0, 0, 0);
        if (step & 1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) totals[r] = __fadd_rn(totals[r], sums[r]);
        }
    };
    for (int step = 0; step < steps; step += 2) {  // a chain is two steps
        advance(step, std::false_type{});
        advance(step + 1, std::true_type{});
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) cells[static_cast<size_t>((r >> 2) * 8 + (r & 3)) * a.width] = totals[r];
}

// Workgroup slots of block_update_from_deviations_kernel on the whole GPU (two per CU).
constexpr int kUpdateSlots = 512;

int launch_update(UpdateArgs a, hipStream_t stream) {
    MK_REQUIRE(mk_cdiv(a.rows, kTileRows) <= 65535, MK_ERR_UNSUPPORTED, "mk_feedback_block_update: too many rows");
    const dim3 grid(mk_cdiv(a.column_end - a.column_begin, kTileColumns), mk_cdiv(a.rows, kTileRows));
    a.tile_first = 0;
    a.column_tiles = static_cast<int>(grid.x);
    const auto aligned = [](const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15u) == 0; };
    const bool vec = a.width % 4 == 0 && a.first_column % 4 == 0 && a.chain_width % 4 == 0 && a.column_begin % 4 == 0 &&
                     aligned(a.original) && aligned(a.output) && aligned(a.coeff);
    // The deviation buffer path handles whole tiles only.
    const bool staged = a.deviation_t && aligned(a.deviation_t) && aligned(a.coeff) && a.rows % kTileRows == 0 &&
                        a.width % 4 == 0 && a.column_begin % 4 == 0 &&
                        (a.column_end - a.column_begin) % kTileColumns == 0 && a.chain_width % kDepthChunk == 0 &&
                        a.chain_width / kDepthChunk >= 4;   // the first chain spans the four steps that read feedback
    // (launches that leave most of the GPU idle with 128 x 128 tiles)
    const unsigned tiles = grid.x * grid.y;
    if (staged && a.chains == 1 && a.chain_width == kWholeChain && tiles <= 128) {
        hipLaunchKernelGGL(block_update_small_tile_kernel, dim3(tiles * 4), dim3(kUpdateThreads), 0, stream, a);
    } else if (staged) {
        // Whole rounds of workgroup slots on 128 x 128 tiles; a last round that would fill at most
        // half of the slots runs as quarter tiles instead (chains of 128 columns only).
        const unsigned tail = tiles % kUpdateSlots;
        const bool split = a.chain_width == kWholeChain && tail > 0 && tail <= kUpdateSlots / 2;
        const unsigned whole = split ? tiles - tail : tiles;
        if (whole) hipLaunchKernelGGL(block_update_from_deviations_kernel, dim3(whole), dim3(kUpdateThreads), 0, stream, a);
        if (split) {
            a.tile_first = static_cast<int>(whole);
            hipLaunchKernelGGL(block_update_small_tile_kernel, dim3(tail * 4), dim3(kUpdateThreads), 0, stream, a);
        }
    } else if (vec)
        hipLaunchKernelGGL((block_update_kernel<true>), grid, dim3(kUpdateThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((block_update_kernel<false>), grid, dim3(kUpdateThreads), 0, stream, a);
    return MK_OK;
}

int check_tile(const char *name, int rows, int width, int tile_start, int tile_width) {
    MK_REQUIRE(rows >= 1 && width >= 1, MK_ERR_INVALID, "%s: sizes must be positive", name);
    MK_REQUIRE(tile_start >= 0 && tile_width >= 1 && tile_start + tile_width <= width, MK_ERR_INVALID,
               "%s: columns [%d, %d) lie outside a row of %d", name, tile_start, tile_start + tile_width, width);
    MK_REQUIRE(tile_width <= 1024, MK_ERR_UNSUPPORTED, "%s: at most 1024 columns per call (got %d)", name, tile_width);
    return MK_OK;
}

}  // namespace

extern "C" int mk_feedback_round_tile(const float *original, const float *feedback, const float *coeff,
                                      const float *scales, const float *zeros, const float *values, int n_values,
                                      float *output, uint8_t *encoded, int rows, int width, int region_start,
                                      int tile_start, int tile_width, int group, int groups_per_row,
                                      int integer_grid, float code_min, float code_max, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(original && feedback && coeff && scales && output && encoded, MK_ERR_INVALID,
               "mk_feedback_round_tile: null tensor pointer");
    if (int status = check_tile("mk_feedback_round_tile", rows, width, tile_start, tile_width)) return status;
    MK_REQUIRE(group >= 1 && region_start >= 0 && region_start <= tile_start, MK_ERR_INVALID,
               "mk_feedback_round_tile: the tile must start inside its region");
    MK_REQUIRE((tile_start + tile_width - 1 - region_start) / group < groups_per_row, MK_ERR_INVALID,
               "mk_feedback_round_tile: %d scale groups per row do not reach column %d of the region", groups_per_row,
               tile_start + tile_width - 1 - region_start);
    SweepArgs a{};
    a.original = original; a.feedback = feedback; a.coeff = coeff; a.scales = scales; a.zeros = zeros;
    a.values = values; a.output = output; a.encoded = encoded; a.rows = rows; a.width = width;
    a.region_start = region_start; a.tile_start = tile_start; a.tile_width = tile_width; a.group = group;
    a.groups_per_row = groups_per_row; a.n_values = n_values; a.code_min = code_min; a.code_max = code_max;
    if (integer_grid) {
        MK_REQUIRE(code_max >= code_min && code_max - code_min <= 255.0f, MK_ERR_INVALID,
                   "mk_feedback_round_tile: integer grid must span at most 256 codes");
        launch_sweep<kModeInteger>(a, stream);
    } else {
        MK_REQUIRE(values && n_values >= 1 && n_values <= 256, MK_ERR_INVALID,
                   "mk_feedback_round_tile: a value table of 1..256 entries is required");
        launch_sweep<kModeCodebook>(a, stream);
    }
    MK_LAUNCH_CHECK("mk_feedback_round_tile");
    return MK_OK;
}

extern "C" int mk_feedback_pending(const float *feedback, const float *coeff, const float *original, float *out,
                                   int rows, int width, int region_start, int region_stop, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(feedback && coeff && out, MK_ERR_INVALID, "mk_feedback_pending: null tensor pointer");
    if (int status = check_tile("mk_feedback_pending", rows, width, region_start, region_stop - region_start)) return status;
    SweepArgs a{};
    a.original = original; a.feedback = feedback; a.coeff = coeff; a.output = out; a.rows = rows; a.width = width;
    a.region_start = region_start; a.tile_start = region_start; a.tile_width = region_stop - region_start;
    a.group = 1; a.groups_per_row = 0;
    launch_sweep<kModeSolve>(a, stream);
    MK_LAUNCH_CHECK("mk_feedback_pending");
    return MK_OK;
}

extern "C" int mk_feedback_block_update_range(float *feedback, const float *original, const float *output,
                                              const float *coeff, int rows, int width, int first_column,
                                              int chain_width, int chains, int column_begin, int column_end,
                                              void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(feedback && original && output && coeff, MK_ERR_INVALID, "mk_feedback_block_update: null tensor pointer");
    MK_REQUIRE(rows >= 1 && width >= 1 && first_column >= 0 && chain_width >= 1 && chains >= 1 &&
                   first_column + static_cast<long long>(chain_width) * chains <= width,
               MK_ERR_INVALID, "mk_feedback_block_update: %d chains of %d columns from column %d lie outside a row of %d",
               chains, chain_width, first_column, width);
    MK_REQUIRE(column_begin >= first_column + chain_width * chains && column_end <= width, MK_ERR_INVALID,
               "mk_feedback_block_update: updated columns [%d, %d) must follow the chains and lie inside the row",
               column_begin, column_end);
    if (column_begin >= column_end) return MK_OK;
    UpdateArgs a{feedback, original, output, coeff, rows, width, first_column, chain_width, chains, column_begin, column_end, nullptr};
    if (int status = launch_update(a, stream)) return status;
    MK_LAUNCH_CHECK("mk_feedback_block_update");
    return MK_OK;
}

extern "C" int mk_feedback_block_update_staged(float *feedback, const float *deviations, const float *coeff, int rows,
                                               int width, int first_column, int chain_width, int chains,
                                               int column_begin, int column_end, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(feedback && deviations && coeff, MK_ERR_INVALID, "mk_feedback_block_update_staged: null tensor pointer");
    MK_REQUIRE(rows >= 1 && width >= 1 && first_column >= 0 && chain_width >= 1 && chains >= 1 &&
                   first_column + static_cast<long long>(chain_width) * chains <= width,
               MK_ERR_INVALID, "mk_feedback_block_update_staged: %d chains of %d columns from column %d lie outside a row of %d",
               chains, chain_width, first_column, width);
    MK_REQUIRE(column_begin >= first_column + chain_width * chains && column_end <= width, MK_ERR_INVALID,
               "mk_feedback_block_update_staged: updated columns [%d, %d) must follow the chains and lie inside the row",
               column_begin, column_end);
    if (column_begin >= column_end) return MK_OK;
    const auto aligned = [](const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15u) == 0; };
    MK_REQUIRE(aligned(deviations) && aligned(coeff) && rows % kTileRows == 0 && width % 4 == 0 && column_begin % 4 == 0 &&
                   (column_end - column_begin) % kTileColumns == 0 && chain_width % kDepthChunk == 0 &&
                   chain_width / kDepthChunk >= 4,
               MK_ERR_UNSUPPORTED,
               "mk_feedback_block_update_staged: whole %d x %d tiles, chains of at least %d columns and 16-byte aligned "
               "operands are required; use mk_feedback_block_update_range otherwise",
               kTileRows, kTileColumns, 4 * kDepthChunk);
    UpdateArgs a{feedback, nullptr, nullptr, coeff, rows, width, first_column, chain_width, chains, column_begin, column_end,
                 deviations};
    if (int status = launch_update(a, stream)) return status;
    MK_LAUNCH_CHECK("mk_feedback_block_update_staged");
    return MK_OK;
}

extern "C" int mk_feedback_block_update(float *feedback, const float *original, const float *output,
                                        const float *coeff, int rows, int width, int tile_start, int tile_stop,
                                        void *stream) {
    MK_REQUIRE(tile_start >= 0 && tile_start < tile_stop && tile_stop <= width, MK_ERR_INVALID,
               "mk_feedback_block_update: columns [%d, %d) lie outside a row of %d", tile_start, tile_stop, width);
    return mk_feedback_block_update_range(feedback, original, output, coeff, rows, width, tile_start,
                                          tile_stop - tile_start, 1, tile_stop, width, stream);
}

// The whole natural-order sweep of a layer, enqueued from here so that a region costs a few
// kernel launches and no host round trips: per region the pending-continuation solve into
// `workspace`, the scale fit on those targets, then per tile the column sweep and the
// (deferred, chained) trailing updates.
extern "C" int mk_feedback_sweep(const float *original, float *feedback, float *output, uint8_t *encoded,
                                 const float *coeff, float *scales, float *zeros, float *workspace,
                                 float *deviations, const float *values, int n_values, int rows, int width,
                                 int group, int refit,
                                 int block, int integer_grid, float code_min, float code_max, int asym,
                                 float reciprocal, float value_minimum, int scale_format, int deferred_tiles,
                                 void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(original && feedback && output && encoded && coeff && scales && (!asym || zeros), MK_ERR_INVALID,
               "mk_feedback_sweep: null tensor pointer");
    MK_REQUIRE(rows >= 1 && width >= 1 && group >= 1 && block >= 1 && block <= 1024 && refit >= 1 && deferred_tiles >= 1,
               MK_ERR_INVALID, "mk_feedback_sweep: sizes must be positive and tiles at most 1024 columns wide");
    MK_REQUIRE(refit >= width || (refit <= 1024 && workspace), MK_ERR_INVALID,
               "mk_feedback_sweep: regions of %d columns need a workspace and at most 1024 columns", refit);
    if (integer_grid) {
        MK_REQUIRE(code_max >= code_min && code_max - code_min <= 255.0f, MK_ERR_INVALID,
                   "mk_feedback_sweep: integer grid must span at most 256 codes");
    } else {
        MK_REQUIRE(values && n_values >= 1 && n_values <= 256, MK_ERR_INVALID,
                   "mk_feedback_sweep: a value table of 1..256 entries is required");
    }
    const int region_width = refit < width ? refit : width;
    long long total_groups = 0;
    for (int start = 0; start < width; start += region_width) {
        const int span = width - start < region_width ? width - start : region_width;
        total_groups += mk_cdiv(span, group < span ? group : span);
    }
    MK_REQUIRE(total_groups < (1ll << 31) / rows, MK_ERR_INVALID, "mk_feedback_sweep: too many scale groups");

    struct Tile { int start, stop; };
    Tile deferred[64];
    int deferred_count = 0, limit = 0;
    auto update = [&](int first, int chain, int chains, int begin, int end) -> int {
        if (begin >= end) return MK_OK;
        UpdateArgs u{feedback, original, output, coeff, rows, width, first, chain, chains, begin, end, deviations};
        return launch_update(u, stream);
    };
    auto flush = [&]() -> int {
        int index = 0;
        while (index < deferred_count) {
            const int chain = deferred[index].stop - deferred[index].start;
            int run = index + 1;
            while (run < deferred_count && deferred[run].stop - deferred[run].start == chain) ++run;
            if (int status = update(deferred[index].start, chain, run - index, limit, width)) return status;
            index = run;
        }
        deferred_count = 0;
        return MK_OK;
    };

    long long group_offset = 0;
    for (int region_start = 0; region_start < width; region_start += region_width) {
        const int region_stop = region_start + region_width < width ? region_start + region_width : width;
        const int span = region_stop - region_start;
        const int fitted_group = group < span ? group : span;
        const int region_groups = mk_cdiv(span, fitted_group);
        if (deferred_count && region_stop > limit)
            if (int status = flush()) return status;
        if (!deferred_count) {
            limit = region_start + deferred_tiles * block;
            if (limit < region_stop) limit = region_stop;
            if (limit > width) limit = width;
        }
        float *region_scales = scales + group_offset;
        float *region_zeros = asym ? zeros + group_offset : nullptr;
        const bool fused = region_fusable(span, block, fitted_group, integer_grid != 0, n_values) && scale_format >= 0 &&
                           scale_format <= 4;
        if (fused) {
            // fitted inside the sweep kernel below
        } else if (region_start == 0) {
            if (int status = mk_fit_scales_strided(original, width, region_scales, region_zeros, total_groups, rows, span,
                                                   fitted_group, asym, reciprocal, value_minimum, scale_format, 1, stream))
                return status;
        } else {
            SweepArgs solve{};
            solve.original = original; solve.feedback = feedback; solve.coeff = coeff; solve.output = workspace;
            solve.rows = rows; solve.width = width; solve.region_start = region_start; solve.tile_start = region_start;
            solve.tile_width = span; solve.group = 1;
            launch_sweep<kModeSolve>(solve, stream);
            if (int status = mk_fit_scales_strided(workspace, span, region_scales, region_zeros, total_groups, rows, span,
                                                   fitted_group, asym, reciprocal, value_minimum, scale_format, 1, stream))
                return status;
        }
        for (int tile_start = region_start; tile_start < region_stop; tile_start += block) {
            const int tile_stop = tile_start + block < region_stop ? tile_start + block : region_stop;
            SweepArgs a{};
            a.original = original; a.feedback = feedback; a.coeff = coeff; a.scales = region_scales;
            a.zeros = region_zeros; a.values = values; a.output = output; a.encoded = encoded; a.rows = rows;
            a.width = width; a.region_start = region_start; a.tile_start = tile_start;
            a.tile_width = tile_stop - tile_start; a.group = fitted_group;
            a.groups_per_row = static_cast<int>(total_groups); a.n_values = n_values;
            a.code_min = code_min; a.code_max = code_max; a.deviation_t = deviations;
            if (fused) {
                a.fit_scales = region_scales; a.fit_zeros = region_zeros; a.solve_first = region_start != 0;
                a.asym = asym; a.scale_format = scale_format; a.reciprocal = reciprocal; a.value_minimum = value_minimum;
                launch_region(a, integer_grid != 0, stream);
            } else if (integer_grid) launch_sweep<kModeInteger>(a, stream);
            else launch_sweep<kModeCodebook>(a, stream);
            if (tile_stop >= width) continue;
            if (tile_stop < limit)
                if (int status = update(tile_start, tile_stop - tile_start, 1, tile_stop, limit)) return status;
            if (limit < width) {
                deferred[deferred_count].start = tile_start;
                deferred[deferred_count].stop = tile_stop;
                ++deferred_count;
                if (tile_stop >= limit || deferred_count == 64)
                    if (int status = flush()) return status;
            }
        }
        group_offset += region_groups;
    }
    MK_LAUNCH_CHECK("mk_feedback_sweep");
    return MK_OK;
}
