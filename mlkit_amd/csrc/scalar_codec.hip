// Scalar grouped-scale codec on gfx950: nearest-code encoding, decoding of unpacked codes,
// the shrunken-scale search and snapping to a codebook.
//
// Everything here is compared bit for bit with IEEE binary32 tensor arithmetic, so each
// operation is spelled as a separately rounded one (this file is also compiled with
// -ffp-contract=off): true division, round half to even, multiply then add.
//
// Replaces, in /root/reference/src/mlkit/kernels:
//   scalar_encode.py:65-146    encode_scalar_codes / encode        -> mk_scalar_encode
//   scalar_encode.py:149-304   search_group_scales / search_scales -> mk_search_scales
//   scalar_encode.py:307-345   snap_to_codebook / snap             -> mk_snap
//   scalar_decode.py:37-97     decode_scalar_codes / decode        -> mk_scalar_decode
//   scalar_rounding.py:15-73   rounding helpers (device functions below)

#include "mk_common.h"
#include "packed_matvec_impl.h"   // lane_exchange

namespace {

constexpr int kMaxTable = 256;
constexpr int kThreads = 256;

// Index of the first table entry >= x by bisection over a table padded with +inf, then
// the nearer of that entry and the one below it; equal distances pick the lower entry.
__device__ __forceinline__ int nearest_entry(float x, const float *table, int count, int steps) {
    int lower = 0, upper = count;
    for (int s = 0; s < steps; ++s) {
        const int middle = (lower + upper) >> 1;
        const float candidate = middle < count ? table[middle] : __builtin_inff();
        const bool right = candidate < x;
        lower = right ? middle + 1 : lower;
        upper = right ? upper : middle;
    }
    const int above = lower < count - 1 ? lower : count - 1;
    const int below = above > 0 ? above - 1 : 0;
    const float below_distance = fabsf(__fsub_rn(x, table[below]));
    const float above_distance = fabsf(__fsub_rn(x, table[above]));
    return below_distance <= above_distance ? below : above;
}

__device__ __forceinline__ float nearest_integer(float x, float minimum, float maximum) {
    return fminf(fmaxf(rintf(x), minimum), maximum);
}

__device__ __forceinline__ int bisection_steps(int count) {
    int steps = 0;
    while ((1 << steps) < count + 1) ++steps;
    return steps;
}

__device__ __forceinline__ void stage_table(float *shared, const float *values, int count) {
    for (int i = threadIdx.x; i < count; i += blockDim.x) shared[i] = values[i];
    __syncthreads();
}

struct CodecArgs {
    const float *value;
    const float *scales;
    const float *zeros;
    const float *values;
    const uint8_t *codes_in;
    uint8_t *codes_out;
    float *out;
    int rows, width, group, groups_per_row, refit, groups_per_region;
    int n_values, integer;
    float minimum, maximum;
};

__device__ __forceinline__ int scale_slot(const CodecArgs &a, int column) {
    if (a.refit == 0) return column / a.group;
    const int region = column / a.refit;
    return region * a.groups_per_region + (column - region * a.refit) / a.group;
}

// One thread encodes VEC adjacent elements of a row; blockIdx.y strides over rows.
template <int VEC>
__global__ void __launch_bounds__(kThreads) encode_kernel(const CodecArgs a) {
    __shared__ float table[kMaxTable];
    if (!a.integer) stage_table(table, a.values, a.n_values);
    const int steps = bisection_steps(a.n_values);
    const int column = (blockIdx.x * kThreads + threadIdx.x) * VEC;
    if (column >= a.width) return;
    const bool one_slot = a.group % VEC == 0;
    if constexpr (VEC == 4) {
        if (one_slot) {
            // Four rows per trip, all their loads issued before the first is used.
            constexpr int kRowsPerTrip = 4;
            const int group_index = column / a.group;
            for (int first = blockIdx.y; first < a.rows; first += kRowsPerTrip * gridDim.y) {
                float4 loaded[kRowsPerTrip];
                float scale[kRowsPerTrip], zero[kRowsPerTrip];
#pragma unroll
                for (int u = 0; u < kRowsPerTrip; ++u) {
                    const int wanted = first + u * static_cast<int>(gridDim.y);
                    const int row = wanted < a.rows ? wanted : first;
                    loaded[u] = *reinterpret_cast<const float4 *>(a.value + static_cast<size_t>(row) * a.width + column);
                    const int slot = row * a.groups_per_row + group_index;
                    scale[u] = a.scales[slot];
                    zero[u] = a.zeros ? a.zeros[slot] : 0.0f;
                }
#pragma unroll
                for (int u = 0; u < kRowsPerTrip; ++u) {
                    const int row = first + u * static_cast<int>(gridDim.y);
                    const float sample[4] = {loaded[u].x, loaded[u].y, loaded[u].z, loaded[u].w};
                    uint32_t packed = 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float centered = sample[i];
                        if (a.zeros) centered = __fsub_rn(centered, zero[u]);
                        const float normalized = __fdiv_rn(centered, scale[u]);
                        int index;
                        if (a.integer)
                            index = static_cast<int>(__fsub_rn(nearest_integer(normalized, a.minimum, a.maximum), a.minimum));
                        else
                            index = nearest_entry(normalized, table, a.n_values, steps);
                        packed |= static_cast<uint32_t>(index & 255) << (8 * i);
                    }
                    if (row < a.rows)
                        *reinterpret_cast<uint32_t *>(a.codes_out + static_cast<size_t>(row) * a.width + column) = packed;
                }
            }
            return;
        }
    }
    for (int row = blockIdx.y; row < a.rows; row += gridDim.y) {
        const size_t base = static_cast<size_t>(row) * a.width + column;
        float sample[VEC];
        if constexpr (VEC == 4) {
            const float4 loaded = *reinterpret_cast<const float4 *>(a.value + base);
            sample[0] = loaded.x; sample[1] = loaded.y; sample[2] = loaded.z; sample[3] = loaded.w;
        } else {
            sample[0] = a.value[base];
        }
        uint32_t packed = 0;
        int slot = row * a.groups_per_row + column / a.group;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            if (!one_slot && i) slot = row * a.groups_per_row + (column + i) / a.group;
            float centered = sample[i];
            if (a.zeros) centered = __fsub_rn(centered, a.zeros[slot]);
            const float normalized = __fdiv_rn(centered, a.scales[slot]);
            int index;
            if (a.integer)
                index = static_cast<int>(__fsub_rn(nearest_integer(normalized, a.minimum, a.maximum), a.minimum));
            else
                index = nearest_entry(normalized, table, a.n_values, steps);
            packed |= static_cast<uint32_t>(index & 255) << (8 * i);
        }
        if constexpr (VEC == 4)
            *reinterpret_cast<uint32_t *>(a.codes_out + base) = packed;
        else
            a.codes_out[base] = static_cast<uint8_t>(packed);
    }
}

template <int VEC>
__global__ void __launch_bounds__(kThreads) decode_kernel(const CodecArgs a) {
    __shared__ float table[kMaxTable];
    stage_table(table, a.values, a.n_values);
    const int column = (blockIdx.x * kThreads + threadIdx.x) * VEC;
    if (column >= a.width) return;
    const bool one_slot = a.refit == 0 && a.group % VEC == 0;
    const int limit = a.n_values - 1;
    if constexpr (VEC == 4) {
        if (one_slot) {
            // Four rows per trip, all their loads issued before the first is used.
            constexpr int kRowsPerTrip = 4;
            const int group_index = column / a.group;
            for (int first = blockIdx.y; first < a.rows; first += kRowsPerTrip * gridDim.y) {
                uint32_t packed[kRowsPerTrip];
                float scale[kRowsPerTrip], zero[kRowsPerTrip];
#pragma unroll
                for (int u = 0; u < kRowsPerTrip; ++u) {
                    const int wanted = first + u * static_cast<int>(gridDim.y);
                    const int row = wanted < a.rows ? wanted : first;
                    packed[u] = *reinterpret_cast<const uint32_t *>(a.codes_in + static_cast<size_t>(row) * a.width + column);
                    const int slot = row * a.groups_per_row + group_index;
                    scale[u] = a.scales[slot];
                    zero[u] = a.zeros ? a.zeros[slot] : 0.0f;
                }
#pragma unroll
                for (int u = 0; u < kRowsPerTrip; ++u) {
                    const int row = first + u * static_cast<int>(gridDim.y);
                    float weight[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int code = static_cast<int>((packed[u] >> (8 * i)) & 255u);
                        weight[i] = __fmul_rn(table[code < limit ? code : limit], scale[u]);
                        if (a.zeros) weight[i] = __fadd_rn(weight[i], zero[u]);
                    }
                    if (row < a.rows)
                        *reinterpret_cast<float4 *>(a.out + static_cast<size_t>(row) * a.width + column) =
                            make_float4(weight[0], weight[1], weight[2], weight[3]);
                }
            }
            return;
        }
    }
    for (int row = blockIdx.y; row < a.rows; row += gridDim.y) {
        const size_t base = static_cast<size_t>(row) * a.width + column;
        uint32_t packed;
        if constexpr (VEC == 4)
            packed = *reinterpret_cast<const uint32_t *>(a.codes_in + base);
        else
            packed = a.codes_in[base];
        float weight[VEC];
        int slot = row * a.groups_per_row + scale_slot(a, column);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            if (!one_slot && i) slot = row * a.groups_per_row + scale_slot(a, column + i);
            const int code = static_cast<int>((packed >> (8 * i)) & 255u);
            weight[i] = __fmul_rn(table[code < limit ? code : limit], a.scales[slot]);
            if (a.zeros) weight[i] = __fadd_rn(weight[i], a.zeros[slot]);
        }
        if constexpr (VEC == 4)
            *reinterpret_cast<float4 *>(a.out + base) = make_float4(weight[0], weight[1], weight[2], weight[3]);
        else
            a.out[base] = weight[0];
    }
}

__global__ void __launch_bounds__(kThreads) snap_kernel(const float *value, const float *values, int n_values,
                                                        float *out, size_t count) {
    __shared__ float table[kMaxTable];
    stage_table(table, values, n_values);
    const int steps = bisection_steps(n_values);
    for (size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; i < count;
         i += static_cast<size_t>(gridDim.x) * kThreads)
        out[i] = table[nearest_entry(value[i], table, n_values, steps)];
}

struct SearchArgs {
    const float *value;
    const float *scales;
    const float *zeros;
    const float *values;
    const float *fractions;
    float *selected;
    int rows, width, group, groups_per_row;
    int n_values, n_fractions, format, integer;
    float minimum, maximum;
    int total_groups;
};

// A team of LANES adjacent lanes owns one (row, group).  Lane p adds the squared errors of
// elements p, p + LANES, ... in ascending order; the LANES partial sums are then folded by
// halving (s[i] += s[i + h], h = LANES/2 ... 1), which a butterfly over lane indices
// reproduces in every lane because fp32 addition is commutative.
template <int LANES>
__device__ __forceinline__ float team_error(const SearchArgs &a, const float *table, int steps,
                                            const float *row_value, int group_start, int lane_in_team,
                                            float scale, float zero) {
    float error = 0.0f;
    for (int within = lane_in_team; within < a.group; within += LANES) {
        const int column = group_start + within;
        const bool valid = column < a.width;
        const float centered = __fsub_rn(valid ? row_value[column] : 0.0f, zero);
        const float normalized = __fdiv_rn(centered, scale);
        float rounded;
        if (a.integer)
            rounded = nearest_integer(normalized, a.minimum, a.maximum);
        else
            rounded = table[nearest_entry(normalized, table, a.n_values, steps)];
        const float difference = valid ? __fsub_rn(__fmul_rn(rounded, scale), centered) : 0.0f;
        error = __fadd_rn(error, __fmul_rn(difference, difference));
    }
    return mk_segment_sum<LANES>(error);
}

template <int LANES>
__global__ void __launch_bounds__(kThreads) search_kernel(const SearchArgs a) {
    __shared__ float table[kMaxTable];
    __shared__ float fraction[64];
    if (!a.integer) stage_table(table, a.values, a.n_values);
    for (int i = threadIdx.x; i < a.n_fractions; i += blockDim.x) fraction[i] = a.fractions[i];
    __syncthreads();
    const int steps = bisection_steps(a.n_values);
    constexpr int kTeams = kThreads / LANES;
    const int lane_in_team = threadIdx.x % LANES;
    // Every lane of a wavefront runs the same trip count: teams past the end recompute the
    // last group and do not store.
    for (int first = blockIdx.x * kTeams; first < a.total_groups; first += gridDim.x * kTeams) {
        const int wanted = first + threadIdx.x / LANES;
        const int identifier = wanted < a.total_groups ? wanted : a.total_groups - 1;
        const int row = identifier / a.groups_per_row;
        const int group_start = (identifier - row * a.groups_per_row) * a.group;
        const float *row_value = a.value + static_cast<size_t>(row) * a.width;
        const float base = a.scales[identifier];
        const float zero = a.zeros ? a.zeros[identifier] : 0.0f;
        float best_scale = base;
        float best_error = team_error<LANES>(a, table, steps, row_value, group_start, lane_in_team, base, zero);
        for (int c = 0; c < a.n_fractions; ++c) {
            const float scale = mk_rounded_scale(__fmul_rn(base, fraction[c]), a.format);
            const float error = team_error<LANES>(a, table, steps, row_value, group_start, lane_in_team, scale, zero);
            const bool improved = error < best_error;
            best_scale = improved ? scale : best_scale;
            best_error = fminf(best_error, error);
        }
        if (lane_in_team == 0 && wanted < a.total_groups) a.selected[identifier] = best_scale;
    }
}

// The same sums with four (or two) adjacent partial sums of a group in one lane: a team of LANES / V lanes owns a
// group, lane q the partial sums 4 q ... 4 q + 3 (elements 4 q ... 4 q + 3, + LANES, + 2 LANES, ...: one vector load
// each).  The butterfly's first stages (partners 1 and 2 apart) are then additions inside a lane, in the same
// order, and the rest runs over the team: bit for bit the result of search_kernel<LANES>, with the group's values
// held in registers across the candidates and a quarter of the exchanges, scale roundings and comparisons per
// element.  For groups of at most 256 values (at most sixteen registers of them per lane).
template <int LANES, int V>
__global__ void __launch_bounds__(kThreads) search_kernel_in_registers(const SearchArgs a) {
    static_assert(LANES % V == 0 && (V == 4 || V == 2), "two or four partial sums per lane");
    constexpr int kTeam = LANES / V;
    constexpr int kMaxTrips = 256 / LANES;   // elements per partial sum
    __shared__ float table[kMaxTable];
    __shared__ float fraction[64];
    if (!a.integer) stage_table(table, a.values, a.n_values);
    for (int i = threadIdx.x; i < a.n_fractions; i += blockDim.x) fraction[i] = a.fractions[i];
    __syncthreads();
    const int steps = bisection_steps(a.n_values);
    constexpr int kTeams = kThreads / kTeam;
    const int lane_in_team = threadIdx.x % kTeam;
    const int trips = a.group / LANES;   // uniform; at most kMaxTrips
    for (int first = blockIdx.x * kTeams; first < a.total_groups; first += gridDim.x * kTeams) {
        const int wanted = first + threadIdx.x / kTeam;
        const int identifier = wanted < a.total_groups ? wanted : a.total_groups - 1;
        const int row = identifier / a.groups_per_row;
        const int group_start = (identifier - row * a.groups_per_row) * a.group;
        const float *row_value = a.value + static_cast<size_t>(row) * a.width;
        const float base = a.scales[identifier];
        const float zero = a.zeros ? a.zeros[identifier] : 0.0f;
        float centered[kMaxTrips][V];
        bool valid[kMaxTrips][V];
#pragma unroll
        for (int k = 0; k < kMaxTrips; ++k)
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const int column = group_start + k * LANES + lane_in_team * V + v;
                valid[k][v] = k < trips && column < a.width;
                centered[k][v] = __fsub_rn(valid[k][v] ? row_value[column] : 0.0f, zero);
            }
        auto error_of = [&](float scale) __attribute__((always_inline)) {
            float partial[V];
#pragma unroll
            for (int v = 0; v < V; ++v) partial[v] = 0.0f;
#pragma unroll
            for (int k = 0; k < kMaxTrips; ++k) {
                if (k < trips) {   // uniform
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        const float normalized = __fdiv_rn(centered[k][v], scale);
                        float rounded;
                        if (a.integer)
                            rounded = nearest_integer(normalized, a.minimum, a.maximum);
                        else
                            rounded = table[nearest_entry(normalized, table, a.n_values, steps)];
                        const float difference = valid[k][v] ? __fsub_rn(__fmul_rn(rounded, scale), centered[k][v]) : 0.0f;
                        partial[v] = __fadd_rn(partial[v], __fmul_rn(difference, difference));
                    }
                }
            }
            float folded;
            if constexpr (V == 4)
                folded = __fadd_rn(__fadd_rn(partial[0], partial[1]), __fadd_rn(partial[2], partial[3]));
            else
                folded = __fadd_rn(partial[0], partial[1]);
            return mk_segment_sum<kTeam>(folded);
        };
        float best_scale = base;
        float best_error = error_of(base);
        for (int c = 0; c < a.n_fractions; ++c) {
            const float scale = mk_rounded_scale(__fmul_rn(base, fraction[c]), a.format);
            const float error = error_of(scale);
            const bool improved = error < best_error;
            best_scale = improved ? scale : best_scale;
            best_error = fminf(best_error, error);
        }
        if (lane_in_team == 0 && wanted < a.total_groups) a.selected[identifier] = best_scale;
    }
}

template <int LANES>
void launch_search(const SearchArgs &a, hipStream_t stream) {
    if constexpr (LANES >= 32) {
        if (a.group <= 256) {
            constexpr int kV = LANES == 64 ? 4 : 2;
            const int teams = kThreads / (LANES / kV);
            int blocks = mk_cdiv(a.total_groups, teams);
            if (blocks > 256 * 64) blocks = 256 * 64;
            hipLaunchKernelGGL((search_kernel_in_registers<LANES, kV>), dim3(blocks), dim3(kThreads), 0, stream, a);
            return;
        }
    }
    const int teams = kThreads / LANES;
    int blocks = mk_cdiv(a.total_groups, teams);
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL((search_kernel<LANES>), dim3(blocks), dim3(kThreads), 0, stream, a);
}

struct FitArgs {
    const float *value;
    float *scales;
    float *zeros;
    long long row_stride, out_row_stride;
    int rows, span, group, groups_per_row, total_groups;
    int asym, format, store_zero;
    float reciprocal, value_minimum;
};

// A team of LANES lanes finds one group's extrema (order does not matter for min and max)
// and lane 0 derives the stored scale and offset from them.
// Scale and offset of one group from its extrema, written by one lane.
__device__ __forceinline__ void store_fit(const FitArgs &a, size_t slot, float low, float high, bool finite) {
    if (!finite) {  // fminf/fmaxf drop NaNs: report them as the tensor reductions would
        a.scales[slot] = __builtin_nanf("");
        if (a.zeros) a.zeros[slot] = __builtin_nanf("");
        return;
    }
    float scale, zero = 0.0f;
    if (a.asym) {
        scale = __fmul_rn(fmaxf(__fsub_rn(high, low), 1e-12f), a.reciprocal);
        zero = __fsub_rn(low, __fmul_rn(a.value_minimum, scale));
    } else {
        scale = __fmul_rn(fmaxf(fmaxf(high, -low), 1e-12f), a.reciprocal);
    }
    a.scales[slot] = mk_rounded_scale(scale, a.format);
    if (a.zeros) {
        if (a.store_zero) {
            const float magnitude = mk_rounded_scale(fmaxf(fabsf(zero), 1e-12f), a.format);
            zero = zero > 0.0f ? magnitude : (zero < 0.0f ? -magnitude : 0.0f);
        }
        a.zeros[slot] = zero;
    }
}

// Minimum, maximum and "all finite" over the LANES adjacent lanes of a team, by vector-ALU
// lane moves (an LDS permute per step cost more than the loads of the group).
template <int LANES>
__device__ __forceinline__ void team_range(float &low, float &high, bool &finite, int lane) {
    float bad = finite ? 0.0f : 1.0f;
    auto stage = [&](auto s) __attribute__((always_inline)) {
        constexpr int S = decltype(s)::value;
        if constexpr ((1 << S) < LANES) {
            low = fminf(low, mk_matvec::lane_exchange<S>(low, lane));
            high = fmaxf(high, mk_matvec::lane_exchange<S>(high, lane));
            bad = fmaxf(bad, mk_matvec::lane_exchange<S>(bad, lane));
        }
    };
    stage(std::integral_constant<int, 0>{});
    stage(std::integral_constant<int, 1>{});
    stage(std::integral_constant<int, 2>{});
    stage(std::integral_constant<int, 3>{});
    stage(std::integral_constant<int, 4>{});
    stage(std::integral_constant<int, 5>{});
    finite = bad == 0.0f;
}

template <int LANES>
__global__ void __launch_bounds__(kThreads) fit_kernel(const FitArgs a) {
    constexpr int kTeams = kThreads / LANES;
    const int lane_in_team = threadIdx.x % LANES;
    // Whole groups of exactly 4 * LANES values, 16-byte aligned: one float4 per lane and group,
    // four groups per trip with all four loads issued first.
    const bool single_load = a.group == 4 * LANES && a.span % a.group == 0 && a.row_stride % 4 == 0 &&
                             (reinterpret_cast<uintptr_t>(a.value) & 15u) == 0;
    if (single_load) {
        constexpr int kPerTrip = 4;
        const int team = threadIdx.x / LANES;
        const int lane = threadIdx.x & 63;
        for (int first = (blockIdx.x * kTeams + team) * kPerTrip; first < a.total_groups; first += gridDim.x * kTeams * kPerTrip) {
            // One division per trip: the trip's groups are adjacent, so their rows follow by
            // stepping (a division per group cost more than the group's arithmetic).
            int row[kPerTrip], in_row[kPerTrip];
            row[0] = first / a.groups_per_row;
            in_row[0] = first - row[0] * a.groups_per_row;
#pragma unroll
            for (int u = 1; u < kPerTrip; ++u) {
                const bool wraps = in_row[u - 1] + 1 == a.groups_per_row;
                row[u] = wraps ? row[u - 1] + 1 : row[u - 1];
                in_row[u] = wraps ? 0 : in_row[u - 1] + 1;
            }
            float4 loaded[kPerTrip];
#pragma unroll
            for (int u = 0; u < kPerTrip; ++u) {
                const bool present = first + u < a.total_groups;
                loaded[u] = *reinterpret_cast<const float4 *>(a.value + static_cast<size_t>(present ? row[u] : row[0]) * a.row_stride +
                                                              (present ? in_row[u] : in_row[0]) * a.group + 4 * lane_in_team);
            }
#pragma unroll
            for (int u = 0; u < kPerTrip; ++u) {
                const float4 v = loaded[u];
                bool finite = (v.x - v.x == 0.0f) && (v.y - v.y == 0.0f) && (v.z - v.z == 0.0f) && (v.w - v.w == 0.0f);
                float low = fminf(fminf(v.x, v.y), fminf(v.z, v.w));
                float high = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
                team_range<LANES>(low, high, finite, lane);
                if (lane_in_team == 0 && first + u < a.total_groups)
                    store_fit(a, static_cast<size_t>(row[u]) * a.out_row_stride + in_row[u], low, high, finite);
            }
        }
        return;
    }
    for (int first = blockIdx.x * kTeams; first < a.total_groups; first += gridDim.x * kTeams) {
        const int wanted = first + threadIdx.x / LANES;
        const int identifier = wanted < a.total_groups ? wanted : a.total_groups - 1;
        const int row = identifier / a.groups_per_row;
        const int start = (identifier - row * a.groups_per_row) * a.group;
        const int stop = start + a.group < a.span ? start + a.group : a.span;
        const float *row_value = a.value + static_cast<size_t>(row) * a.row_stride;
        float low = __builtin_inff(), high = -__builtin_inff();
        bool finite = true;
        // Four adjacent values per lane and step where the group allows 16-byte loads.
        const bool wide = ((reinterpret_cast<uintptr_t>(row_value + start) & 15u) == 0) && ((stop - start) & 3) == 0;
        if (wide) {
            for (int column = start + 4 * lane_in_team; column < stop; column += 4 * LANES) {
                const float4 v = *reinterpret_cast<const float4 *>(row_value + column);
                finite = finite && (v.x - v.x == 0.0f) && (v.y - v.y == 0.0f) && (v.z - v.z == 0.0f) && (v.w - v.w == 0.0f);
                low = fminf(fminf(low, fminf(v.x, v.y)), fminf(v.z, v.w));
                high = fmaxf(fmaxf(high, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
            }
        } else {
            for (int column = start + lane_in_team; column < stop; column += LANES) {
                const float v = row_value[column];
                finite = finite && v - v == 0.0f;
                low = fminf(low, v);
                high = fmaxf(high, v);
            }
        }
        team_range<LANES>(low, high, finite, threadIdx.x & 63);
        if (lane_in_team != 0 || wanted >= a.total_groups) continue;
        store_fit(a, static_cast<size_t>(row) * a.out_row_stride + (identifier - row * a.groups_per_row), low, high, finite);
    }
}

template <int LANES>
void launch_fit(const FitArgs &a, hipStream_t stream) {
    int blocks = mk_cdiv(a.total_groups, kThreads / LANES);
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL((fit_kernel<LANES>), dim3(blocks), dim3(kThreads), 0, stream, a);
}

struct ReconstructArgs {
    const void *inputs;
    void *output;
    const float *values;
    int rows, width, group, groups_per_row, total_groups;
    int dtype, n_values, format, asym, integer;
    float reciprocal, minimum, maximum;
};

// Online quantize-dequantize of activations: a team of LANES lanes owns one (row, group);
// it finds the group's range, derives the stored scale (and offset) exactly as fit_kernel
// does, then rounds every element to the grid and writes scale * value (+ offset) in the
// input's dtype.  The second pass re-reads the group from cache.
template <int LANES>
__global__ void __launch_bounds__(kThreads) reconstruct_kernel(const ReconstructArgs a) {
    __shared__ float table[kMaxTable];
    if (!a.integer) stage_table(table, a.values, a.n_values);
    const int steps = bisection_steps(a.n_values);
    constexpr int kTeams = kThreads / LANES;
    const int lane_in_team = threadIdx.x % LANES;
    for (int first = blockIdx.x * kTeams; first < a.total_groups; first += gridDim.x * kTeams) {
        const int wanted = first + threadIdx.x / LANES;
        const int identifier = wanted < a.total_groups ? wanted : a.total_groups - 1;
        const int row = identifier / a.groups_per_row;
        const int start = (identifier - row * a.groups_per_row) * a.group;
        const int stop = start + a.group < a.width ? start + a.group : a.width;
        const size_t base = static_cast<size_t>(row) * a.width;
        float low = __builtin_inff(), high = -__builtin_inff();
        for (int column = start + lane_in_team; column < stop; column += LANES) {
            const float v = mk_load_as_float(a.inputs, base + column, a.dtype);
            low = fminf(low, v);
            high = fmaxf(high, v);
        }
#pragma unroll
        for (int offset = 1; offset < LANES; offset <<= 1) {
            low = fminf(low, __shfl_xor(low, offset, 64));
            high = fmaxf(high, __shfl_xor(high, offset, 64));
        }
        float scale, zero = 0.0f;
        if (a.asym) {
            const float raw = __fmul_rn(fmaxf(__fsub_rn(high, low), 1e-12f), a.reciprocal);
            zero = __fsub_rn(low, __fmul_rn(a.minimum, raw));
            scale = mk_rounded_scale(raw, a.format);
            const float magnitude = mk_rounded_scale(fmaxf(fabsf(zero), 1e-12f), a.format);
            zero = zero > 0.0f ? magnitude : (zero < 0.0f ? -magnitude : 0.0f);
        } else {
            scale = mk_rounded_scale(__fmul_rn(fmaxf(fmaxf(high, -low), 1e-12f), a.reciprocal), a.format);
        }
        if (wanted >= a.total_groups) continue;
        for (int column = start + lane_in_team; column < stop; column += LANES) {
            const float v = mk_load_as_float(a.inputs, base + column, a.dtype);
            const float normalized = __fdiv_rn(__fsub_rn(v, zero), scale);
            const float rounded = a.integer ? nearest_integer(normalized, a.minimum, a.maximum)
                                            : table[nearest_entry(normalized, table, a.n_values, steps)];
            mk_store_from_float(a.output, base + column, a.dtype, __fadd_rn(__fmul_rn(rounded, scale), zero));
        }
    }
}

template <int LANES>
void launch_reconstruct(const ReconstructArgs &a, hipStream_t stream) {
    int blocks = mk_cdiv(a.total_groups, kThreads / LANES);
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL((reconstruct_kernel<LANES>), dim3(blocks), dim3(kThreads), 0, stream, a);
}

int check_table(const char *name, const float *values, int n_values) {
    MK_REQUIRE(values && n_values >= 1 && n_values <= kMaxTable, MK_ERR_INVALID,
               "%s: a value table of 1..256 entries is required", name);
    return MK_OK;
}

dim3 row_grid(int rows, int width, int vec) {
    const int columns = mk_cdiv(mk_cdiv(width, vec), kThreads);
    int row_blocks = mk_cdiv(256 * 16, columns);
    if (row_blocks > rows) row_blocks = rows;
    if (row_blocks > 65535) row_blocks = 65535;
    return dim3(columns, row_blocks);
}

}  // namespace

extern "C" int mk_scalar_encode(const float *value, const float *scales, const float *zeros,
                                const float *values, int n_values, uint8_t *codes, int rows, int width,
                                int group, int groups_per_row, int integer, float minimum, float maximum,
                                void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(value && scales && codes, MK_ERR_INVALID, "mk_scalar_encode: null tensor pointer");
    MK_REQUIRE(rows >= 1 && width >= 1 && group >= 1, MK_ERR_INVALID, "mk_scalar_encode: sizes must be positive");
    MK_REQUIRE(groups_per_row >= mk_cdiv(width, group), MK_ERR_INVALID,
               "mk_scalar_encode: %d scale groups per row cannot cover width %d at group %d", groups_per_row,
               width, group);
    if (integer) {
        MK_REQUIRE(maximum >= minimum && maximum - minimum <= 255.0f, MK_ERR_INVALID,
                   "mk_scalar_encode: integer grid must span at most 256 codes");
    } else if (int status = check_table("mk_scalar_encode", values, n_values)) {
        return status;
    }
    CodecArgs a{};
    a.value = value; a.scales = scales; a.zeros = zeros; a.values = values; a.codes_out = codes;
    a.rows = rows; a.width = width; a.group = group; a.groups_per_row = groups_per_row;
    a.n_values = integer ? 1 : n_values; a.integer = integer; a.minimum = minimum; a.maximum = maximum;
    const bool vector = width % 4 == 0 && (reinterpret_cast<uintptr_t>(value) & 15u) == 0 &&
                        (reinterpret_cast<uintptr_t>(codes) & 3u) == 0;
    if (vector)
        hipLaunchKernelGGL((encode_kernel<4>), row_grid(rows, width, 4), dim3(kThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((encode_kernel<1>), row_grid(rows, width, 1), dim3(kThreads), 0, stream, a);
    MK_LAUNCH_CHECK("mk_scalar_encode");
    return MK_OK;
}

extern "C" int mk_scalar_decode(const uint8_t *codes, const float *scales, const float *values, int n_values,
                                const float *zeros, float *out, int rows, int width, int group,
                                int groups_per_row, int refit, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(codes && scales && out, MK_ERR_INVALID, "mk_scalar_decode: null tensor pointer");
    MK_REQUIRE(rows >= 1 && width >= 1 && group >= 1 && refit >= 0, MK_ERR_INVALID,
               "mk_scalar_decode: sizes must be positive");
    if (int status = check_table("mk_scalar_decode", values, n_values)) return status;
    CodecArgs a{};
    a.codes_in = codes; a.scales = scales; a.zeros = zeros; a.values = values; a.out = out;
    a.rows = rows; a.width = width; a.group = group; a.groups_per_row = groups_per_row;
    a.refit = refit >= width ? 0 : refit;
    a.groups_per_region = refit ? mk_cdiv(refit, group) : 0;
    const int needed = a.refit ? mk_cdiv(width, a.refit) * a.groups_per_region : mk_cdiv(width, group);
    // The last refit region may be narrower than the others and hold fewer groups.
    const int needed_minimum = a.refit ? (mk_cdiv(width, a.refit) - 1) * a.groups_per_region + 1 : needed;
    MK_REQUIRE(groups_per_row >= needed_minimum, MK_ERR_INVALID,
               "mk_scalar_decode: %d scale groups per row cannot cover width %d (group %d, refit %d)",
               groups_per_row, width, group, refit);
    a.n_values = n_values;
    const bool vector = width % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0 &&
                        (reinterpret_cast<uintptr_t>(codes) & 3u) == 0;
    if (vector)
        hipLaunchKernelGGL((decode_kernel<4>), row_grid(rows, width, 4), dim3(kThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((decode_kernel<1>), row_grid(rows, width, 1), dim3(kThreads), 0, stream, a);
    MK_LAUNCH_CHECK("mk_scalar_decode");
    return MK_OK;
}

extern "C" int mk_search_scales(const float *value, const float *scales, const float *zeros,
                                const float *values, int n_values, const float *fractions, int n_fractions,
                                float *selected, int rows, int width, int group, int groups_per_row,
                                int scale_format, int integer, float minimum, float maximum, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(value && scales && selected && fractions, MK_ERR_INVALID, "mk_search_scales: null tensor pointer");
    MK_REQUIRE(rows >= 1 && width >= 1 && group >= 1, MK_ERR_INVALID, "mk_search_scales: sizes must be positive");
    MK_REQUIRE(groups_per_row == mk_cdiv(width, group), MK_ERR_INVALID,
               "mk_search_scales: expected %d scale groups per row, got %d", mk_cdiv(width, group), groups_per_row);
    MK_REQUIRE(n_fractions >= 0 && n_fractions <= 64, MK_ERR_INVALID, "mk_search_scales: at most 64 candidate fractions");
    MK_REQUIRE(scale_format >= 0 && scale_format <= 4, MK_ERR_INVALID, "mk_search_scales: unknown scale format code");
    MK_REQUIRE(static_cast<long long>(rows) * groups_per_row < (1ll << 31), MK_ERR_INVALID,
               "mk_search_scales: too many scale groups");
    if (!integer)
        if (int status = check_table("mk_search_scales", values, n_values)) return status;
    SearchArgs a{};
    a.value = value; a.scales = scales; a.zeros = zeros; a.values = values; a.fractions = fractions;
    a.selected = selected; a.rows = rows; a.width = width; a.group = group; a.groups_per_row = groups_per_row;
    a.n_values = integer ? 1 : n_values; a.n_fractions = n_fractions; a.format = scale_format; a.integer = integer;
    a.minimum = minimum; a.maximum = maximum; a.total_groups = rows * groups_per_row;
    int lanes = group & -group;
    if (lanes > 64) lanes = 64;
    switch (lanes) {
        case 64: launch_search<64>(a, stream); break;
        case 32: launch_search<32>(a, stream); break;
        case 16: launch_search<16>(a, stream); break;
        case 8: launch_search<8>(a, stream); break;
        case 4: launch_search<4>(a, stream); break;
        case 2: launch_search<2>(a, stream); break;
        default: launch_search<1>(a, stream); break;
    }
    MK_LAUNCH_CHECK("mk_search_scales");
    return MK_OK;
}

extern "C" int mk_snap(const float *value, const float *values, int n_values, float *out, long long count,
                       void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(count >= 0, MK_ERR_INVALID, "mk_snap: negative element count");
    if (count == 0) return MK_OK;
    MK_REQUIRE(value && out, MK_ERR_INVALID, "mk_snap: null tensor pointer");
    if (int status = check_table("mk_snap", values, n_values)) return status;
    long long blocks = (count + kThreads - 1) / kThreads;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(snap_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, stream, value, values,
                       n_values, out, static_cast<size_t>(count));
    MK_LAUNCH_CHECK("mk_snap");
    return MK_OK;
}

// Shared with the error-feedback sweep: scales of row r land at scales[r * out_row_stride + g].
int mk_fit_scales_strided(const float *value, long long row_stride, float *scales, float *zeros,
                          long long out_row_stride, int rows, int span, int group, int asym, float reciprocal,
                          float value_minimum, int scale_format, int store_zero, hipStream_t stream) {
    MK_REQUIRE(value && scales && (!asym || zeros), MK_ERR_INVALID, "mk_fit_scales: null tensor pointer");
    MK_REQUIRE(rows >= 1 && span >= 1 && group >= 1 && row_stride >= span, MK_ERR_INVALID,
               "mk_fit_scales: sizes must be positive and rows at least `span` apart");
    MK_REQUIRE(scale_format >= 0 && scale_format <= 4, MK_ERR_INVALID, "mk_fit_scales: unknown scale format code");
    const int groups_per_row = mk_cdiv(span, group);
    MK_REQUIRE(out_row_stride >= groups_per_row, MK_ERR_INVALID, "mk_fit_scales: output rows overlap");
    MK_REQUIRE(static_cast<long long>(rows) * groups_per_row < (1ll << 31), MK_ERR_INVALID,
               "mk_fit_scales: too many scale groups");
    FitArgs a{};
    a.value = value; a.scales = scales; a.zeros = asym ? zeros : nullptr; a.row_stride = row_stride;
    a.out_row_stride = out_row_stride;
    a.rows = rows; a.span = span; a.group = group; a.groups_per_row = groups_per_row;
    a.total_groups = rows * groups_per_row; a.asym = asym; a.format = scale_format; a.store_zero = store_zero;
    a.reciprocal = reciprocal; a.value_minimum = value_minimum;
    int reach = group < span ? group : span;
    const bool wide = row_stride % 4 == 0 && group % 4 == 0 && span % 4 == 0 && (reinterpret_cast<uintptr_t>(value) & 15u) == 0;
    if (wide) reach /= 4;  // lanes read four values at a time
    if (reach >= 64) launch_fit<64>(a, stream);
    else if (reach >= 32) launch_fit<32>(a, stream);
    else if (reach >= 16) launch_fit<16>(a, stream);
    else if (reach >= 8) launch_fit<8>(a, stream);
    else launch_fit<4>(a, stream);
    MK_LAUNCH_CHECK("mk_fit_scales");
    return MK_OK;
}

extern "C" int mk_fit_scales(const float *value, long long row_stride, float *scales, float *zeros, int rows,
                             int span, int group, int asym, float reciprocal, float value_minimum,
                             int scale_format, int store_zero, void *stream) {
    const int groups = group >= 1 ? mk_cdiv(span, group) : 0;
    return mk_fit_scales_strided(value, row_stride, scales, zeros, groups, rows, span, group, asym, reciprocal,
                                 value_minimum, scale_format, store_zero, static_cast<hipStream_t>(stream));
}

extern "C" int mk_reconstruct_activations(const void *inputs, int dtype, void *output, const float *values,
                                          int n_values, int rows, int width, int group, int scale_format,
                                          int asym, int integer, float minimum, float maximum, float reciprocal,
                                          void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(rows >= 0 && width >= 1 && group >= 1, MK_ERR_INVALID, "mk_reconstruct_activations: sizes must be positive");
    if (rows == 0) return MK_OK;
    MK_REQUIRE(inputs && output, MK_ERR_INVALID, "mk_reconstruct_activations: null tensor pointer");
    MK_REQUIRE(mk_dtype_valid(dtype), MK_ERR_INVALID, "mk_reconstruct_activations: unknown dtype code");
    MK_REQUIRE(scale_format >= 0 && scale_format <= 4, MK_ERR_INVALID, "mk_reconstruct_activations: unknown scale format code");
    if (!integer)
        if (int status = check_table("mk_reconstruct_activations", values, n_values)) return status;
    if (group > width) group = width;
    const int groups_per_row = mk_cdiv(width, group);
    MK_REQUIRE(static_cast<long long>(rows) * groups_per_row < (1ll << 31), MK_ERR_INVALID,
               "mk_reconstruct_activations: too many scale groups");
    ReconstructArgs a{};
    a.inputs = inputs; a.output = output; a.values = values; a.rows = rows; a.width = width; a.group = group;
    a.groups_per_row = groups_per_row; a.total_groups = rows * groups_per_row; a.dtype = dtype;
    a.n_values = integer ? 1 : n_values; a.format = scale_format; a.asym = asym; a.integer = integer;
    a.reciprocal = reciprocal; a.minimum = minimum; a.maximum = maximum;
    if (group >= 64) launch_reconstruct<64>(a, stream);
    else if (group >= 32) launch_reconstruct<32>(a, stream);
    else if (group >= 16) launch_reconstruct<16>(a, stream);
    else launch_reconstruct<8>(a, stream);
    MK_LAUNCH_CHECK("mk_reconstruct_activations");
    return MK_OK;
}
