// Diagonal-block step of a blocked Cholesky factorisation on gfx950.
//
// The error-feedback coefficients are U blockdiag(U)^-1 for the damped Hessian H = U^T U
// (K up to 16384).  The library factorisation spends most of its time in its small
// unblocked panel kernel, so the blocked algorithm is driven from the host with library
// matrix products for the trailing updates, and this file supplies the rest: a workgroup
// factors a diagonal block of at most 128 x 128 in registers and, on request, carries 128
// columns of the block's rows through the same elimination, which makes them the factor's
// block row (one workgroup per 128 columns; no triangular solve is needed).
//
// Replaces the `torch.linalg.cholesky_ex` call of `feedback_coefficients`
// (quantization/algorithms/error_feedback.py:37-83 in /root/reference/src/mlkit) for large
// matrices on the device; mk_hessian_reversed and mk_unit_upper_from_factor are the tensor
// operations in front of it and behind it (:55-66 index reversal and damping, :72-75 division
// by the diagonal and reversal back), one pass over the matrix each.

#include "mk_common.h"

#include <type_traits>

namespace {

constexpr int kBlock = 128;
constexpr int kThreads = 256;

struct BlockArgs {
    float *matrix;       // the block's top-left element; row-major with `leading` floats per row
    long long leading;
    int size;            // rows = columns of the block, 1 ... 128
    int first_column;    // index of the block's first column in the whole matrix (for status)
    int *status;         // stays 0, or becomes 1 + the column whose pivot is not positive
    int row_columns;     // columns to the right of the block, in the same rows, that take the same elimination
    float *factor_out;   // where the factor goes when row_columns > 0 (128 floats per row); else in place
};

constexpr int kTile = kBlock / 16;
constexpr int kRowFloats = 2 * kBlock;   // a published row: the block's columns, then the columns carried beside it

// Columns 16 SIXTEEN ... 16 SIXTEEN + 15 of the factorisation below, two per step (their rows
// sit in register row SIXTEEN of their owners).  False after a pivot that is not positive and
// finite, which every thread sees in the same step.
//
// A step takes rows j and j + 1 as the updates of columns < j left them (`pivot_rows`), and
// every thread derives what it needs of the two finished rows itself:
//   U[j][k]     = A[j][k] / sqrt(A[j][j])
//   U[j+1][k]   = (A[j+1][k] - U[j][j+1] U[j][k]) / sqrt(A[j+1][j+1] - U[j][j+1]^2)
// and subtracts both outer products from its sub-block: one LDS round trip and one barrier
// per two columns.
//
// ROW: the workgroup also carries 128 columns to the right of the block (`beside`), which take
// the same row operations and so become U_jj^-T A_jr, the block row of the factor.
template <int SIXTEEN, bool ROW, int BT>
__device__ __forceinline__ bool sixteen_steps(const BlockArgs &a, float (&mine)[kTile][kTile], float (&beside)[kTile][BT],
                                              float (&pivot_rows)[2][2][kRowFloats], int tx, int ty) {
#pragma unroll 1
    for (int lane = 0; lane < 16; lane += 2) {
        const int j = 16 * SIXTEEN + lane;
        const float *first = pivot_rows[(j >> 1) & 1][0], *second = pivot_rows[(j >> 1) & 1][1];
        const float pivot = first[j];
        if (!(pivot > 0.0f) || !(pivot - pivot == 0.0f)) {
            if (threadIdx.x == 0) *a.status = a.first_column + j + 1;
            return false;
        }
        // (one v_rsq_f32, accurate to an ulp; the IEEE square root and division were a fifth of a step's chain)
        const float reciprocal = __builtin_amdgcn_rsqf(pivot);
        const float link = first[j + 1] * reciprocal;                 // U[j][j+1]
        const float next_pivot = second[j + 1] - link * link;
        if (!(next_pivot > 0.0f) || !(next_pivot - next_pivot == 0.0f)) {
            if (threadIdx.x == 0) *a.status = a.first_column + j + 2;
            return false;
        }
        const float next_reciprocal = __builtin_amdgcn_rsqf(next_pivot);
        // Register rows below SIXTEEN hold only rows <= j (finished); register columns below
        // SIXTEEN only columns < j, which for the rows still changing lie below the diagonal
        // (never read): neither takes part, so a step costs 2 (8 - SIXTEEN)^2 multiply-adds.
        float rows_first[kTile], rows_second[kTile], columns_first[kTile], columns_second[kTile];
#pragma unroll
        for (int u = SIXTEEN; u < kTile; ++u) {
            const int i = ty + 16 * u, k = tx + 16 * u;
            const float upper = first[i] * reciprocal;                                   // U[j][i]
            const float lower = (second[i] - link * upper) * next_reciprocal;            // U[j+1][i]
            rows_first[u] = i > j + 1 ? upper : 0.0f;   // zero keeps rows <= j + 1 as they are
            rows_second[u] = i > j + 1 ? lower : 0.0f;
            columns_first[u] = first[k] * reciprocal;                                    // U[j][k]
            columns_second[u] = (second[k] - link * columns_first[u]) * next_reciprocal; // U[j+1][k]
        }
        float beside_first[BT], beside_second[BT];
        if constexpr (ROW) {
#pragma unroll
            for (int v = 0; v < BT; ++v) {
                const int c = kBlock + tx + 16 * v;
                beside_first[v] = first[c] * reciprocal;
                beside_second[v] = (second[c] - link * beside_first[v]) * next_reciprocal;
            }
        }
        // The two rows' owners keep the finished rows.
        if (ty == lane) {
#pragma unroll
            for (int v = SIXTEEN; v < kTile; ++v) mine[SIXTEEN][v] = columns_first[v];
            if constexpr (ROW) {
#pragma unroll
                for (int v = 0; v < BT; ++v) beside[SIXTEEN][v] = beside_first[v];
            }
        }
        if (ty == lane + 1) {
#pragma unroll
            for (int v = SIXTEEN; v < kTile; ++v) mine[SIXTEEN][v] = columns_second[v];
            if constexpr (ROW) {
#pragma unroll
                for (int v = 0; v < BT; ++v) beside[SIXTEEN][v] = beside_second[v];
            }
        }
#pragma unroll
        for (int u = SIXTEEN; u < kTile; ++u) {
#pragma unroll
            for (int v = SIXTEEN; v < kTile; ++v)
                mine[u][v] -= rows_first[u] * columns_first[v] + rows_second[u] * columns_second[v];
            if constexpr (ROW) {
#pragma unroll
                for (int v = 0; v < BT; ++v)
                    beside[u][v] -= rows_first[u] * beside_first[v] + rows_second[u] * beside_second[v];
            }
        }
        // Rows j + 2 and j + 3 have all their updates now: their owners publish them.
        float (*next)[kRowFloats] = pivot_rows[((j >> 1) + 1) & 1];
        if (lane < 14) {
            if (ty == lane + 2 || ty == lane + 3) {
#pragma unroll
                for (int v = SIXTEEN; v < kTile; ++v) next[ty - lane - 2][tx + 16 * v] = mine[SIXTEEN][v];   // columns < j are not read
                if constexpr (ROW) {
#pragma unroll
                    for (int v = 0; v < BT; ++v) next[ty - lane - 2][kBlock + tx + 16 * v] = beside[SIXTEEN][v];
                }
            }
        } else if constexpr (SIXTEEN + 1 < kTile) {
            if (ty < 2) {
#pragma unroll
                for (int v = SIXTEEN + 1; v < kTile; ++v) next[ty][tx + 16 * v] = mine[SIXTEEN + 1][v];
                if constexpr (ROW) {
#pragma unroll
                    for (int v = 0; v < BT; ++v) next[ty][kBlock + tx + 16 * v] = beside[SIXTEEN + 1][v];
                }
            }
        }
        __syncthreads();
    }
    return true;
}

// In: the upper triangle of a symmetric positive definite block.  Out: U with block = U^T U
// in the upper triangle, zeros below it.  A pivot that is not positive (or not finite)
// records its column and leaves the block unspecified.
//
// Right-looking, two columns per step.  The block lives in registers for the whole
// factorisation: thread (ty, tx) of a 16 x 16 grid owns entries (ty + 16 u, tx + 16 v),
// an 8 x 8 sub-block.  Per step only the two pivot rows travel: the threads that own them
// put them (as updated so far) into one of two LDS buffers, one barrier later every thread
// reads the entries it needs, finishes the two rows for itself and subtracts their outer
// products from its sub-block.  Rows up to the pivot rows are masked out of the update by
// zero factors, so finished rows keep their values.
// BT: sixteenths of 128 columns a workgroup carries beside the block (8: 128 columns, 4: 64).
template <bool ROW, int BT>
__global__ void __launch_bounds__(kThreads) cholesky_block_kernel(const BlockArgs a) {
    __shared__ float pivot_rows[2][2][kRowFloats];   // [buffer][row j, row j + 1][column]
    __shared__ int failed;
    const int n = a.size;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    if (threadIdx.x == 0) failed = *a.status != 0;   // an earlier block already failed: do nothing
    float mine[kTile][kTile], beside[kTile][BT];
    constexpr int kCarried = 16 * BT;
    // ROW: workgroup b carries columns kCarried b ... kCarried (b + 1) - 1 of the block row; every workgroup
    // factors the block itself (from the matrix, which nobody overwrites: the factor goes to
    // `factor_out`), and the first one stores it.
    const int beside_first_column = n + kCarried * blockIdx.x;
#pragma unroll
    for (int u = 0; u < kTile; ++u)
#pragma unroll
        for (int v = 0; v < kTile; ++v) {
            const int row = ty + 16 * u, column = tx + 16 * v;
            const bool inside = row < n && column < n && column >= row;
            const float loaded = a.matrix[(inside ? row : 0) * a.leading + (inside ? column : 0)];
            // Outside the block: an identity diagonal keeps every pivot of the padding at one.
            mine[u][v] = inside ? loaded : (row == column ? 1.0f : 0.0f);
            if (v < BT) {
                beside[u][v] = 0.0f;
                if constexpr (ROW) {
                    const bool present = row < n && kCarried * static_cast<int>(blockIdx.x) + column < a.row_columns;
                    const float carried = a.matrix[(present ? row : 0) * a.leading + (present ? beside_first_column + column : 0)];
                    beside[u][v] = present ? carried : 0.0f;
                }
            }
        }
    if (ty < 2) {
#pragma unroll
        for (int v = 0; v < kTile; ++v) {
            pivot_rows[0][ty][tx + 16 * v] = mine[0][v];
            if constexpr (ROW) {
                if (v < BT) pivot_rows[0][ty][kBlock + tx + 16 * v] = beside[0][v];
            }
        }
    }
    __syncthreads();
    if (failed) return;

    // All 128 columns run (the padding is an identity): no data-dependent exit other than a bad pivot.
    bool good = sixteen_steps<0, ROW, BT>(a, mine, beside, pivot_rows, tx, ty);
    good = good && sixteen_steps<1, ROW, BT>(a, mine, beside, pivot_rows, tx, ty);
    good = good && sixteen_steps<2, ROW, BT>(a, mine, beside, pivot_rows, tx, ty);
    good = good && sixteen_steps<3, ROW, BT>(a, mine, beside, pivot_rows, tx, ty);
    good = good && sixteen_steps<4, ROW, BT>(a, mine, beside, pivot_rows, tx, ty);
    good = good && sixteen_steps<5, ROW, BT>(a, mine, beside, pivot_rows, tx, ty);
    good = good && sixteen_steps<6, ROW, BT>(a, mine, beside, pivot_rows, tx, ty);
    good = good && sixteen_steps<7, ROW, BT>(a, mine, beside, pivot_rows, tx, ty);
    if (!good) return;
    float *factor = ROW ? a.factor_out : a.matrix;
    const long long factor_leading = ROW ? kBlock : a.leading;
#pragma unroll
    for (int u = 0; u < kTile; ++u)
#pragma unroll
        for (int v = 0; v < kTile; ++v) {
            const int row = ty + 16 * u, column = tx + 16 * v;
            if (blockIdx.x == 0 && row < n && column < n) factor[row * factor_leading + column] = column >= row ? mine[u][v] : 0.0f;
            if constexpr (ROW) {
                if (v < BT && row < n && kCarried * static_cast<int>(blockIdx.x) + column < a.row_columns)
                    a.matrix[row * a.leading + beside_first_column + column] = beside[u][v];
            }
        }
}

}  // namespace

// ---- the matrix that goes into the factorisation, and the coefficients that come out ---------

struct ReverseArgs {
    const float *source;
    float *target;
    const long long *order;  // null: index a reads row / column width - 1 - a
    const float *addend;     // one float: added to every diagonal entry (after zeros became ones)
    int width;
};

// target[a][b] = source[i(a)][i(b)]; on the diagonal a zero becomes one and *addend is added.
__global__ void __launch_bounds__(256) reversed_matrix_kernel(const ReverseArgs a) {
    const int row = blockIdx.y;
    const int column = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (column >= a.width) return;
    const long long source_row = a.order ? a.order[row] : a.width - 1 - row;
    const float *from = a.source + static_cast<size_t>(source_row) * a.width;
    float values[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int b = column + i;
        const bool inside = b < a.width;
        const long long source_column = a.order ? a.order[inside ? b : 0] : a.width - 1 - (inside ? b : 0);
        float value = from[source_column];
        if (b == row) value = __fadd_rn(value == 0.0f ? 1.0f : value, *a.addend);
        values[i] = value;
    }
    float *to = a.target + static_cast<size_t>(row) * a.width + column;
    if (column + 3 < a.width && (a.width & 3) == 0) {
        *reinterpret_cast<float4 *>(to) = make_float4(values[0], values[1], values[2], values[3]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (column + i < a.width) to[i] = values[i];
    }
}

// out[a][b] = U[w-1-b][w-1-a] / U[w-1-b][w-1-b]: the factor transposed, every column divided by
// its diagonal entry, both index orders reversed; 32 x 32 tiles turned in LDS so that reads and
// writes both run along rows.
__global__ void __launch_bounds__(256) unit_upper_kernel(const float *factor, float *out, int width) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 8 rows of 32 threads
    const int r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = r0 + ty + 8 * j, c = c0 + tx;
        const bool inside = r < width && c < width;
        const float value = factor[static_cast<size_t>(inside ? r : 0) * width + (inside ? c : 0)];
        const float pivot = factor[static_cast<size_t>(inside ? r : 0) * (width + 1)];
        tile[ty + 8 * j][tx] = inside ? __fdiv_rn(value, pivot) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int c = c0 + ty + 8 * j, r = r0 + tx;   // tile[r - r0][c - c0] goes to out[w-1-c][w-1-r]
        if (r < width && c < width)
            out[static_cast<size_t>(width - 1 - c) * width + (width - 1 - r)] = tile[tx][ty + 8 * j];
    }
}

extern "C" int mk_hessian_reversed(const float *source, float *target, int width, const long long *order,
                                   const float *addend, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(source && target && addend, MK_ERR_INVALID, "mk_hessian_reversed: null pointer");
    MK_REQUIRE(width >= 1 && width <= 65535, MK_ERR_INVALID, "mk_hessian_reversed: width out of range");
    MK_REQUIRE(source != target, MK_ERR_INVALID, "mk_hessian_reversed: source and target must not alias");
    ReverseArgs a{source, target, order, addend, width};
    hipLaunchKernelGGL(reversed_matrix_kernel, dim3(mk_cdiv(width, 1024), width), dim3(256), 0, stream, a);
    MK_LAUNCH_CHECK("mk_hessian_reversed");
    return MK_OK;
}

extern "C" int mk_unit_upper_from_factor(const float *factor, float *out, int width, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(factor && out, MK_ERR_INVALID, "mk_unit_upper_from_factor: null pointer");
    MK_REQUIRE(width >= 1 && width <= 65535 * 32, MK_ERR_INVALID, "mk_unit_upper_from_factor: width out of range");
    MK_REQUIRE(factor != out, MK_ERR_INVALID, "mk_unit_upper_from_factor: factor and out must not alias");
    hipLaunchKernelGGL(unit_upper_kernel, dim3(mk_cdiv(width, 32), mk_cdiv(width, 32)), dim3(256), 0, stream, factor, out, width);
    MK_LAUNCH_CHECK("mk_unit_upper_from_factor");
    return MK_OK;
}

extern "C" int mk_cholesky_block(float *matrix, long long leading, int size, int first_column, int row_columns,
                                 float *factor_out, int *status, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MK_REQUIRE(matrix && status, MK_ERR_INVALID, "mk_cholesky_block: null pointer");
    MK_REQUIRE(size >= 1 && size <= kBlock, MK_ERR_UNSUPPORTED, "mk_cholesky_block: blocks of 1 to %d rows (got %d)", kBlock, size);
    MK_REQUIRE(row_columns >= 0 && leading >= static_cast<long long>(size) + row_columns && first_column >= 0, MK_ERR_INVALID,
               "mk_cholesky_block: rows overlap");
    MK_REQUIRE(row_columns == 0 || factor_out, MK_ERR_INVALID,
               "mk_cholesky_block: a block row needs a separate place for the factor");
    BlockArgs a{matrix, leading, size, first_column, status, row_columns, factor_out};
    // 64 columns per workgroup while that still fits one workgroup per CU (a step then costs a
    // third less arithmetic); 128 beyond.
    if (row_columns > 256 * 64)
        hipLaunchKernelGGL((cholesky_block_kernel<true, 8>), dim3(mk_cdiv(row_columns, 128)), dim3(kThreads), 0, stream, a);
    else if (row_columns > 0)
        hipLaunchKernelGGL((cholesky_block_kernel<true, 4>), dim3(mk_cdiv(row_columns, 64)), dim3(kThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((cholesky_block_kernel<false, 4>), dim3(1), dim3(kThreads), 0, stream, a);
    MK_LAUNCH_CHECK("mk_cholesky_block");
    return MK_OK;
}
