/* Oracle (test infrastructure, never linked into the product): scalar C restatement of
 * the sequential pieces of the LDL error-feedback sweep.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp -shared -fPIC (see ../Makefile).
 * Every float operation below is a separate IEEE binary32 operation unless it is
 * spelled fmaf().
 *
 * Follows, in the reference (/root/reference/src/mlkit):
 *   kernels/error_feedback.py:22-96          round_feedback_tile  -> mk_ref_round_tile
 *   algorithms/error_feedback.py:366-370     trailing addmm_      -> mk_ref_block_update
 *   algorithms/error_feedback.py:373-393     _pending_continuation-> mk_ref_pending
 *   formats/grouped_scaling.py:274-289       absmax/minmax scales -> mk_ref_fit_scales
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>

static float half_round(float value) {
    /* fp32 -> fp16 -> fp32, round to nearest even, for values already clamped to
     * [2^-24, 65504] (formats/scale_storage.py:20-21): round to a multiple of the fp16
     * quantum 2^(e-10), e = max(floor(log2 value), -14). */
    int exponent;
    frexpf(value, &exponent);
    exponent -= 1;
    const int quantum = (exponent < -14 ? -14 : exponent) - 10;
    return ldexpf(nearbyintf(ldexpf(value, -quantum)), quantum);
}

/* Sequential rounding of one tile of columns for every row.
 * original, feedback, output: [rows, width] fp32; coeff: [width, width] fp32 unit upper;
 * scales/zeros: [rows, groups_per_row] of the current region; encoded: [rows, width] u8. */
void mk_ref_round_tile(const float *original, const float *feedback, const float *coeff,
                       const float *scales, const float *zeros, const float *values,
                       int n_values, float *output, uint8_t *encoded, int rows, int width,
                       int region_start, int tile_start, int tile_width, int group,
                       int groups_per_row, int integer, float code_min, float code_max) {
#pragma omp parallel for schedule(static)
    for (int row = 0; row < rows; ++row) {
        float corrections[1024];
        const size_t base = (size_t)row * (size_t)width;
        for (int c = 0; c < tile_width; ++c) corrections[c] = feedback[base + tile_start + c];
        for (int column = 0; column < tile_width; ++column) {
            const int position = tile_start + column;
            const float weight = original[base + position];
            const float target = weight + corrections[column];
            const int slot = row * groups_per_row + (position - region_start) / group;
            const float scale = scales[slot];
            const float zero = zeros ? zeros[slot] : 0.0f;
            const float normalized = (target - zero) / scale;
            float reconstruction;
            int index;
            if (integer) {
                float code = nearbyintf(normalized);
                code = fminf(fmaxf(code, code_min), code_max);
                index = (int)(code - code_min);
                reconstruction = code * scale;
                reconstruction = reconstruction + zero;
            } else {
                float best = INFINITY;
                index = 0;
                for (int e = 0; e < n_values; ++e) {
                    float distance = fabsf(normalized - values[e]);
                    if (distance < best) { best = distance; index = e; }
                }
                reconstruction = values[index] * scale;
                reconstruction = reconstruction + zero;
            }
            const float deviation = weight - reconstruction;
            const float *coefficient_row = coeff + (size_t)position * (size_t)width + tile_start;
            for (int c = column + 1; c < tile_width; ++c) {
                float product = deviation * coefficient_row[c];
                corrections[c] = corrections[c] + product;
            }
            output[base + position] = reconstruction;
            encoded[base + position] = (uint8_t)index;
        }
    }
}

/* feedback[:, stop:] += (original[:, tile] - output[:, tile]) @ coeff[tile, stop:]
 * mode 0: each product sum starts at zero and runs fmaf over ascending k, then one add;
 * mode 1: same with separate multiply and add. */
void mk_ref_block_update(float *feedback, const float *original, const float *output,
                         const float *coeff, int rows, int width, int tile_start,
                         int tile_stop, int mode) {
    const int depth = tile_stop - tile_start;
#pragma omp parallel for schedule(static)
    for (int row = 0; row < rows; ++row) {
        float deviation[1024];
        const size_t base = (size_t)row * (size_t)width;
        for (int k = 0; k < depth; ++k)
            deviation[k] = original[base + tile_start + k] - output[base + tile_start + k];
        for (int c = tile_stop; c < width; ++c) {
            float sum = 0.0f;
            if (mode == 0) {
                for (int k = 0; k < depth; ++k)
                    sum = fmaf(deviation[k], coeff[(size_t)(tile_start + k) * width + c], sum);
            } else {
                for (int k = 0; k < depth; ++k) {
                    float product = deviation[k] * coeff[(size_t)(tile_start + k) * width + c];
                    sum = sum + product;
                }
            }
            feedback[base + c] = feedback[base + c] + sum;
        }
    }
}

/* out[rows, region_width] = feedback[:, region] * U^-1, U = coeff[region, region] unit upper.
 * Right-looking forward substitution: once column j is final, every later column c
 * receives  x[c] = x[c] - x[j]*U[j,c]  (multiply, then subtract), j ascending. */
void mk_ref_pending(const float *feedback, const float *coeff, float *out, int rows, int width,
                    int region_start, int region_stop) {
    const int span = region_stop - region_start;
#pragma omp parallel for schedule(static)
    for (int row = 0; row < rows; ++row) {
        float *x = out + (size_t)row * span;
        for (int c = 0; c < span; ++c) x[c] = feedback[(size_t)row * width + region_start + c];
        for (int j = 0; j < span; ++j) {
            const float pivot = x[j];
            const float *u = coeff + (size_t)(region_start + j) * width + region_start;
            for (int c = j + 1; c < span; ++c) {
                float product = pivot * u[c];
                x[c] = x[c] - product;
            }
        }
    }
}

/* Per-group fp16-stored scales (and offsets) of targets[rows, span].
 * Symmetric: max(max, -min) clamped at 1e-12, times reciprocal; asymmetric:
 * (max-min) clamped, times reciprocal, zero = min - value_min*scale, zero stored as
 * fp16(|zero| clamped at 1e-12) with its sign.  fp16 storage clamps to [2^-24, 65504]. */
void mk_ref_fit_scales(const float *targets, float *scales, float *zeros, int rows, int span,
                       int group, int asym, float reciprocal, float value_min) {
    const int groups = (span + group - 1) / group;
    for (int row = 0; row < rows; ++row) {
        for (int g = 0; g < groups; ++g) {
            const int start = g * group;
            const int stop = start + group < span ? start + group : span;
            float low = INFINITY, high = -INFINITY;
            for (int c = start; c < stop; ++c) {
                float v = targets[(size_t)row * span + c];
                low = fminf(low, v);
                high = fmaxf(high, v);
            }
            float scale, zero = 0.0f;
            if (asym) {
                scale = fmaxf(high - low, 1e-12f) * reciprocal;
                float shift = value_min * scale;
                zero = low - shift;
            } else {
                scale = fmaxf(fmaxf(high, -low), 1e-12f) * reciprocal;
            }
            scale = half_round(fminf(fmaxf(scale, 0x1p-24f), 65504.0f));
            scales[row * groups + g] = scale;
            if (asym) {
                float magnitude = fmaxf(fabsf(zero), 1e-12f);
                magnitude = half_round(fminf(fmaxf(magnitude, 0x1p-24f), 65504.0f));
                zeros[row * groups + g] = zero > 0.0f ? magnitude : (zero < 0.0f ? -magnitude : 0.0f);
            }
        }
    }
}

/* Scalar dequantise + dot product, the CPU baseline of the packed matvec when numpy's
 * BLAS is not wanted: y[m, n] = sum_k (values[code]*scale + zero) * x[m, k]. */
void mk_ref_matvec(const uint8_t *codes, const float *scales, const float *zeros,
                   const float *values, const float *x, float *y, int samples, int rows,
                   int width, int group) {
    const int groups = (width + group - 1) / group;
#pragma omp parallel for schedule(static)
    for (int row = 0; row < rows; ++row) {
        for (int m = 0; m < samples; ++m) {
            float sum = 0.0f;
            for (int k = 0; k < width; ++k) {
                float w = values[codes[(size_t)row * width + k]] * scales[row * groups + k / group];
                if (zeros) w = w + zeros[row * groups + k / group];
                sum = fmaf(w, x[(size_t)m * width + k], sum);
            }
            y[(size_t)m * rows + row] = sum;
        }
    }
}
