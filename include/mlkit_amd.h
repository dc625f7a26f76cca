/* C ABI of libmlkit_amd.so: the gfx950 kernels behind mlkit's packed-inference and
 * fused-quantization path.
 *
 * Conventions
 *   - every pointer is a device pointer owned by the caller unless it says "host";
 *     the library allocates nothing and retains nothing;
 *   - `stream` is a hipStream_t (NULL = the default stream); every entry point only
 *     enqueues work on it and returns without synchronising;
 *   - return value 0 = enqueued; nonzero = nothing was launched (MK_ERR_*), and
 *     mk_last_error() describes why (per host thread);
 *   - dtype codes: MK_F32 = 0, MK_F16 = 1, MK_BF16 = 2.
 *
 * Each declaration names the reference interface (path under /root/reference/src/mlkit)
 * whose launch it replaces.
 */
#ifndef MLKIT_AMD_H
#define MLKIT_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MK_F32 0
#define MK_F16 1
#define MK_BF16 2

#define MK_OK 0
#define MK_ERR_INVALID 1     /* shape / dtype / alignment the entry point does not accept */
#define MK_ERR_UNSUPPORTED 2 /* valid request with no kernel (e.g. a layout that splits a word) */
#define MK_ERR_HIP 3         /* the HIP runtime reported an error at launch */

/* Library version, "major.minor.patch". */
const char *mk_version(void);

/* Message of the last nonzero status returned to this host thread ("" if none). */
const char *mk_last_error(void);

/* 1 when (bits, input_width, group) has a fused layout, i.e. rows and scale groups hold
 * whole packing words and a tile has at least 16 codes; 0 otherwise.
 * Replaces: kernels/packed_linear.py:63-79 (layout_for is None / not None). */
int mk_packed_layout_supported(int bits, int input_width, int group);

/* y[m, n] = sum_k dequant(code[n, k]) * x[m, k] (+ bias[n]), fp32 accumulate, y in x's dtype.
 * dequant(c) = (uniform ? grid_min + c*grid_step : values[c]) * scales[n, k/group] (+ zeros[n, k/group]).
 *   x       [samples, input_width]   x_dtype, contiguous
 *   packed  little-endian bit stream of [output_width, input_width] codes of `bits` bits
 *   scales  [output_width, groups] scale_dtype, groups = ceil(input_width / group)
 *   values  [n_values] fp32 (n_values <= 2^bits); read only when uniform == 0
 *   zeros   NULL or same shape/dtype as scales
 *   bias    NULL or [output_width] bias_dtype
 *   y       [samples, output_width] x_dtype
 * Any samples >= 1 is accepted (the caller applies its own fused-row limit).
 * Replaces: kernels/packed_linear.py:181-226 (matrix_vector) and the direct launch of
 * packed_matrix_vector in inference/packed_linear.py:181-245. */
int mk_packed_matvec(const void *x, int x_dtype, const uint8_t *packed, const void *scales,
                     int scale_dtype, const float *values, int n_values, const void *zeros,
                     const void *bias, int bias_dtype, void *y, int samples, int output_width,
                     int input_width, int group, int bits, int uniform, float grid_min,
                     float grid_step, void *stream);

/* mk_packed_matvec for `count` (1..8) weight matrices of one input width and one codec in a
 * single call: y[i] = x[i] @ dequant(packed[i])^T (+ bias[i]) for every i, each with
 * output_widths[i] rows.  The activation pointers may all be the same (sibling projections
 * fed by one tensor: attention q/k/v, MLP gate/up) or differ (the experts of a
 * mixture-of-experts layer, each with its own `samples` rows).  The matrices share samples,
 * input_width, group, bits, the grid (uniform, grid_min, grid_step, values) and the dtypes;
 * either every matrix has offsets or none has.  x, packed, scales, zeros (NULL = none), bias
 * (NULL = none; single entries may be NULL) and y are HOST arrays of `count` device pointers,
 * output_widths a host array of `count` ints; the arrays are read before the call returns.
 * Layouts the streaming and table kernels take (2- to 8-bit codes of any grid with 16-bit
 * activations and scales, or 4-bit codes of a uniform grid with fp32 activations and scales of
 * any type; input_width a multiple of 32 up to 16384, scale groups of whole multiples of 32
 * codes) run as ONE launch whose grid covers all the matrices; every other layout runs as
 * `count` launches of mk_packed_matvec.  With one and two samples the results equal those of
 * `count` separate calls bit for bit; from three samples on the kernels split a row's sum by
 * the size of the launch, and a few outputs in a thousand differ from the separate call's by
 * one rounding of the output type.
 * Replaces: the consecutive launches of kernels/packed_linear.py:181-226 that a model makes
 * for such layers (it calls PackedLinear.forward, inference/packed_linear.py:148-245, once
 * per layer). */
int mk_packed_matvec_group(const void *const *x, int x_dtype, int count, const uint8_t *const *packed,
                           const void *const *scales, int scale_dtype, const float *values, int n_values,
                           const void *const *zeros, const void *const *bias, int bias_dtype,
                           void *const *y, const int *output_widths, int samples, int input_width,
                           int group, int bits, int uniform, float grid_min, float grid_step, void *stream);

/* The online input rotation of a rotated layer and its packed matvec from one call:
 * rotated = T(x * signs), T = (basis (x) H_power) * scale along the input width
 * (input_width = order * power, power a power of two; order == 1: a plain Walsh-Hadamard
 * transform, basis unused; order > 1 with basis NULL: the `order` blocks of `power` values are
 * transformed one by one, T = (I (x) H_power) * scale, through mk_fwht), written to `rotated`
 * ([samples, input_width] of x_dtype, a
 * buffer of the caller's that must not alias x), then mk_packed_matvec on `rotated` with the
 * remaining arguments.  signs: NULL (or [input_width] fp32 of +-1, 16-byte aligned for the
 * one-launch form).  Results equal mk_rotate_rows followed by mk_packed_matvec bit for bit;
 * MK_ERR_UNSUPPORTED when mk_rotate_rows does not take (order, power).  One exception, taken
 * whenever it applies: one fp16 or bf16 sample, no basis (a plain transform of 2048 / 4096 / 8192 /
 * 16384 values, or separate blocks of 64 to 16384 values that tile a row of whole 2048-value
 * slices, 14336 = 7 x 2048 for one), INT4 codes with 16-bit scales and whole tiles of rows (16,
 * or 4 below 4096 rows) run as ONE launch in which every workgroup transforms the activations
 * in its registers; `rotated` is then left untouched, and the result equals mk_packed_matvec on
 * mk_fwht's (stagewise) output rounded to x_dtype bit for bit -- for a plain transform the same
 * linear map as mk_rotate_rows, summed in the order of the stages.
 * Replaces: the rotate_inputs forward pre-hook (conversion/model_transforms.py:116-128) in
 * front of PackedLinear.forward (inference/packed_linear.py:148-245). */
int mk_rotated_packed_matvec(const void *x, int x_dtype, void *rotated, int order, int power,
                             const float *basis, const float *signs, float scale, const uint8_t *packed,
                             const void *scales, int scale_dtype, const float *values, int n_values,
                             const void *zeros, const void *bias, int bias_dtype, void *y, int samples,
                             int output_width, int input_width, int group, int bits, int uniform,
                             float grid_min, float grid_step, void *stream);

/* mk_rotated_packed_matvec without the `rotated` argument: the rotated activations go to a
 * fixed 512 KiB array inside the library's own device memory (one per GPU, held until the
 * process ends), so the call allocates nothing and asks the caller for no workspace.
 * samples * input_width * (bytes of x_dtype) must not exceed 524288 (8 rows of 16384 fp32
 * values); larger requests return MK_ERR_INVALID and name mk_rotated_packed_matvec.  All
 * calls on one GPU share the array: calls that overlap on one GPU (different streams) race,
 * calls on one stream do not.  Results equal mk_rotated_packed_matvec bit for bit.
 * No counterpart in the reference: it exists for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). */
int mk_rotated_packed_matvec_static(const void *x, int x_dtype, int order, int power, const float *basis,
                                    const float *signs, float scale, const uint8_t *packed,
                                    const void *scales, int scale_dtype, const float *values, int n_values,
                                    const void *zeros, const void *bias, int bias_dtype, void *y, int samples,
                                    int output_width, int input_width, int group, int bits, int uniform,
                                    float grid_min, float grid_step, void *stream);

/* out[n, k] = dequant(code[n, k]) in out_dtype, same dequantisation as mk_packed_matvec
 * with multiply and add kept separate (no fused multiply-add).
 * Replaces: kernels/packed_linear.py:279-313 (decode / decode_rows). */
int mk_packed_decode(const uint8_t *packed, const void *scales, int scale_dtype,
                     const float *values, int n_values, const void *zeros, void *out,
                     int out_dtype, int output_width, int input_width, int group, int bits,
                     int uniform, float grid_min, float grid_step, void *stream);

/* Rows rows[0 .. n_rows) of the [output_width, input_width] packed matrix, decoded as by
 * mk_packed_decode into out [n_rows, input_width]: the embedding lookup of a tied output
 * projection.  rows: device int64; a negative index i means output_width + i, as in the
 * reference's tensor indexing; an index still outside [0, output_width) decodes row 0 (the
 * reference raises there; the kernel stays within the matrix and reports nothing).
 * Replaces: the gather + unpack + decode_scaled of PackedEmbedding.forward
 * (inference/packed_linear.py:273-287). */
int mk_packed_decode_rows(const uint8_t *packed, const void *scales, int scale_dtype, const float *values,
                          int n_values, const void *zeros, const long long *rows, int n_rows, void *out,
                          int out_dtype, int output_width, int input_width, int group, int bits, int uniform,
                          float grid_min, float grid_step, void *stream);

/* packed = the little-endian bit stream of `count` codes of `bits` (1..16) bits: code i
 * occupies stream bits [i * bits, (i + 1) * bits), byte j holds stream bits [8 j, 8 j + 8);
 * ceil(count * bits / 8) bytes are written, the last one zero padded.  codes: uint8
 * (code_bytes 1) or signed int16 / int32 / int64 (code_bytes 2 / 4 / 8).  *overflow (device
 * int, NULL to skip; the caller zeroes it) becomes 1 when a code lies outside [0, 2^bits).
 * Replaces: quantization/operations/bit_packing.py:13-77 (pack). */
int mk_pack(const void *codes, int code_bytes, long long count, int bits, uint8_t *packed, int *overflow,
            void *stream);

/* codes[i] = code i of the stream written by mk_pack: uint8 for bits <= 8, int32 above.
 * Replaces: quantization/operations/bit_packing.py:80-135 (unpack). */
int mk_unpack(const uint8_t *packed, long long count, int bits, void *codes, void *stream);

/* Scale storage formats of the scalar codec (formats/scale_storage.py:11-26). */
#define MK_SCALE_FP32 0
#define MK_SCALE_FP16 1
#define MK_SCALE_BF16 2
#define MK_SCALE_FP8 3  /* e4m3 */
#define MK_SCALE_E8M0 4 /* power of two */

/* codes[r, c] = code of the grid value nearest to (value[r, c] - zeros[r, c/group]) / scales[r, c/group]
 * (IEEE division).  integer != 0: round half to even, clamp to [minimum, maximum], subtract
 * minimum; otherwise the nearest entry of the ascending table `values`, ties to the lower
 * index.  value [rows, width] fp32; scales, zeros (NULL or) [rows, groups_per_row] fp32;
 * codes [rows, width] uint8.
 * Replaces: kernels/scalar_encode.py:110-146 (encode). */
int mk_scalar_encode(const float *value, const float *scales, const float *zeros, const float *values,
                     int n_values, uint8_t *codes, int rows, int width, int group, int groups_per_row,
                     int integer, float minimum, float maximum, void *stream);

/* out[r, c] = values[codes[r, c]] * scales[r, s(c)] (+ zeros[r, s(c)]), multiply and add
 * separately rounded.  refit == 0: s(c) = c / group; refit > 0 (error-feedback codec):
 * s(c) = (c / refit) * ceil(refit / group) + (c % refit) / group.
 * Replaces: kernels/scalar_decode.py:70-97 (decode) and the scale indexing of
 * quantization/codecs/scaled.py:67-101 (decode_feedback). */
int mk_scalar_decode(const uint8_t *codes, const float *scales, const float *values, int n_values,
                     const float *zeros, float *out, int rows, int width, int group, int groups_per_row,
                     int refit, void *stream);

/* selected[r, g] = the candidate among scales[r, g] and store(scales[r, g] * fractions[i]),
 * i ascending, with the least squared rounding error over the group; a later candidate
 * wins only if strictly better.  `scale_format` is one of MK_SCALE_*.  Per-group errors
 * are summed by P = min(64, largest power of two dividing group) strided partial sums
 * folded by halving.
 * Replaces: kernels/scalar_encode.py:261-304 (search_scales). */
int mk_search_scales(const float *value, const float *scales, const float *zeros, const float *values,
                     int n_values, const float *fractions, int n_fractions, float *selected, int rows,
                     int width, int group, int groups_per_row, int scale_format, int integer,
                     float minimum, float maximum, void *stream);

/* out[i] = nearest entry of the ascending table `values` to value[i] (ties to the lower entry).
 * Replaces: kernels/scalar_encode.py:327-345 (snap). */
int mk_snap(const float *value, const float *values, int n_values, float *out, long long count,
            void *stream);

/* Per-group scales (and offsets) from each group's range, over columns [0, span) of rows
 * that lie row_stride elements apart:
 *   symmetric:  scale = max(max, -min, 1e-12) * reciprocal
 *   asymmetric: scale = max(max - min, 1e-12) * reciprocal, zero = min - value_minimum * scale
 * scales are rounded to `scale_format`; zeros are stored raw, or with store_zero != 0 as the
 * rounded magnitude carrying the sign.  A group holding a non-finite value yields NaN.
 * scales, zeros: [rows, ceil(span / group)] fp32.
 * Replaces: the tensor reductions of formats/grouped_scaling.py:30-43,274-289
 * (group_extrema, Scaled._initial_scales) and the storage rounding of :160-175. */
int mk_fit_scales(const float *value, long long row_stride, float *scales, float *zeros, int rows,
                  int span, int group, int asym, float reciprocal, float value_minimum,
                  int scale_format, int store_zero, void *stream);

/* output = quantize-dequantize of `inputs` ([rows, width], fp32 / fp16 / bf16; output has the
 * same dtype and may alias) with per-group scales fitted on the fly: the result equals
 * mk_fit_scales (zeros stored rounded) + mk_scalar_encode + mk_scalar_decode on the fp32
 * values, rounded to the input dtype.  `group` is clipped to width.
 * Replaces: kernels/activation_reconstruction.py:76-103 (reconstruct). */
int mk_reconstruct_activations(const void *inputs, int dtype, void *output, const float *values,
                               int n_values, int rows, int width, int group, int scale_format,
                               int asym, int integer, float minimum, float maximum, float reciprocal,
                               void *stream);

/* Walsh-Hadamard transform of `rows` rows of `width` = 2^S values: radix-2 butterflies in
 * ascending stride in fp32, then one multiplication by `scale`.  Input and output may be
 * fp32, fp16 or bf16 and may alias.  signs_before / signs_after (NULL or fp32 vectors of
 * +-1 with `sign_period` entries, a multiple of width) multiply the input / the output;
 * element (r, i) uses sign (r * width + i) mod sign_period, which lets a tensor of wider
 * rows be transformed block by block.
 * Replaces: kernels/hadamard.py:108-136 (transform). */
int mk_fwht(const void *source, int source_dtype, void *target, int target_dtype, long long rows,
            int width, const float *signs_before, const float *signs_after, int sign_period,
            float scale, void *stream);

/* target[r, f', p] = sum_f mix[f', f] * source[r, f, p] for fp32 tensors [rows, order, power];
 * mix = basis (transpose == 0) or its transpose; signs_after (NULL or [order * power])
 * multiplies the result.  order <= 256.  source and target must not alias.
 * Replaces: the basis product of quantization/operations/orthogonal_transforms.py:101-109
 * (structured_transform). */
int mk_basis_mix(const float *source, float *target, const float *basis, long long rows, int order,
                 int power, int transpose, const float *signs_after, void *stream);

/* Diagonal-block step of a blocked Cholesky factorisation: the upper triangle of the
 * symmetric positive definite size x size block at `matrix` (row-major, `leading` floats per
 * row, size <= 128) yields U with block = U^T U.  With row_columns == 0 (one workgroup) U
 * replaces the block in place, zeros below the diagonal.  With row_columns > 0 the
 * row_columns columns to the right of the block, in the same rows, take the same elimination
 * and become U^-T times themselves (the block row of the factor), in place, one workgroup
 * per 128 of them; the block itself is then left untouched and U goes to `factor_out`
 * (size rows of 128 floats), because every workgroup reads the block.
 * *status (device memory, zero before the first block) receives 1 + first_column + j if
 * pivot j is not positive and finite, as torch.linalg.cholesky_ex reports it; a block
 * launched after a failure does nothing.  The host drives the blocked algorithm with
 * matrix products for the trailing updates.
 * Replaces: the factorisation inside feedback_coefficients,
 * quantization/algorithms/error_feedback.py:37-83 (torch.linalg.cholesky_ex). */
int mk_cholesky_block(float *matrix, long long leading, int size, int first_column, int row_columns,
                      float *factor_out, int *status, void *stream);

/* The blocked transform of a width order * power (power a power of two) in one launch:
 * every row [order, power] of `source` is multiplied by signs_before (NULL or
 * [order * power] floats), each block goes through the Walsh-Hadamard stages of mk_fwht
 * and is multiplied by `scale`, the blocks are mixed as in mk_basis_mix, and the result
 * times signs_after is written to `target` in target_dtype.  Results equal mk_fwht
 * followed by mk_basis_mix bit for bit.  Returns MK_ERR_UNSUPPORTED when order * power
 * values do not fit one workgroup (order > 96, power < 32, or more than 160 KB of LDS);
 * callers then use the two calls.
 * Replaces: quantization/operations/orthogonal_transforms.py:87-109 (structured_transform)
 * and the rotate_inputs hook of conversion/model_transforms.py:116-128 for blocked widths. */
int mk_rotate_blocks(const void *source, int source_dtype, void *target, int target_dtype, long long rows,
                     int order, int power, const float *basis, int transpose, const float *signs_before,
                     const float *signs_after, float scale, void *stream);

/* The rotation of mk_rotate_blocks for a few activation rows, on order * rows workgroups:
 * target[r, f', :] = scale * H_power( sum_f basis[f', f] * (source[r, f, :] * signs[f, :]) ),
 * the same transform with the mix applied before the Walsh-Hadamard stages (they commute),
 * so every output block is independent work.  basis == NULL: the +-1 Hadamard matrix of
 * size `order` (a power of two), which makes the whole a Walsh-Hadamard transform of
 * order * power points.  32 <= power <= 1024; rows, order <= 65535.  Results agree with
 * mk_rotate_blocks / mk_fwht to fp32 rounding (another summation order), not bit for bit.
 * Replaces: the rotate_inputs hook of conversion/model_transforms.py:116-128
 * (quantization/operations/orthogonal_transforms.py:101-122) for activations. */
int mk_rotate_rows(const void *source, int source_dtype, void *target, int target_dtype, int rows, int order,
                   int power, const float *basis, const float *signs, float scale, void *stream);

/* Error-feedback sweep over columns [tile_start, tile_start + tile_width) of every row:
 * target = original + correction; the nearest grid value (as in mk_scalar_encode, with the
 * table's nearest entry taken as the lowest index of the least distance) times scale plus
 * zero is written to output, its code to encoded, and (original - reconstruction) times
 * coeff[column, later columns of the tile] is added to the later corrections, which start
 * from feedback[:, tile].  scales / zeros: [rows, groups_per_row] of the region starting at
 * column region_start.  tile_width <= 1024.
 * Replaces: kernels/error_feedback.py:99-143 (round_tile). */
int mk_feedback_round_tile(const float *original, const float *feedback, const float *coeff,
                           const float *scales, const float *zeros, const float *values, int n_values,
                           float *output, uint8_t *encoded, int rows, int width, int region_start,
                           int tile_start, int tile_width, int group, int groups_per_row,
                           int integer_grid, float code_min, float code_max, void *stream);

/* out[rows, stop - start] = feedback[:, start:stop] * U^-1 (+ original[:, start:stop] when
 * original is not NULL), U = coeff[start:stop, start:stop] unit upper triangular, by
 * right-looking substitution (x[c] -= x[j] * U[j, c], j ascending).  stop - start <= 1024.
 * Replaces: quantization/algorithms/error_feedback.py:373-393 (_pending_continuation). */
int mk_feedback_pending(const float *feedback, const float *coeff, const float *original, float *out,
                        int rows, int width, int region_start, int region_stop, void *stream);

/* feedback[:, tile_stop:] += (original - output)[:, tile_start:tile_stop] @ coeff[tile_start:tile_stop, tile_stop:]
 * on the fp32 matrix cores; each product sum starts at zero, accumulates over ascending k
 * and is added to feedback once.
 * Replaces: the addmm_ of quantization/algorithms/error_feedback.py:366-370. */
int mk_feedback_block_update(float *feedback, const float *original, const float *output,
                             const float *coeff, int rows, int width, int tile_start, int tile_stop,
                             void *stream);

/* The same update for `chains` consecutive tiles of chain_width columns starting at
 * first_column, restricted to columns [column_begin, column_end) of feedback (which must
 * follow the last chain): f = (((f + S_0) + S_1) ...), every S_i a sum from zero over the k of
 * tile i.  The result equals applying mk_feedback_block_update tile after tile, which lets a
 * sweep defer the update of far columns and touch them once per several tiles.
 * Replaces: the same addmm_ (quantization/algorithms/error_feedback.py:366-370), batched. */
int mk_feedback_block_update_range(float *feedback, const float *original, const float *output,
                                   const float *coeff, int rows, int width, int first_column,
                                   int chain_width, int chains, int column_begin, int column_end,
                                   void *stream);

/* mk_feedback_block_update_range with the deviations handed over instead of recomputed:
 * deviations [width, rows] fp32 holds column c of (original - output) at deviations[c, :]
 * (what mk_feedback_sweep leaves in its `deviations` argument), so both operands of the
 * matrix-core product are read as row tiles.  Whole 128 x 128 tiles only: rows and
 * column_end - column_begin multiples of 128, chain_width a multiple of 32 and at least 128,
 * 16-byte aligned operands; MK_ERR_UNSUPPORTED otherwise.  Same sums, bit for bit.
 * Replaces: the addmm_ of quantization/algorithms/error_feedback.py:366-370, whose first
 * operand is this deviation matrix. */
int mk_feedback_block_update_staged(float *feedback, const float *deviations, const float *coeff, int rows,
                                    int width, int first_column, int chain_width, int chains, int column_begin,
                                    int column_end, void *stream);

/* The whole natural-order error-feedback sweep of a layer with per-region absmax / minmax
 * scale fits, enqueued in one call: for every region of `refit` columns the pending
 * continuation (into workspace, [rows, refit] fp32; may be NULL when refit >= width), the
 * scale fit on those targets (scales rounded to scale_format, zeros stored as rounded
 * magnitude with sign), then per tile of `block` columns mk_feedback_round_tile and the
 * trailing updates, far columns deferred by up to deferred_tiles tiles
 * (mk_feedback_block_update_range).  scales / zeros: [rows, G] fp32, G = sum over regions of
 * ceil(region width / min(group, region width)), region after region.  deviations: NULL, or
 * [width, rows] fp32 scratch in which the sweep leaves original - reconstruction column by
 * column for the trailing updates to read (faster; same results).  Results equal those of
 * issuing the separate entry points region by region.
 * Replaces: the host loop of quantization/algorithms/error_feedback.py:296-370. */
int mk_feedback_sweep(const float *original, float *feedback, float *output, uint8_t *encoded,
                      const float *coeff, float *scales, float *zeros, float *workspace,
                      float *deviations, const float *values, int n_values, int rows, int width,
                      int group, int refit,
                      int block, int integer_grid, float code_min, float code_max, int asym,
                      float reciprocal, float value_minimum, int scale_format, int deferred_tiles,
                      void *stream);

/* The matrix feedback_coefficients factors: target[a][b] = source[i(a)][i(b)] with
 * i(a) = order[a] (int64 indices) or, with order NULL, width - 1 - a; on the diagonal a zero
 * becomes one (a channel that was never activated) and *addend (one fp32 on the device: the
 * damping) is added.  source, target: [width, width] fp32, distinct.
 * Replaces: quantization/algorithms/error_feedback.py:55-66 (flip / index, masked_fill_, add_). */
int mk_hessian_reversed(const float *source, float *target, int width, const long long *order,
                        const float *addend, void *stream);

/* Unit upper-triangular coefficients from the upper Cholesky factor U of the reversed matrix:
 * out[a][b] = U[w-1-b][w-1-a] / U[w-1-b][w-1-b] (true division).  [width, width] fp32, distinct.
 * Replaces: quantization/algorithms/error_feedback.py:72-75 for step == 1 (division of the
 * lower factor's columns by its diagonal, flip back, contiguous copy). */
int mk_unit_upper_from_factor(const float *factor, float *out, int width, void *stream);

/* Index of the nearest codeword for `count` vectors of `dimension` (2, 4, 8 or 16) fp32
 * coordinates: the smallest sum over ascending coordinates of squared differences, the
 * lowest index on ties.  codebook: [codebook_size, dimension] fp32.  With lattice != 0 the
 * codebook is the E8P table (65,536 points of 8 coordinates followed by the 256 magnitude
 * patterns that generate them) and the search is the structured one: per coset, every
 * magnitude pattern scored against |v - shift|, a pattern whose sign parity disagrees with the
 * input's paying for the flip of its cheapest coordinate; code = pattern * 128 + sign bits
 * (+ 32768 for the -1/4 coset).  codes: [count] int32.
 * Replaces: kernels/lattice_search.py:10-70 (nearest_lattice_code, nearest_lattice, search)
 * and the device side of quantization/operations/search.py:34-79 (nearest). */
int mk_vector_nearest(const float *vectors, long long count, int dimension, const float *codebook,
                      int codebook_size, int lattice, int32_t *codes, void *stream);

/* Columns [tile_start, tile_start + tile_width) of every row, rounded in blocks of
 * `dimension` columns with LDL error feedback: target = weight + correction, code = the
 * codeword nearest to target / scale (search as in mk_vector_nearest), reconstruction =
 * codeword * scale, and the block's deviations times their coefficient rows (products
 * rounded one by one, summed over ascending coordinate) added to the corrections of the
 * tile's later columns.  original, feedback, output: [rows, width] fp32; coeff: [width,
 * width]; scales: [rows, groups_per_row] fp32, group `(column - region_start) / group`;
 * encoded: [rows, width / dimension] int32.  At most 256 columns per call; width, tile bounds
 * and group multiples of `dimension`.
 * Replaces: kernels/error_feedback.py:146-274 (round_vector_feedback_tile, round_vector_tile). */
int mk_feedback_round_vector_tile(const float *original, const float *feedback, const float *coeff,
                                  const float *scales, const float *codebook, float *output,
                                  int32_t *encoded, int rows, int width, int region_start,
                                  int tile_start, int tile_width, int group, int groups_per_row,
                                  int dimension, int codebook_size, int lattice, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MLKIT_AMD_H */
