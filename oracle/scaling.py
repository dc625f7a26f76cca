"""Oracle (test infrastructure): grouped scaling, nearest-code encoding and decoding.

All arithmetic is IEEE binary32 through numpy (no fused multiply-add, round to nearest
even, true division), which is what the reference's tensor path computes and what its
fused kernels are written to reproduce (``enable_fp_fusion=False``, ``div_rn``,
``nearbyint``).

Follows, in the reference:
  formats/scale_storage.py:11-26            store_scale
  formats/grouped_scaling.py:24-43          single_precision_reciprocal, group_extrema
  formats/grouped_scaling.py:147-175        Scaled.fit (scale/offset storage)
  formats/grouped_scaling.py:274-289        Scaled._initial_scales
  formats/grouped_scaling.py:291-351        Scaled._search_scales
  formats/grouped_scaling.py:46-51,353-392  nearest_codes, Scaled._scalar_codes
  kernels/scalar_rounding.py:15-73          kernel twins of the rounding helpers
  codecs/scaled.py:19-101                   decode_grouped / decode_scaled / decode_feedback

``search_scales`` fixes one summation order for the per-group squared error (stated in
its docstring); the reference leaves that order to ``Tensor.sum`` / ``tl.sum``.  The tests
pin the candidate order, the storage rounding of candidates, the strict comparison and the
"base scale wins ties" rule against a float64 brute force wherever the winner is clear (a
gap above 1e-4 relative) and on an exact tie; only the candidate chosen when the two best
errors lie within 1e-4 relative of each other is *parity unpinned* against the reference
(its own two code paths may disagree there too).
"""

import numpy as np

F32 = np.float32
SCALE_FORMAT_BITS = {"fp32": 32, "fp16": 16, "bf16": 16, "fp8": 8, "e8m0": 8}


def f32_reciprocal(value: float) -> np.float32:
    """fp32(1) / fp32(value) (grouped_scaling.py:24-27)."""
    return F32(1.0) / F32(value)


def round_bf16(value: np.ndarray) -> np.ndarray:
    words = np.ascontiguousarray(value, dtype=F32).view(np.uint32).astype(np.uint64)
    rounded = (words + 0x7FFF + ((words >> 16) & 1)) & 0xFFFF0000
    return rounded.astype(np.uint32).view(F32)


def round_e4m3(value: np.ndarray) -> np.ndarray:
    """Positive fp32 -> nearest FP8 E4M3 (ties to even), kernels/scalar_rounding.py:15-28."""
    clamped = np.clip(np.asarray(value, dtype=F32), F32(2.0**-9), F32(448.0))
    exponent = ((clamped.view(np.uint32) >> 23) & 255).astype(np.int32) - 127
    quantum_exponent = np.maximum(exponent, -6) - 3
    quantum = np.ldexp(F32(1.0), quantum_exponent).astype(F32)
    reciprocal = np.ldexp(F32(1.0), -quantum_exponent).astype(F32)
    return (np.rint(clamped * reciprocal) * quantum).astype(F32)


def store_scale(value: np.ndarray, fmt: str) -> tuple[np.ndarray, int]:
    value = np.asarray(value, dtype=F32)
    if fmt == "fp32":
        return value.copy(), 32
    if fmt == "fp16":
        return np.clip(value, F32(2.0**-24), F32(65504.0)).astype(np.float16).astype(F32), 16
    if fmt == "bf16":
        return round_bf16(value), 16
    if fmt == "fp8":
        return round_e4m3(value), 8
    if fmt == "e8m0":
        # log2 in float64: the rounding thresholds 2^(k+1/2) are irrational, so no fp32
        # value sits close enough to one for the float64 error to matter.
        clamped = np.maximum(value, F32(2.0**-127)).astype(np.float64)
        exponent = np.clip(np.rint(np.log2(clamped)), -127, 127)
        return np.ldexp(np.float64(1.0), exponent.astype(np.int32)).astype(F32), 8
    raise ValueError(f"unsupported scale storage format {fmt!r}")


def group_extrema(weight: np.ndarray, group: int) -> tuple[np.ndarray, np.ndarray]:
    rows, width = weight.shape
    whole = width - width % group
    minima, maxima = [], []
    if whole:
        blocks = weight[:, :whole].reshape(rows, -1, group)
        minima.append(blocks.min(-1))
        maxima.append(blocks.max(-1))
    if whole < width:
        minima.append(weight[:, whole:].min(-1, keepdims=True))
        maxima.append(weight[:, whole:].max(-1, keepdims=True))
    return np.concatenate(minima, 1), np.concatenate(maxima, 1)


def initial_scales(weight: np.ndarray, values: np.ndarray, group: int, asym: bool):
    """Unrounded scales and offsets from each group's range (grouped_scaling.py:274-289)."""
    weight = np.asarray(weight, dtype=F32)
    minimum, maximum = group_extrema(weight, group)
    if not (np.isfinite(minimum).all() and np.isfinite(maximum).all()):
        raise ValueError("scaled requires a finite floating-point weight matrix")
    value_minimum, value_maximum = float(values.min()), float(values.max())
    tiny = F32(1e-12)
    if asym:
        reciprocal = f32_reciprocal(value_maximum - value_minimum)
        scales = np.maximum(maximum - minimum, tiny) * reciprocal
        return scales.astype(F32), (minimum - F32(value_minimum) * scales).astype(F32)
    reciprocal = f32_reciprocal(float(np.abs(values).max()))
    magnitude = np.maximum(maximum, -minimum)
    return (np.maximum(magnitude, tiny) * reciprocal).astype(F32), None


def stored_offset(zero: np.ndarray, fmt: str) -> np.ndarray:
    """Offsets keep their sign and store their magnitude (grouped_scaling.py:172-174)."""
    magnitude, _ = store_scale(np.maximum(np.abs(zero), F32(1e-12)), fmt)
    return (magnitude * np.sign(zero)).astype(F32)


def nearest_codes(normalized: np.ndarray, values: np.ndarray) -> np.ndarray:
    """Nearest entry of an ascending table, ties to the lower index (grouped_scaling.py:46-51)."""
    upper = np.minimum(np.searchsorted(values, normalized, side="left"), values.size - 1)
    lower = np.maximum(upper - 1, 0)
    pick_lower = np.abs(normalized - values[lower]) <= np.abs(normalized - values[upper])
    return np.where(pick_lower, lower, upper)


def normalize(value, scales, zero, group, start=0):
    columns = (np.arange(start, start + value.shape[1]) // group)
    centered = np.asarray(value, dtype=F32)
    if zero is not None:
        centered = centered - zero[:, columns]
    return (centered / scales[:, columns]).astype(F32)


def encode(value, scales, zero, values, group, integer: bool, start: int = 0) -> np.ndarray:
    """Codes of the nearest grid values (grouped_scaling.py:353-392)."""
    values = np.asarray(values, dtype=F32)
    normalized = normalize(value, scales, zero, group, start)
    if integer:
        low, high = F32(values.min()), F32(values.max())
        codes = np.clip(np.rint(normalized), low, high) - low
    else:
        codes = nearest_codes(normalized, values)
    return codes.astype(np.uint8 if values.size <= 256 else np.int32)


def group_error_ordered(value, candidate, zero, values, group, integer) -> np.ndarray:
    """Per-group squared rounding error in the order the HIP search kernel uses.

    Lane ``p`` of ``P = min(64, largest power of two dividing group, at most 128)`` adds
    the squared errors of elements ``p, p+P, p+2P, ...`` of the group in ascending order
    (multiply, then add), then the ``P`` partial sums are folded by halving:
    ``s[0:h] += s[h:2h]`` for ``h = P/2 ... 1``.
    """
    rows, width = value.shape
    groups = candidate.shape[1]
    padded = np.zeros((rows, groups * group), dtype=F32)
    padded[:, :width] = value
    occupied = (np.arange(groups * group) < width).reshape(1, groups, group)
    blocks = padded.reshape(rows, groups, group)
    centered = blocks if zero is None else (blocks - zero[..., None]).astype(F32)
    normalized = (centered / candidate[..., None]).astype(F32)
    if integer:
        rounded = np.clip(np.rint(normalized), F32(values.min()), F32(values.max()))
    else:
        rounded = values[nearest_codes(normalized, values)]
    difference = np.where(occupied, (rounded * candidate[..., None]).astype(F32) - centered, F32(0))
    squares = (difference * difference).astype(F32)
    lanes = min(64, group & -group, 128)
    partial = np.zeros((rows, groups, lanes), dtype=F32)
    for step in range(group // lanes):
        partial = (partial + squares[..., step * lanes:(step + 1) * lanes]).astype(F32)
    half = lanes // 2
    while half:
        partial = (partial[..., :half] + partial[..., half:2 * half]).astype(F32)
        half //= 2
    return partial[..., 0]


def search_scales(value, scales, zero, values, fractions, group, fmt, integer) -> np.ndarray:
    """Best shrunken stored scale per group; the base scale wins ties (grouped_scaling.py:291-351)."""
    value = np.asarray(value, dtype=F32)
    values = np.asarray(values, dtype=F32)
    selected = scales.copy()
    best = group_error_ordered(value, scales, zero, values, group, integer)
    for fraction in np.asarray(fractions, dtype=F32):
        candidate, _ = store_scale((scales * fraction).astype(F32), fmt)
        error = group_error_ordered(value, candidate, zero, values, group, integer)
        improved = error < best
        selected = np.where(improved, candidate, selected)
        best = np.minimum(best, error)
    return selected.astype(F32)


def decode_grouped(codes, scales, values, group, zero=None) -> np.ndarray:
    """``values[codes] * scale (+ zero)``, multiply then add (codecs/scaled.py:19-64)."""
    columns = np.arange(codes.shape[1]) // group
    out = (np.asarray(values, dtype=F32)[codes.astype(np.int64)] * scales[:, columns]).astype(F32)
    return out if zero is None else (out + zero[:, columns]).astype(F32)


def feedback_scale_index(width: int, group: int, refit: int) -> np.ndarray:
    """Column -> scale index of the feedback codec (codecs/scaled.py:91-95)."""
    columns = np.arange(width)
    per_region = (refit + group - 1) // group
    return (columns // refit) * per_region + (columns % refit) // group


def decode_feedback(codes, scales, values, group, refit, zero=None) -> np.ndarray:
    index = feedback_scale_index(codes.shape[1], group, refit)
    out = (np.asarray(values, dtype=F32)[codes.astype(np.int64)] * scales[:, index]).astype(F32)
    return out if zero is None else (out + zero[:, index]).astype(F32)


def int_values(bits: int) -> np.ndarray:
    """The signed integer grid (grids/factory.py:61-72)."""
    return np.arange(-(2 ** (bits - 1)), 2 ** (bits - 1), dtype=F32)


NF4_VALUES = np.array([
    -1.0, -0.6961928, -0.52507305, -0.39491749, -0.28444138, -0.18477343,
    -0.09105004, 0.0, 0.07958030, 0.16093020, 0.24611230, 0.33791524,
    0.44070983, 0.56261700, 0.72295684, 1.0,
], dtype=F32)


def quantize(weight, values, *, group, integer, asym=False, scale="absmax", fmt="fp16",
             fractions=None) -> dict:
    """End-to-end ``Scaled(...)(w)``: returns codes, scales, zero, group, bits."""
    weight = np.asarray(weight, dtype=F32)
    values = np.asarray(values, dtype=F32)
    rows, width = weight.shape
    group = width if group is None else min(group, width)
    scales, zero = initial_scales(weight, values, group, asym)
    scales, scale_bits = store_scale(scales, fmt)
    if scale == "mse":
        if fractions is None:
            fractions = np.linspace(0.5, 1.0, 20).astype(F32)
        scales = search_scales(weight, scales, zero, values, fractions, group, fmt, integer)
    side_bits = scales.size * scale_bits * (2 if zero is not None else 1)
    if zero is not None:
        zero = stored_offset(zero, fmt)
    codes = encode(weight, scales, zero, values, group, integer)
    return {"codes": codes, "scales": scales, "zero": zero, "group": group, "values": values,
            "side_bits": side_bits}
