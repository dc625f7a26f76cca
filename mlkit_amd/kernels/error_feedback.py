"""LDL error feedback: tile sweep, pending-continuation solve and trailing block update.

``round_tile`` has the call surface of the reference's ``kernels/error_feedback.py``
(/root/reference/src/mlkit/kernels/error_feedback.py:99-143).  ``pending_continuation`` and
``block_update`` replace the ``solve_triangular`` and ``addmm_`` calls of
quantization/algorithms/error_feedback.py:366-393.
"""

import torch
from torch import Tensor

from mlkit_amd import native

MAXIMUM_TILE_WIDTH = 1024


def _check(name: str, tensor: Tensor, shape: tuple[int, ...] | None = None) -> None:
    if tensor.dtype != torch.float32 or not tensor.is_contiguous():
        raise ValueError(f"{name} must be a contiguous FP32 tensor")
    if shape is not None and tuple(tensor.shape) != shape:
        raise ValueError(f"{name} must have shape {shape}, got {tuple(tensor.shape)}")


def round_tile(
    original: Tensor,
    feedback: Tensor,
    coefficients: Tensor,
    scales: Tensor,
    zeros: Tensor | None,
    output: Tensor,
    encoded: Tensor,
    *,
    region_start: int,
    tile_start: int,
    tile_width: int,
    group: int,
    bits: int,
    values: Tensor,
    integer_grid: bool,
) -> None:
    """Round columns ``tile_start`` to ``tile_start + tile_width`` of every row."""
    device = native.require_device(original, feedback, coefficients, scales, zeros, output, encoded, values)
    rows, width = original.shape
    _check("original", original)
    _check("feedback", feedback, (rows, width))
    _check("coefficients", coefficients, (width, width))
    _check("output", output, (rows, width))
    _check("scales", scales)
    if zeros is not None:
        _check("zeros", zeros, tuple(scales.shape))
    if encoded.dtype != torch.uint8 or tuple(encoded.shape) != (rows, width) or not encoded.is_contiguous():
        raise ValueError("encoded must be a contiguous uint8 tensor shaped like the weight")
    values = values.to(torch.float32).contiguous()
    native.check(native.library().mk_feedback_round_tile(
        original.data_ptr(), feedback.data_ptr(), coefficients.data_ptr(), scales.data_ptr(),
        native.pointer(zeros), values.data_ptr(), values.numel(), output.data_ptr(), encoded.data_ptr(),
        rows, width, region_start, tile_start, tile_width, group, scales.shape[1], int(integer_grid),
        float(-(2 ** (bits - 1))), float(2 ** (bits - 1) - 1), native.current_stream(device),
    ))


def pending_continuation(
    feedback: Tensor,
    coefficients: Tensor,
    region_start: int,
    region_stop: int,
    original: Tensor | None = None,
) -> Tensor:
    """``feedback[:, region] @ inverse(coefficients[region, region])`` (unit upper triangular).

    With ``original`` the region's weights are added, which gives the targets a region's
    format is fitted to.
    """
    device = native.require_device(feedback, coefficients, original)
    rows, width = feedback.shape
    _check("feedback", feedback)
    _check("coefficients", coefficients, (width, width))
    if original is not None:
        _check("original", original, (rows, width))
    output = torch.empty((rows, region_stop - region_start), device=device, dtype=torch.float32)
    native.check(native.library().mk_feedback_pending(
        feedback.data_ptr(), coefficients.data_ptr(), native.pointer(original), output.data_ptr(), rows,
        width, region_start, region_stop, native.current_stream(device),
    ))
    return output


def block_update(
    feedback: Tensor,
    original: Tensor,
    output: Tensor,
    coefficients: Tensor,
    tile_start: int,
    tile_stop: int,
) -> None:
    """``feedback[:, stop:] += (original - output)[:, start:stop] @ coefficients[start:stop, stop:]``."""
    device = native.require_device(feedback, original, output, coefficients)
    rows, width = original.shape
    _check("original", original)
    _check("feedback", feedback, (rows, width))
    _check("output", output, (rows, width))
    _check("coefficients", coefficients, (width, width))
    native.check(native.library().mk_feedback_block_update(
        feedback.data_ptr(), original.data_ptr(), output.data_ptr(), coefficients.data_ptr(), rows, width,
        tile_start, tile_stop, native.current_stream(device),
    ))


def block_update_range(
    feedback: Tensor,
    original: Tensor,
    output: Tensor,
    coefficients: Tensor,
    first_column: int,
    chain_width: int,
    chains: int,
    column_begin: int,
    column_end: int,
) -> None:
    """The updates of ``chains`` consecutive tiles applied to columns ``[column_begin,
    column_end)`` in one pass, with the roundings of applying them tile after tile."""
    device = native.require_device(feedback, original, output, coefficients)
    rows, width = original.shape
    _check("original", original)
    _check("feedback", feedback, (rows, width))
    _check("output", output, (rows, width))
    _check("coefficients", coefficients, (width, width))
    native.check(native.library().mk_feedback_block_update_range(
        feedback.data_ptr(), original.data_ptr(), output.data_ptr(), coefficients.data_ptr(), rows, width,
        first_column, chain_width, chains, column_begin, column_end, native.current_stream(device),
    ))


def sweep(
    original: Tensor,
    feedback: Tensor,
    output: Tensor,
    encoded: Tensor,
    coefficients: Tensor,
    *,
    values: Tensor,
    group: int,
    refit: int,
    block: int,
    integer_grid: bool,
    code_minimum: float,
    code_maximum: float,
    asym: bool,
    reciprocal: float,
    value_minimum: float,
    scale_format: str,
    deferred_tiles: int = 4,
) -> tuple[Tensor, Tensor | None]:
    """The whole natural-order sweep in one call; returns the regions' scales (and offsets)
    side by side, ``[rows, total groups]``."""
    device = native.require_device(original, feedback, output, encoded, coefficients, values)
    rows, width = original.shape
    _check("original", original)
    _check("feedback", feedback, (rows, width))
    _check("output", output, (rows, width))
    _check("coefficients", coefficients, (width, width))
    if encoded.dtype != torch.uint8 or tuple(encoded.shape) != (rows, width) or not encoded.is_contiguous():
        raise ValueError("encoded must be a contiguous uint8 tensor shaped like the weight")
    region = min(refit, width)
    groups = 0
    for start in range(0, width, region):
        span = min(region, width - start)
        groups += -(-span // min(group, span))
    scales = torch.empty((rows, groups), device=device, dtype=torch.float32)
    zeros = torch.empty_like(scales) if asym else None
    workspace = torch.empty((rows, region), device=device, dtype=torch.float32) if region < width else None
    # column-major deviations of finished columns: what the trailing updates multiply
    deviations = torch.empty((width, rows), device=device, dtype=torch.float32) if rows % 4 == 0 and width % 4 == 0 else None
    values = values.to(torch.float32).contiguous()
    native.check(native.library().mk_feedback_sweep(
        original.data_ptr(), feedback.data_ptr(), output.data_ptr(), encoded.data_ptr(), coefficients.data_ptr(),
        scales.data_ptr(), native.pointer(zeros), native.pointer(workspace), native.pointer(deviations),
        values.data_ptr(), values.numel(),
        rows, width, group, refit, block, int(integer_grid), float(code_minimum), float(code_maximum), int(asym),
        float(reciprocal), float(value_minimum), native.SCALE_FORMAT_CODES[scale_format], deferred_tiles,
        native.current_stream(device),
    ))
    return scales, zeros


MAXIMUM_VECTOR_TILE_WIDTH = 256


def round_vector_tile(
    original: Tensor,
    feedback: Tensor,
    coefficients: Tensor,
    scales: Tensor,
    codebook: Tensor,
    output: Tensor,
    encoded: Tensor,
    *,
    region_start: int,
    tile_start: int,
    tile_width: int,
    group: int,
    dimension: int,
    codebook_size: int,
    lattice: bool,
) -> None:
    """Round columns ``tile_start`` to ``tile_start + tile_width`` of every row in blocks of
    ``dimension`` columns (/root/reference/src/mlkit/kernels/error_feedback.py:241-274).
    ``codebook`` holds the reconstruction of every code; for the lattice its 256 magnitude
    patterns follow the ``codebook_size`` points."""
    device = native.require_device(original, feedback, coefficients, scales, codebook, output, encoded)
    rows, width = original.shape
    _check("original", original)
    _check("feedback", feedback, (rows, width))
    _check("coefficients", coefficients, (width, width))
    _check("output", output, (rows, width))
    _check("scales", scales)
    _check("codebook", codebook, (codebook_size + (256 if lattice else 0), dimension))
    if encoded.dtype != torch.int32 or tuple(encoded.shape) != (rows, width // dimension) or not encoded.is_contiguous():
        raise ValueError("encoded must be a contiguous int32 tensor with one code per block of columns")
    native.check(native.library().mk_feedback_round_vector_tile(
        original.data_ptr(), feedback.data_ptr(), coefficients.data_ptr(), scales.data_ptr(), codebook.data_ptr(),
        output.data_ptr(), encoded.data_ptr(), rows, width, region_start, tile_start, tile_width, group,
        scales.shape[1], dimension, codebook_size, int(lattice), native.current_stream(device),
    ))
