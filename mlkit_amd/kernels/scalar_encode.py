"""Nearest-code encoding, scale fitting, the shrunken-scale search and codebook snapping.

Same call surface as the reference's ``kernels/scalar_encode.py`` (``tile_for``, ``encode``,
``search_scales``, ``snap``; /root/reference/src/mlkit/kernels/scalar_encode.py:58-146,
261-345) plus ``fit_scales``, which replaces the tensor reductions of ``Scaled._initial_scales``
(formats/grouped_scaling.py:274-289).  Every function enqueues one kernel of
``libmlkit_amd.so`` on the current HIP stream.
"""

import torch
from torch import Tensor

from mlkit_amd import native

MINIMUM_TILE = 16
MAXIMUM_TILE = 128


def tile_for(group: int) -> int | None:
    """Columns per tile in the reference's kernels: the largest power of two dividing a group.

    The HIP kernels accept any group; the value is kept for API parity and for capability
    reports (``None`` means the reference would not have taken its fused path).
    """
    tile = min(MAXIMUM_TILE, group & -group)
    return tile if tile >= MINIMUM_TILE else None


def _check_matrix(name: str, value: Tensor) -> None:
    if value.dim() != 2 or value.dtype != torch.float32 or not value.is_contiguous():
        raise ValueError(f"{name} must be a contiguous two-dimensional FP32 tensor")


def _check_side(name: str, side: Tensor | None, rows: int) -> None:
    if side is None:
        return
    if side.dim() != 2 or side.shape[0] != rows or side.dtype != torch.float32 or not side.is_contiguous():
        raise ValueError(f"{name} must be a contiguous FP32 tensor with one row per weight row")


def encode(
    value: Tensor,
    scales: Tensor,
    zeros: Tensor | None,
    values: Tensor,
    group: int,
    tile: int | None = None,
    *,
    integer: bool,
    minimum: float,
    maximum: float,
) -> Tensor:
    """Codes of the nearest grid values of ``(value - zeros) / scales``, one byte each."""
    device = native.require_device(value, scales, zeros, values)
    _check_matrix("value", value)
    rows, width = value.shape
    _check_side("scales", scales, rows)
    _check_side("zeros", zeros, rows)
    codes = torch.empty((rows, width), device=device, dtype=torch.uint8)
    if codes.numel() == 0:
        return codes
    values = values.to(torch.float32).contiguous()
    native.check(native.library().mk_scalar_encode(
        value.data_ptr(), scales.data_ptr(), native.pointer(zeros), values.data_ptr(), values.numel(),
        codes.data_ptr(), rows, width, group, scales.shape[1], int(integer), float(minimum),
        float(maximum), native.current_stream(device),
    ))
    return codes


def search_scales(
    value: Tensor,
    scales: Tensor,
    zeros: Tensor | None,
    values: Tensor,
    fractions: Tensor,
    group: int,
    tile: int | None,
    scale_format: str,
    *,
    integer: bool,
    minimum: float,
    maximum: float,
) -> Tensor:
    """For every row group, the candidate ``scales * fraction`` with least squared error.

    The stored scale itself is the first candidate and is kept on ties; candidates are
    rounded to ``scale_format`` before they are evaluated.
    """
    device = native.require_device(value, scales, zeros, values, fractions)
    _check_matrix("value", value)
    rows, width = value.shape
    _check_side("scales", scales, rows)
    _check_side("zeros", zeros, rows)
    selected = torch.empty_like(scales)
    values = values.to(torch.float32).contiguous()
    fractions = fractions.to(torch.float32).contiguous()
    native.check(native.library().mk_search_scales(
        value.data_ptr(), scales.data_ptr(), native.pointer(zeros), values.data_ptr(), values.numel(),
        fractions.data_ptr(), fractions.numel(), selected.data_ptr(), rows, width, group,
        scales.shape[1], native.SCALE_FORMAT_CODES[scale_format], int(integer), float(minimum),
        float(maximum), native.current_stream(device),
    ))
    return selected


def snap(value: Tensor, values: Tensor) -> Tensor:
    """The nearest entry of an ascending codebook for every element of ``value``."""
    device = native.require_device(value, values)
    if value.dtype != torch.float32 or not value.is_contiguous():
        raise ValueError("snap requires a contiguous FP32 tensor")
    output = torch.empty_like(value)
    values = values.to(torch.float32).contiguous()
    native.check(native.library().mk_snap(
        value.data_ptr(), values.data_ptr(), values.numel(), output.data_ptr(), value.numel(),
        native.current_stream(device),
    ))
    return output


def fit_scales(
    value: Tensor,
    group: int,
    *,
    asym: bool,
    reciprocal: float,
    value_minimum: float,
    scale_format: str,
    store_zero: bool,
) -> tuple[Tensor, Tensor | None]:
    """Stored scales (and offsets) of every row group from the group's range.

    ``value`` is an FP32 matrix whose rows may be strided (a column slice of a wider
    matrix).  ``reciprocal`` is ``fp32(1) / fp32(value range)`` of the grid.
    """
    device = native.require_device(value)
    if value.dim() != 2 or value.dtype != torch.float32 or value.stride(1) != 1:
        raise ValueError("fit_scales requires a two-dimensional FP32 tensor with unit column stride")
    rows, span = value.shape
    groups = -(-span // group)
    scales = torch.empty((rows, groups), device=device, dtype=torch.float32)
    zeros = torch.empty_like(scales) if asym else None
    row_stride = value.stride(0) if rows > 1 else span
    native.check(native.library().mk_fit_scales(
        value.data_ptr(), row_stride, scales.data_ptr(), native.pointer(zeros), rows, span, group,
        int(asym), float(reciprocal), float(value_minimum), native.SCALE_FORMAT_CODES[scale_format],
        int(store_zero), native.current_stream(device),
    ))
    return scales, zeros


def reconstruct(
    inputs: Tensor,
    values: Tensor,
    group: int,
    scale_format: str,
    asymmetric: bool,
    integer: bool,
    minimum: float,
    maximum: float,
    scale_reciprocal: float,
) -> Tensor:
    """Round ``inputs`` (two-dimensional, fp32 / fp16 / bf16) to a scaled scalar grid with scales
    fitted per group on the fly; same signature as the reference's
    kernels/activation_reconstruction.py:76-103."""
    device = native.require_device(inputs, values)
    if inputs.dim() != 2 or not inputs.is_contiguous():
        raise ValueError("reconstruct requires a contiguous two-dimensional tensor")
    output = torch.empty_like(inputs)
    values = values.to(torch.float32).contiguous()
    native.check(native.library().mk_reconstruct_activations(
        inputs.data_ptr(), native.dtype_code(inputs), output.data_ptr(), values.data_ptr(), values.numel(),
        inputs.shape[0], inputs.shape[1], min(group, inputs.shape[1]), native.SCALE_FORMAT_CODES[scale_format],
        int(asymmetric), int(integer), float(minimum), float(maximum), float(scale_reciprocal),
        native.current_stream(device),
    ))
    return output
