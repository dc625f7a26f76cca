"""Walsh-Hadamard transform along the last dimension, one launch per tensor.

Same call surface as the reference's ``kernels/hadamard.py`` (``transform``;
/root/reference/src/mlkit/kernels/hadamard.py:108-136), widened to fp16 / bf16 tensors
(computed in fp32) and to fused sign flips; ``mix_blocks`` is the dense basis product of
the blocked transform (quantization/operations/orthogonal_transforms.py:101-109).
"""

import math

import numpy as np
import torch
from torch import Tensor

from mlkit_amd import native


def normaliser(width: int) -> float:
    """``fp32(1) / fp32(sqrt(width))``, the constant the normalised transform multiplies by."""
    return float(np.float32(1.0) / np.float32(math.sqrt(width)))


def transform(
    value: Tensor,
    *,
    normalize: bool = True,
    signs_before: Tensor | None = None,
    signs_after: Tensor | None = None,
    out: Tensor | None = None,
) -> Tensor:
    """The transform of every row of ``value`` (any leading shape, power-of-two last dimension).

    ``signs_before`` / ``signs_after`` are FP32 vectors of +-1 whose length is a multiple of
    the last dimension; they multiply the flattened input / output periodically, so a
    ``[..., order, power]`` view of wider rows can carry one sign per original column.
    """
    device = native.require_device(value, signs_before, signs_after, out)
    width = value.shape[-1]
    if width <= 0 or width & (width - 1):
        raise ValueError("hadamard currently requires a power-of-two final dimension")
    if not value.is_contiguous():
        raise ValueError("hadamard requires a contiguous tensor")
    output = torch.empty_like(value) if out is None else out
    if output.shape != value.shape or not output.is_contiguous():
        raise ValueError("hadamard output must be contiguous and shaped like its input")
    period = 0
    for signs in (signs_before, signs_after):
        if signs is None:
            continue
        if signs.dtype != torch.float32 or not signs.is_contiguous() or signs.numel() % width:
            raise ValueError("sign vectors must be contiguous FP32 with a multiple of the row width entries")
        if period and signs.numel() != period:
            raise ValueError("sign vectors must have equal lengths")
        period = signs.numel()
    rows = value.numel() // width
    native.check(native.library().mk_fwht(
        value.data_ptr(), native.dtype_code(value), output.data_ptr(), native.dtype_code(output), rows,
        width, native.pointer(signs_before), native.pointer(signs_after), period,
        normaliser(width) if normalize else 1.0, native.current_stream(device),
    ))
    return output


def mix_blocks(value: Tensor, basis: Tensor, *, transpose: bool, signs_after: Tensor | None = None) -> Tensor:
    """``out[..., f', p] = sum_f mix[f', f] * value[..., f, p]`` with ``mix = basis`` or ``basis.T``."""
    device = native.require_device(value, basis, signs_after)
    if value.dtype != torch.float32 or not value.is_contiguous() or value.dim() < 2:
        raise ValueError("mix_blocks requires a contiguous FP32 tensor [..., order, power]")
    order, power = value.shape[-2], value.shape[-1]
    if basis.shape != (order, order) or basis.dtype != torch.float32 or not basis.is_contiguous():
        raise ValueError("basis must be a contiguous FP32 [order, order] matrix")
    output = torch.empty_like(value)
    rows = value.numel() // (order * power)
    native.check(native.library().mk_basis_mix(
        value.data_ptr(), output.data_ptr(), basis.data_ptr(), rows, order, power, int(transpose),
        native.pointer(signs_after), native.current_stream(device),
    ))
    return output


MAXIMUM_FUSED_ORDER = 96      # basis rows the one-launch blocked transform handles
MAXIMUM_FUSED_LDS = 160 * 1024


def fits_one_launch(order: int, power: int) -> bool:
    """Whether ``rotate_blocks`` takes ``order`` blocks of ``power`` values (one workgroup holds them)."""
    if order > MAXIMUM_FUSED_ORDER or power < 32 or power & (power - 1):
        return False
    padded = power + (power >> 4)
    if (order * padded + order * order) * 4 > MAXIMUM_FUSED_LDS:
        return False
    return order * (power // 16) <= 1024 or order * (power // 32) <= 1024


def streams_in_one_pass(value: Tensor, order: int, power: int) -> bool:
    """Whether ``rotate_blocks`` has its register-resident one-pass kernel for a weight-sized
    ``value``: FP32, at most 32 blocks of 256 or 512 values that fit half a CU's LDS beside the
    basis."""
    return (value.dtype == torch.float32 and order <= 32 and power in (256, 512)
            and (order * power + 1024) * 4 <= MAXIMUM_FUSED_LDS // 2 and value.data_ptr() % 16 == 0)


def rotate_blocks(
    value: Tensor,
    basis: Tensor,
    *,
    transpose: bool,
    signs_before: Tensor | None = None,
    signs_after: Tensor | None = None,
    normalize: bool = True,
) -> Tensor:
    """``transform`` of every block of a ``[..., order, power]`` tensor followed by ``mix_blocks``,
    in one launch and in ``value``'s dtype; bit-identical to the two calls."""
    device = native.require_device(value, basis, signs_before, signs_after)
    if value.dim() < 2 or not value.is_contiguous():
        raise ValueError("rotate_blocks requires a contiguous tensor [..., order, power]")
    order, power = value.shape[-2], value.shape[-1]
    if basis.shape != (order, order) or basis.dtype != torch.float32 or not basis.is_contiguous():
        raise ValueError("basis must be a contiguous FP32 [order, order] matrix")
    for signs in (signs_before, signs_after):
        if signs is not None and (signs.dtype != torch.float32 or not signs.is_contiguous()
                                  or signs.numel() != order * power):
            raise ValueError("sign vectors must be contiguous FP32 with order * power entries")
    output = torch.empty_like(value)
    rows = value.numel() // (order * power)
    native.check(native.library().mk_rotate_blocks(
        value.data_ptr(), native.dtype_code(value), output.data_ptr(), native.dtype_code(output), rows,
        order, power, basis.data_ptr(), int(transpose), native.pointer(signs_before),
        native.pointer(signs_after), normaliser(power) if normalize else 1.0, native.current_stream(device),
    ))
    return output
