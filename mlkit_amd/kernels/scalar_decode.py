"""Reconstruction of unpacked scalar codes: ``values[codes] * scales (+ zeros)``.

Same call surface as the reference's ``kernels/scalar_decode.py`` (``tile_for``, ``decode``;
/root/reference/src/mlkit/kernels/scalar_decode.py:30-97); ``refit`` adds the scale indexing
of the error-feedback codec (quantization/codecs/scaled.py:67-101).
"""

import torch
from torch import Tensor

from mlkit_amd import native
from mlkit_amd.kernels.scalar_encode import tile_for  # noqa: F401  (same rule on both sides)


def decode(
    codes: Tensor,
    scales: Tensor,
    values: Tensor,
    zeros: Tensor | None,
    group: int,
    tile: int | None = None,
    *,
    refit: int = 0,
) -> Tensor:
    """Reconstruct ``values[codes] * scales + zeros`` with one scale per row and group."""
    device = native.require_device(codes, scales, values, zeros)
    if codes.dim() != 2 or codes.dtype != torch.uint8 or not codes.is_contiguous():
        raise ValueError("codes must be a contiguous two-dimensional uint8 tensor")
    rows, width = codes.shape
    for name, side in (("scales", scales), ("zeros", zeros)):
        if side is not None and (side.dtype != torch.float32 or not side.is_contiguous() or side.shape[0] != rows):
            raise ValueError(f"{name} must be a contiguous FP32 tensor with one row per code row")
    output = torch.empty((rows, width), device=device, dtype=torch.float32)
    if output.numel() == 0:
        return output
    values = values.to(torch.float32).contiguous()
    native.check(native.library().mk_scalar_decode(
        codes.data_ptr(), scales.data_ptr(), values.data_ptr(), values.numel(), native.pointer(zeros),
        output.data_ptr(), rows, width, group, scales.shape[1], refit, native.current_stream(device),
    ))
    return output
