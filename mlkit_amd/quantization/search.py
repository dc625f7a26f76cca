"""Nearest-entry search over an ascending scalar codebook (ties choose the lower entry).

``snap`` has the call surface of the reference's
/root/reference/src/mlkit/quantization/operations/search.py:9-27; FP32 HIP tensors run
``mk_snap``.  Tensors that track gradients, other dtypes and host tensors use the bisection
in tensor operations, which is the same rule the kernel implements.
"""

import torch
from torch import Tensor


def nearest_indices(value: Tensor, table: Tensor) -> Tensor:
    """Index of the nearest entry of the ascending ``table``; equal distances pick the lower."""
    upper = torch.searchsorted(table, value.contiguous()).clamp_max(table.numel() - 1)
    lower = (upper - 1).clamp_min(0)
    take_lower = (value - table[lower]).abs() <= (value - table[upper]).abs()
    return torch.where(take_lower, lower, upper)


def snap(value: Tensor, codebook: Tensor) -> Tensor:
    table = codebook.to(device=value.device, dtype=value.dtype).flatten().sort().values
    if table.numel() == 0:
        raise ValueError("codebook cannot be empty")
    tracked = torch.is_grad_enabled() and (value.requires_grad or table.requires_grad)
    if value.is_cuda and value.dtype == torch.float32 and not tracked and value.numel() and table.numel() <= 256:
        from mlkit_amd.kernels import scalar_encode

        return scalar_encode.snap(value.contiguous(), table)
    return table[nearest_indices(value, table)]
