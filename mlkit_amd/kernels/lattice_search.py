"""Nearest-codeword search on a HIP device: any codebook of 2-, 4-, 8- or 16-dimensional
codewords, and the structured search of the E8P lattice.

``search`` has the call surface of the reference's
/root/reference/src/mlkit/kernels/lattice_search.py:60-70; ``nearest`` is the device side of
quantization/operations/search.py:34-79.  Both run ``mk_vector_nearest``.
"""

import torch
from torch import Tensor

from mlkit_amd import native

DIMENSIONS = (2, 4, 8, 16)


def _codes(vectors: Tensor, table: Tensor, dimension: int, size: int, lattice: bool) -> Tensor:
    device = native.require_device(vectors, table)
    flat = vectors.reshape(-1, dimension).to(torch.float32).contiguous()
    codes = torch.empty(flat.shape[0], device=device, dtype=torch.int32)
    native.check(native.library().mk_vector_nearest(
        flat.data_ptr(), flat.shape[0], dimension, table.data_ptr(), size, int(lattice), codes.data_ptr(),
        native.current_stream(device),
    ))
    return codes.reshape(vectors.shape[:-1])


def search(inputs: Tensor, table: Tensor) -> Tensor:
    """E8P codes (int32) of ``inputs[..., 8]``; ``table`` is the 65,536 points followed by the
    256 magnitude patterns, FP32, contiguous."""
    if inputs.shape[-1] != 8 or tuple(table.shape) != (65536 + 256, 8):
        raise ValueError("the lattice search takes eight-dimensional inputs and the full E8P table")
    if table.dtype != torch.float32 or not table.is_contiguous():
        raise ValueError("the E8P table must be a contiguous FP32 tensor")
    return _codes(inputs, table, 8, 65536, True)


def nearest(inputs: Tensor, codebook: Tensor) -> Tensor:
    """Index (int32) of the codeword nearest to every ``inputs[..., dimension]``."""
    dimension = codebook.shape[1]
    if dimension not in DIMENSIONS or inputs.shape[-1] != dimension:
        raise ValueError(f"codewords of {DIMENSIONS} coordinates matching the inputs are required")
    table = codebook.to(torch.float32).contiguous()
    return _codes(inputs, table, dimension, table.shape[0], False)
