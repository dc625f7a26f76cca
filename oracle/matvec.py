"""Oracle (test infrastructure): reconstruct-then-matmul, the reference's CPU path.

``PackedLinear`` is defined to equal the dense layer built from the dequantised weight
(``inference/packed_linear.py:110-154``, dequantisation ``kernels/packed_linear.py:156-165``):
``w = values[code] * scale (+ zero)`` in fp32, then ``y = x @ w.T (+ bias)`` accumulated in
fp32 and cast to the dtype of ``x``.
"""

import numpy as np

from . import bitstream, scaling

F32 = np.float32


def dequantise(packed, bits, shape, scales, values, group, zero=None, uniform=None) -> np.ndarray:
    """Dense fp32 weight from the packed stream.

    ``uniform=(minimum, step)`` selects ``minimum + code*step`` instead of the table
    (kernels/packed_linear.py:158-161); for integer grids both give the same floats.
    """
    codes = bitstream.unpack(packed, bits, shape)
    if uniform is not None:
        table = (F32(uniform[0]) + np.arange(2**bits, dtype=F32) * F32(uniform[1])).astype(F32)
    else:
        table = np.asarray(values, dtype=F32)
    return scaling.decode_grouped(codes, np.asarray(scales, dtype=F32), table, group,
                                  None if zero is None else np.asarray(zero, dtype=F32))


def reconstruct_then_matmul(x, packed, bits, shape, scales, values, group, zero=None, bias=None,
                            dense=None) -> np.ndarray:
    """fp32 result ``[M, N]``; pass ``dense`` to time the matmul without the reconstruction."""
    if dense is None:
        dense = dequantise(packed, bits, shape, scales, values, group, zero)
    y = np.asarray(x, dtype=F32) @ dense.T
    if bias is not None:
        y = y + np.asarray(bias, dtype=F32)[None, :]
    return y.astype(F32)


def reconstruct_then_matmul_f64(x, dense, bias=None) -> np.ndarray:
    """Higher-precision yardstick for tolerance tests (float64 accumulate)."""
    y = np.asarray(x, dtype=np.float64) @ np.asarray(dense, dtype=np.float64).T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)[None, :]
    return y


def reconstruct_then_matmul_torch(x, packed, bits, shape, scales, values, group, zero=None, dense=None):
    """The same path as tensor operations on the host's cores, as the reference's own CPU path
    runs it (unpack: quantization/operations/bit_packing.py:80-99 for widths that divide a byte;
    decode: codecs/scaled.py:55-60; then ``x @ w.T`` in fp32).  All arguments are CPU tensors;
    returns ``(y, dense)`` so that a caller can time the product alone on the reconstruction."""
    import torch

    if dense is None:
        if 8 % bits:
            raise ValueError("the tensor restatement covers code widths that divide a byte")
        rows, width = shape
        stream = packed.flatten()
        mask = 2**bits - 1
        fields = [(stream >> shift) & mask for shift in range(0, 8, bits)]
        codes = torch.stack(fields, dim=1).flatten()[: rows * width].reshape(rows, width)
        reconstruction = values[codes.int()]
        grouped = reconstruction.reshape(rows, -1, group) * scales.float()[:, :, None]
        if zero is not None:
            grouped = grouped + zero.float()[:, :, None]
        dense = grouped.reshape(rows, width)
    return x.float() @ dense.T, dense
