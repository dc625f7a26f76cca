"""Packing of integer codes into a little-endian bit stream, and back.

Code ``i`` of width ``b`` occupies stream bits ``[i*b, (i+1)*b)``; byte ``j`` holds stream
bits ``[8j, 8j+8)``, least significant first.  Same layout, return types and errors as the
reference's ``pack`` / ``unpack`` (/root/reference/src/mlkit/quantization/operations/
bit_packing.py:13-135); the stream is what ``PackedLinear.packed`` and checkpoints hold.
These are tensor operations on whatever device the codes live on.
"""

import math

import torch
from torch import Tensor


def _period(bits: int) -> tuple[int, int]:
    """(codes, bytes) of the shortest run of whole codes that fills whole bytes."""
    common = math.gcd(bits, 8)
    return 8 // common, bits // common


def pack(codes: Tensor, bits: int) -> Tensor:
    """A flat uint8 tensor of ``ceil(codes.numel() * bits / 8)`` bytes."""
    if not 1 <= bits <= 16:
        raise ValueError("packing supports one through sixteen bits")
    if codes.is_floating_point() or codes.is_complex():
        raise TypeError("codes must have an integer dtype")
    flat = codes.detach().reshape(-1).to(torch.int64)
    if flat.numel() and (int(flat.min()) < 0 or int(flat.max()) >= 1 << bits):
        raise ValueError(f"codes exceed the unsigned capacity of {bits} bits")
    count = flat.numel()
    per_period, period_bytes = _period(bits)
    padded = -(-count // per_period) * per_period
    if padded != count:
        flat = torch.cat([flat, flat.new_zeros(padded - count)])
    # A period of codes is at most 16 * 8 = 128 bits: assemble it in two 64-bit halves
    # only when needed; with bits <= 8 a period is at most 64 bits.
    grouped = flat.view(-1, per_period)
    out = torch.zeros((grouped.shape[0], period_bytes), dtype=torch.int64, device=codes.device)
    for index in range(per_period):
        start = index * bits
        value = grouped[:, index]
        first_byte, shift = divmod(start, 8)
        spread = value << shift  # at most 16 + 7 bits
        for byte in range((shift + bits + 7) // 8):
            out[:, first_byte + byte] |= (spread >> (8 * byte)) & 0xFF
    return out.to(torch.uint8).reshape(-1)[: (count * bits + 7) // 8]


def unpack(packed: Tensor, bits: int, shape: tuple[int, ...]) -> Tensor:
    """The codes of a stream as a tensor of ``shape``: uint8 for up to 8 bits, int32 above."""
    if not 1 <= bits <= 16 or packed.dtype != torch.uint8:
        raise ValueError("unpack requires uint8 storage and one through sixteen bits")
    shape = tuple(shape)
    if any(dimension < 0 for dimension in shape):
        raise ValueError("shape dimensions must be nonnegative")
    count = math.prod(shape)
    needed = (count * bits + 7) // 8
    if packed.numel() != needed:
        raise ValueError(f"packed byte count {packed.numel()} does not match shape {shape} at {bits} bits")
    per_period, period_bytes = _period(bits)
    periods = -(-count // per_period)
    stream = packed.reshape(-1).to(torch.int64)
    if stream.numel() != periods * period_bytes:
        stream = torch.cat([stream, stream.new_zeros(periods * period_bytes - stream.numel())])
    grouped = stream.view(periods, period_bytes)
    out = torch.empty((periods, per_period), dtype=torch.int64, device=packed.device)
    mask = (1 << bits) - 1
    for index in range(per_period):
        first_byte, shift = divmod(index * bits, 8)
        value = torch.zeros(periods, dtype=torch.int64, device=packed.device)
        for byte in range((shift + bits + 7) // 8):
            value |= grouped[:, first_byte + byte] << (8 * byte)
        out[:, index] = (value >> shift) & mask
    return out.reshape(-1)[:count].to(torch.uint8 if bits <= 8 else torch.int32).reshape(shape)
