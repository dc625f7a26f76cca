"""Oracle (test infrastructure): little-endian unsigned bit streams.

Restates ``quantization/operations/bit_packing.py:13-135`` of the reference as a
closed form: bit ``i*b + t`` of the stream is bit ``t`` of code ``i`` (LSB first) and
byte ``j`` of the stream holds stream bits ``[8j, 8j+8)``, bit 0 in the byte's LSB.
The stream is zero padded to a whole byte and is ``ceil(n*b/8)`` bytes long.
"""

import math

import numpy as np


def pack(codes: np.ndarray, bits: int) -> np.ndarray:
    """``pack`` (bit_packing.py:13-29): flatten, range check, emit the bit stream."""
    if not 1 <= bits <= 16:
        raise ValueError("packing supports one through sixteen bits")
    flat = np.asarray(codes).reshape(-1)
    if flat.dtype.kind not in "iub":
        raise TypeError("codes must have an integer dtype")
    if flat.size and (int(flat.min()) < 0 or int(flat.max()) >= 2**bits):
        raise ValueError("codes exceed the declared unsigned bit capacity")
    wide = flat.astype(np.uint32)
    planes = ((wide[:, None] >> np.arange(bits, dtype=np.uint32)[None, :]) & 1).astype(np.uint8)
    stream = planes.reshape(-1)
    return np.packbits(stream, bitorder="little")[: math.ceil(flat.size * bits / 8)]


def unpack(packed: np.ndarray, bits: int, shape: tuple[int, ...]) -> np.ndarray:
    """``unpack`` (bit_packing.py:80-100): uint8 codes up to 8 bits, int32 above."""
    packed = np.asarray(packed)
    if not 1 <= bits <= 16 or packed.dtype != np.uint8:
        raise ValueError("unpack requires uint8 storage and one through sixteen bits")
    if any(dimension < 0 for dimension in shape):
        raise ValueError("shape dimensions must be nonnegative")
    count = math.prod(shape)
    if packed.size != math.ceil(count * bits / 8):
        raise ValueError("packed byte count does not match the declared shape and precision")
    stream = np.unpackbits(packed.reshape(-1), bitorder="little")[: count * bits]
    planes = stream.reshape(count, bits).astype(np.uint32)
    values = (planes << np.arange(bits, dtype=np.uint32)[None, :]).sum(axis=1, dtype=np.uint32)
    return values.astype(np.uint8 if bits <= 8 else np.int32).reshape(shape)


def pack_bitwise_python(codes: list[int], bits: int) -> bytes:
    """Brute-force packer for tiny inputs: one Python big integer holds the whole stream."""
    stream = 0
    for index, code in enumerate(codes):
        stream |= (code & ((1 << bits) - 1)) << (index * bits)
    return stream.to_bytes(math.ceil(len(codes) * bits / 8), "little")
