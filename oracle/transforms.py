"""Oracle (test infrastructure): Walsh-Hadamard and structured orthogonal transforms.

Follows, in the reference:
  operations/orthogonal_transforms.py:12-31    hadamard (stage by stage)
  kernels/hadamard.py:108-136                  normalisation: multiply by fp32(1/fp32(sqrt n))
  operations/orthogonal_transforms.py:34-67    prime, paley_matrix
  operations/orthogonal_transforms.py:70-98    transform_factor
  operations/orthogonal_transforms.py:101-109  structured_transform
  operations/orthogonal_transforms.py:112-122  randomized_transform / rht (signs are an input here)
  codecs/composition.py:14-20                  deterministic_signs
  quantization/context.py:11-13                layer_seed
"""

import hashlib
import math

import numpy as np

F32 = np.float32


def normaliser(width: int) -> np.float32:
    """The constant the fused kernel multiplies by: fp32(1) / fp32(sqrt(width))."""
    return F32(1.0) / F32(math.sqrt(width))


def fwht(value: np.ndarray, normalize: bool = True) -> np.ndarray:
    """Radix-2 butterflies in ascending stride along the last axis, fp32 adds."""
    value = np.asarray(value, dtype=F32)
    width = value.shape[-1]
    if width <= 0 or width & (width - 1):
        raise ValueError("hadamard currently requires a power-of-two final dimension")
    out = value.copy()
    stride = 1
    while stride < width:
        pairs = out.reshape(*value.shape[:-1], -1, 2, stride)
        first, second = pairs[..., 0, :], pairs[..., 1, :]
        out = np.stack(((first + second).astype(F32), (first - second).astype(F32)), axis=-2)
        out = out.reshape(value.shape)
        stride *= 2
    return (out * normaliser(width)).astype(F32) if normalize else out


def prime(value: int) -> bool:
    return value >= 2 and all(value % d for d in range(2, math.isqrt(value) + 1))


def _characters(field: int) -> np.ndarray:
    """Quadratic-character matrix chi(i - j) over the prime field."""
    index = np.arange(field)
    squares = np.zeros(field, dtype=F32)
    squares[(index[1:] ** 2) % field] = 1
    difference = (index[:, None] - index[None, :]) % field
    return np.where(difference == 0, F32(0), 2 * squares[difference] - 1).astype(F32)


def paley(order: int) -> np.ndarray:
    """Orthonormal Paley-I (q = order-1 = 3 mod 4) or Paley-II (q = order/2-1 = 1 mod 4)."""
    if prime(order - 1) and (order - 1) % 4 == 3:
        field = order - 1
        matrix = np.ones((order, order), dtype=F32)
        matrix[1:, 0] = -1
        matrix[1:, 1:] = _characters(field) + np.eye(field, dtype=F32)
        return (matrix / F32(math.sqrt(order))).astype(F32)
    field = order // 2 - 1
    if order % 2 == 0 and prime(field) and field % 4 == 1:
        conference = np.ones((field + 1, field + 1), dtype=F32)
        conference[0, 0] = 0
        conference[1:, 1:] = _characters(field)
        identity = np.eye(field + 1, dtype=F32)
        matrix = np.block([[conference + identity, conference - identity],
                           [conference - identity, -conference - identity]]).astype(F32)
        return (matrix / F32(math.sqrt(order))).astype(F32)
    raise ValueError(f"no prime-field Paley construction for order {order}")


def transform_factor(width: int):
    """``(order, power, basis)``: dense orthonormal basis order times a Hadamard power of two."""
    if width < 1:
        raise ValueError("transform width must be positive")
    if width & (width - 1) == 0:
        return 1, width, None
    odd = width
    while odd % 2 == 0:
        odd //= 2
    power = width // odd
    for multiplier in (1, 2, 4, 8, 16):
        if power % multiplier:
            continue
        try:
            return odd * multiplier, power // multiplier, paley(odd * multiplier)
        except ValueError:
            continue
    index = np.arange(odd, dtype=np.float64)
    matrix = np.cos(math.pi / odd * (index[None, :] + 0.5) * index[:, None])
    matrix[0] *= 1 / math.sqrt(odd)
    matrix[1:] *= math.sqrt(2 / odd)
    return odd, power, matrix.astype(F32)


def structured(value: np.ndarray, inverse: bool = False) -> np.ndarray:
    """``(basis (x) H_power)`` along the last axis; the basis product is tolerance-level."""
    value = np.asarray(value, dtype=F32)
    order, power, basis = transform_factor(value.shape[-1])
    if basis is None:
        return fwht(value)
    blocks = fwht(value.reshape(*value.shape[:-1], order, power))
    mix = basis.T if inverse else basis
    # out[..., f', p] = sum_f mix[f', f] * blocks[..., f, p]
    out = np.einsum("af,...fp->...ap", mix.astype(np.float64), blocks.astype(np.float64))
    return out.astype(F32).reshape(value.shape)


def randomized(value: np.ndarray, signs: np.ndarray, inverse: bool = False) -> np.ndarray:
    signs = np.asarray(signs, dtype=F32)
    if inverse:
        return (structured(value, inverse=True) * signs).astype(F32)
    return structured((np.asarray(value, dtype=F32) * signs).astype(F32))


def deterministic_signs(width: int, seed: int) -> np.ndarray:
    """Integer-hash Rademacher signs, identical on every device."""
    out = np.empty(width, dtype=F32)
    for index in range(width):
        v = (index + seed) & 0xFFFFFFFF
        for _ in range(2):
            v = ((v ^ (v >> 16)) * 0x45D9F3B) & 0xFFFFFFFF
        v ^= v >> 16
        out[index] = (v & 1) * 2 - 1
    return out


def layer_seed(name: str, seed: int = 0) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") % (2**63 - 1)


def sylvester(width: int) -> np.ndarray:
    """The natural-order +-1 Hadamard matrix, for brute-force checks."""
    matrix = np.ones((1, 1), dtype=np.float64)
    while matrix.shape[0] < width:
        matrix = np.block([[matrix, matrix], [matrix, -matrix]])
    return matrix
