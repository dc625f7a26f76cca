"""Grids: signed integers, explicit value tables, small floating-point formats, codebooks of
vectors and the E8P lattice.

Mirrors the reference's grid factory
(/root/reference/src/mlkit/quantization/grids/factory.py:17-125,146-152): ``Grid``,
``grid.int``, ``grid.values``, ``grid.vector``, ``grid.fp``, ``grid.e8p`` and ``NF4_VALUES``.
Trellis grids are outside this package's path.
"""

import builtins
import math
from collections.abc import Callable

import torch
from torch import Tensor


class Grid:
    """A rounding function and its cost in bits per ``dim`` elements.

    ``values`` lists the representable points (ascending) when they are known; ``integer``
    says they are consecutive integers, which round by arithmetic instead of a table search.
    """

    def __init__(self, function: Callable[[Tensor], Tensor], bits: int, dim: int = 1, *,
                 values: Tensor | None = None, name: str = "custom", integer: bool = False) -> None:
        if bits < 1 or dim < 1:
            raise ValueError("grid bits and dimension must be positive")
        self.function, self.bits, self.dim = function, bits, dim
        self.values, self.name, self.integer = values, name, integer

    def __call__(self, value: Tensor) -> Tensor:
        return self.function(value)

    def __repr__(self) -> str:
        return f"Grid({self.name}, bits={self.bits}, dim={self.dim})"


def _snap(value: Tensor, table: Tensor) -> Tensor:
    from mlkit_amd.quantization.search import snap

    return snap(value, table)


class GridFactory:
    """``grid.int(4)``, ``grid.values([...])``, ``grid.fp("e2m1")``; as a decorator,
    ``@grid(bits=3)`` wraps a rounding function."""

    def __call__(self, *, bits: int, dim: int = 1) -> Callable[[Callable[[Tensor], Tensor]], Grid]:
        return lambda function: Grid(function, bits, dim, name=function.__name__)

    def int(self, bits: int) -> Grid:
        if not 2 <= bits <= 16:
            raise ValueError("signed integer grids support 2 through 16 bits")
        low, high = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
        table = torch.arange(low, high + 1, dtype=torch.float32)
        return Grid(lambda x: x.round().clamp(low, high), bits, values=table, name=f"int{bits}", integer=True)

    def values(self, values: Tensor, *, bits: builtins.int | None = None, name: str = "values") -> Grid:
        table = torch.as_tensor(values, dtype=torch.float32).flatten().sort().values
        if table.numel() == 0 or not bool(torch.isfinite(table).all()):
            raise ValueError("a scalar codebook must contain finite values")
        width = max(1, math.ceil(math.log2(table.numel()))) if bits is None else bits
        if table.numel() > 2**width:
            raise ValueError("codebook size exceeds the declared bit capacity")
        return Grid(lambda x: _snap(x, table), width, values=table, name=name)

    def vector(self, codebook: Tensor, *, bits: builtins.int | None = None) -> Grid:
        """Round blocks of ``codebook.shape[1]`` values to the nearest row of ``codebook``."""
        table = torch.as_tensor(codebook, dtype=torch.float32)
        if table.ndim != 2 or min(table.shape) < 1 or not bool(torch.isfinite(table).all()):
            raise ValueError("a vector codebook must be a nonempty finite matrix")
        width = max(1, math.ceil(math.log2(table.shape[0]))) if bits is None else bits
        if table.shape[0] > 2**width:
            raise ValueError("codebook size exceeds the declared bit capacity")
        dimension = table.shape[1]

        def round_vectors(value: Tensor) -> Tensor:
            from mlkit_amd.quantization.search import nearest

            return nearest(value.reshape(-1, dimension), table).reshape_as(value)

        return Grid(round_vectors, width, dimension, values=table, name="vector")

    def e8p(self) -> Grid:
        """The 16-bit, eight-dimensional E8P lattice codebook."""
        from mlkit_amd.quantization.lattice import e8p_points, nearest_e8p

        return Grid(nearest_e8p, 16, 8, values=e8p_points(), name="e8p")

    def fp(self, format: str) -> Grid:
        """Sign-magnitude minifloats without infinities or NaNs: e2m1, e3m2, e2m3, e4m3, e5m2."""
        if format == "e2m1":
            positive = [0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
            return self.values(torch.tensor([-v for v in positive[::-1]] + [0.0] + positive), bits=4, name=format)
        if format not in {"e3m2", "e2m3", "e4m3", "e5m2"}:
            raise ValueError(f"unsupported floating-point grid {format!r}")
        exponent_bits, mantissa_bits = builtins.int(format[1]), builtins.int(format[3])
        bias = (1 << (exponent_bits - 1)) - 1
        fractions = [m / (1 << mantissa_bits) for m in range(1 << mantissa_bits)]
        magnitudes = {f * 2.0 ** (1 - bias) for f in fractions}  # subnormals and zero
        for exponent in range(1, (1 << exponent_bits) - 1):
            magnitudes.update((1 + f) * 2.0 ** (exponent - bias) for f in fractions)
        table = sorted({-m for m in magnitudes} | magnitudes)
        return self.values(torch.tensor(table), bits=1 + exponent_bits + mantissa_bits, name=format)


grid = GridFactory()

NF4_VALUES = torch.tensor([
    -1.0, -0.6961928, -0.52507305, -0.39491749, -0.28444138, -0.18477343, -0.09105004, 0.0,
    0.07958030, 0.16093020, 0.24611230, 0.33791524, 0.44070983, 0.56261700, 0.72295684, 1.0,
])
