"""The value types every quantizer exchanges: ``Q``, ``Ctx`` and the ``Quantizer`` protocol.

Mirrors the reference's interfaces so that user code written against them keeps working:
  quantization/representation.py:9-75   Q, as_q
  quantization/context.py:11-163        layer_seed, Ctx
  quantization/protocol.py:17-164       ScalarRounding, FittedRounder, Quantizer, quantizer, fit_quantizer
(paths under /root/reference/src/mlkit).  Vector-grid rounding state is outside this
package's path and has no counterpart here.
"""

import dataclasses
import functools
import hashlib
import inspect
from collections.abc import Callable, Mapping
from typing import Any

import torch
from torch import Tensor, nn


class Q:
    """A quantized matrix: a dense reconstruction, or codes with the decoder that expands them.

    ``bits`` counts everything stored for the matrix, side information included (``None`` =
    unknown).  ``w`` decodes on every access, so decoder parameters stay live tensors.
    """

    def __init__(self, w: Tensor | None = None, *, bits: int | float | None = None,
                 codes: Tensor | None = None, params: Mapping[str, Any] | None = None,
                 decode: Callable[..., Tensor] | None = None, codec: str | None = None,
                 metadata: Mapping[str, Any] | None = None) -> None:
        if w is None and (codes is None or decode is None):
            raise ValueError("Q requires a reconstruction or codes and a decoder")
        if bits is not None and bits < 0:
            raise ValueError("bits must be nonnegative")
        self._dense = w
        self.bits = bits
        self.codes = codes
        self.params = dict(params or {})
        self.decode = decode
        self.codec = codec
        self.metadata = dict(metadata or {})

    @property
    def w(self) -> Tensor:
        if self.codes is not None and self.decode is not None:
            return self.decode(self.codes, **self.params)
        assert self._dense is not None
        return self._dense

    @property
    def bpw(self) -> float | None:
        if self.bits is None:
            return None
        return float(self.bits) / self.w.numel()

    def to(self, device: str | torch.device, *, detach: bool = False) -> "Q":
        def move(item: Any) -> Any:
            if isinstance(item, Tensor):
                return (item.detach() if detach else item).to(device)
            if isinstance(item, dict):
                return {key: move(value) for key, value in item.items()}
            return item

        return Q(move(self._dense), bits=self.bits, codes=move(self.codes), params=move(self.params),
                 decode=self.decode, codec=self.codec, metadata=self.metadata)

    def __repr__(self) -> str:
        return f"Q(shape={tuple(self.w.shape)}, bits={self.bits}, codec={self.codec!r})"


def as_q(value: "Q | Tensor") -> Q:
    if isinstance(value, Q):
        return value
    if isinstance(value, Tensor):
        return Q(value)
    raise TypeError(f"quantizers must return a Tensor or Q, received {type(value).__name__}")


def layer_seed(name: str, seed: int = 0) -> int:
    """A 63-bit seed that depends only on the layer name and the run seed (sha256)."""
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") % (2**63 - 1)


StatisticProvider = Callable[[str, Callable[[Tensor], Tensor] | None, str], Tensor]
_DERIVED_FROM_INPUTS: dict[str, Callable[[Tensor], Tensor]] = {
    "H": lambda x: x.T @ x / x.shape[0],
    "act_absmean": lambda x: x.abs().mean(0),
    "act_absmax": lambda x: x.abs().amax(0),
}


class Ctx:
    """What a quantizer may know about its layer; statistics are computed when first read.

    Standalone use: ``Ctx(H=...)`` or ``Ctx(X=...)``.  An engine passes ``provider``, which
    is asked for a statistic the first time a quantizer reads it.
    """

    def __init__(self, name: str = "", module: nn.Module | None = None, block: nn.Module | None = None,
                 block_idx: int = 0, *, H: Tensor | None = None, X: Tensor | None = None,
                 stats: Mapping[str, Tensor] | None = None, provider: StatisticProvider | None = None,
                 cache: dict[str, Any] | None = None, siblings: tuple[str, ...] = (), seed: int = 0,
                 device: str | torch.device | None = None) -> None:
        self.name, self.module, self.block, self.block_idx = name, module, block, block_idx
        self.siblings = siblings
        self.cache = {} if cache is None else cache
        self._stats: dict[str, Tensor] = dict(stats or {})
        if H is not None:
            self._stats["H"] = H
        if X is not None:
            self._stats["X"] = X
        self._provider = provider
        self._seed = seed
        if device is None:
            device = H.device if H is not None else X.device if X is not None else "cpu"
        self._device = torch.device(device)
        self.rng = torch.Generator(device=self._device).manual_seed(layer_seed(name, seed))
        self._additional_bits = 0.0

    def stat(self, name: str, fn: Callable[[Tensor], Tensor] | None = None, reduce: str = "mean") -> Tensor:
        if reduce not in {"mean", "max", "sum", "sample"}:
            raise ValueError("stat reduction must be mean, max, sum, or sample")
        if name not in self._stats:
            if self._provider is not None:
                self._stats[name] = self._provider(name, fn, reduce)
            elif "X" in self._stats:
                derive = _DERIVED_FROM_INPUTS.get(name, fn)
                if derive is None:
                    raise KeyError(f"no statistic implementation for {name!r}")
                self._stats[name] = derive(self._stats["X"].float())
            else:
                raise RuntimeError(
                    f"layer {self.name!r} needs calibration statistic {name!r}; "
                    "supply calibration data to quantize, or construct Ctx(X=...) / Ctx(H=...)")
        return self._stats[name].to(self._device)

    H = property(lambda self: self.stat("H"))
    X = property(lambda self: self.stat("X", reduce="sample"))
    act_absmean = property(lambda self: self.stat("act_absmean"))
    act_absmax = property(lambda self: self.stat("act_absmax", reduce="max"))

    def add_bits(self, bits: int | float) -> None:
        if bits < 0:
            raise ValueError("additional bits must be nonnegative")
        self._additional_bits += bits

    @property
    def additional_bits(self) -> float:
        return self._additional_bits

    def replace(self, **overrides: Any) -> "Ctx":
        clone = Ctx(self.name, self.module, self.block, self.block_idx, stats=self._stats,
                    provider=self._provider, cache=self.cache, siblings=self.siblings, seed=self._seed,
                    device=self._device)
        for key, value in overrides.items():
            if key in {"H", "X", "act_absmean", "act_absmax"}:
                clone._stats[key] = value
            else:
                setattr(clone, key, value)
        return clone

    def derive(self, provider: StatisticProvider, **overrides: Any) -> "Ctx":
        """A context for transformed weights: statistics come from ``provider``, lazily."""
        clone = self.replace(**overrides)
        clone._stats = {}
        clone._provider = provider
        return clone


@dataclasses.dataclass
class ScalarRounding:
    """Fitted state of a scaled scalar grid: all a fused rounding kernel needs.

    ``bits`` is the cost of the whole fitted region, scales included.
    """

    grid: Any
    scales: Tensor
    zero: Tensor | None
    group: int
    values: Tensor
    bits: float
    metadata: dict[str, Any]


@dataclasses.dataclass
class VectorRounding:
    """Fitted state of a scaled vector grid.  ``codebook`` holds the reconstruction of every
    code; ``lattice`` marks the E8P table, in which the 256 magnitude patterns follow the
    ``codebook_size`` points.  ``bits`` is the cost of the whole fitted region, scales included."""

    grid: Any
    scales: Tensor
    group: int
    codebook: Tensor
    codebook_size: int
    lattice: bool
    bits: float
    metadata: dict[str, Any]


class FittedRounder:
    """``round(values, columns) -> Q`` for a fitted format, plus the fitted state a rounding
    kernel needs when the format is a scaled scalar or vector grid."""

    def __init__(self, function: Callable[[Tensor, slice], Q], *, scalar: ScalarRounding | None = None,
                 vector: VectorRounding | None = None) -> None:
        self.function = function
        self.scalar = scalar
        self.vector = vector

    @property
    def scalar_grid(self) -> Any:
        return None if self.scalar is None else self.scalar.grid

    def __call__(self, values: Tensor, columns: slice) -> Q:
        return self.function(values, columns)

    def with_metadata(self, **metadata: Any) -> "FittedRounder":
        def tagged(values: Tensor, columns: slice) -> Q:
            result = self(values, columns)
            result.metadata.update(metadata)
            return result

        scalar, vector = self.scalar, self.vector
        if scalar is not None:
            scalar = dataclasses.replace(scalar, metadata={**scalar.metadata, **metadata})
        if vector is not None:
            vector = dataclasses.replace(vector, metadata={**vector.metadata, **metadata})
        return FittedRounder(tagged, scalar=scalar, vector=vector)


class Quantizer:
    """A quantizer that can be fitted once and then round narrow column slices.

    ``row_separable``: rounding a matrix equals rounding its rows separately with
    row-independent side information, so wide layers may be converted in row chunks.
    """

    row_separable = False

    def fit(self, w: Tensor, ctx: Ctx) -> Callable[[Tensor, slice], Q]:
        raise NotImplementedError

    def __call__(self, w: Tensor, ctx: Ctx | None = None) -> Q:
        ctx = ctx or Ctx(device=w.device)
        return as_q(self.fit(w, ctx)(w, slice(None)))

    def __repr__(self) -> str:
        # Reports and checkpoints record this text: only values with a stable description.
        from mlkit_amd.quantization.grids import Grid

        stable = (bool, int, float, str, type(None), Quantizer, Grid)
        shown = ", ".join(f"{key}={value!r}" for key, value in vars(self).items()
                          if not key.startswith("_") and isinstance(value, stable))
        return f"{type(self).__name__}({shown})"


class FunctionQuantizer(Quantizer):
    """A plain function ``f(w, ctx, **parameters)`` as a quantizer; calling it with keyword
    arguments only binds parameters and returns a new quantizer."""

    __name__: str

    def __init__(self, function: Callable[..., "Q | Tensor"], parameters: dict[str, Any]) -> None:
        functools.update_wrapper(self, function)
        self.function = function
        self.parameters = parameters
        self.signature = inspect.signature(function)

    def __call__(self, *args: Any, **kwargs: Any) -> Any:
        binding_only = not args and "w" not in kwargs and "ctx" not in kwargs
        merged = {**self.parameters, **kwargs}
        if binding_only:
            self.signature.bind_partial(None, None, **merged)
            return FunctionQuantizer(self.function, merged)
        return as_q(self.function(*args, **merged))

    def fit(self, w: Tensor, ctx: Ctx) -> Callable[[Tensor, slice], Q]:
        def round_columns(value: Tensor, columns: slice) -> Q:
            try:
                return self(value, ctx)
            except (ValueError, RuntimeError) as error:
                raise ValueError(
                    f"{self.__name__} cannot round a narrow slice {tuple(value.shape)}; "
                    "use mk.scaled or implement Quantizer.fit(w, ctx) with round(x, cols)") from error

        return round_columns

    def __repr__(self) -> str:
        shown = ", ".join(f"{key}={value!r}" for key, value in self.parameters.items())
        return f"{self.__name__}({shown})"


def quantizer(function: Callable[..., "Q | Tensor"]) -> FunctionQuantizer:
    return FunctionQuantizer(function, {})


def fit_quantizer(quantization: Callable[..., "Q | Tensor"], w: Tensor, ctx: Ctx) -> Callable[[Tensor, slice], Q]:
    if isinstance(quantization, Quantizer):
        return quantization.fit(w, ctx)
    return FunctionQuantizer(quantization, {}).fit(w, ctx)
