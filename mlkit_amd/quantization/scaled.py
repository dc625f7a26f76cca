"""Grouped scaling of scalar and vector grids: ``scaled``, ``int``, ``nf4``, ``mxfp4`` and
``store_scale``.

Mirrors, in /root/reference/src/mlkit/quantization/formats:
  scale_storage.py:11-26        SCALE_FORMAT_BITS, store_scale
  grouped_scaling.py:24-51      single_precision_reciprocal, group_extrema, nearest_codes
  grouped_scaling.py:54-414     Scaled (fit / logical_bits / repr), scaled
  standard.py:10-23             int, nf4, mxfp4
Weights on a HIP device are fitted, searched and encoded by the kernels of
``mlkit_amd.kernels.scalar_encode`` (one launch each); host tensors go through the same
arithmetic in tensor operations.  Vector grids (``grid.vector``, ``grid.e8p``) take their
scales from the same fit kernel and their codes from ``mk_vector_nearest``.
"""

import builtins
from collections.abc import Callable
from typing import Any

import torch
import torch.nn.functional as functional
from torch import Tensor

from mlkit_amd.quantization.codecs import decode_scaled, decode_vector_scaled
from mlkit_amd.quantization.core import Ctx, FittedRounder, Q, Quantizer, ScalarRounding, VectorRounding
from mlkit_amd.quantization.grids import NF4_VALUES, Grid, grid
from mlkit_amd.quantization.search import nearest, nearest_indices

SCALE_FORMAT_BITS = {"fp32": 32, "fp16": 16, "bf16": 16, "fp8": 8, "e8m0": 8}
FUSED_CODEBOOK_LIMIT = 256


def _e4m3(value: Tensor) -> Tensor:
    """Positive FP32 -> nearest FP8 E4M3 value, ties to even, by rounding to the quantum
    2^(max(e, -6) - 3) (direct, not through FP16)."""
    clamped = value.clamp(2.0**-9, 448.0)
    exponent = ((clamped.view(torch.int32) >> 23) & 255) - 127
    quantum = torch.ldexp(torch.ones_like(clamped), exponent.clamp_min(-6) - 3)
    return (clamped / quantum).round() * quantum


def _e8m0(value: Tensor) -> Tensor:
    """2^round(log2 v) with the rounding decided exactly (mantissa^2 against 2)."""
    clamped = value.clamp_min(2.0**-127).double()
    mantissa, exponent = torch.frexp(clamped)  # mantissa in [0.5, 1)
    exponent = exponent - 1 + (mantissa * mantissa > 0.5).to(exponent.dtype)
    return torch.ldexp(torch.ones_like(clamped), exponent.clamp(-127, 127)).float()


def store_scale(value: Tensor, format: "str | Grid") -> tuple[Tensor, int]:
    """``value`` rounded to its storage format (kept as FP32) and the bits one entry costs."""
    if isinstance(format, Grid):
        if format.dim != 1:
            raise ValueError("scale grids must be scalar")
        return format(value).clamp_min(torch.finfo(torch.float32).tiny), format.bits
    if format == "fp32":
        return value.float(), 32
    if format == "fp16":
        return value.clamp(2**-24, 65504).half().float(), 16
    if format == "bf16":
        return value.bfloat16().float(), 16
    if format == "fp8":
        return _e4m3(value.float()), 8
    if format == "e8m0":
        return _e8m0(value.float()), 8
    raise ValueError(f"unsupported scale storage format {format!r}")


def single_precision_reciprocal(value: float) -> float:
    """FP32(1) / FP32(value): the constant host code and kernels both multiply by."""
    return float(torch.tensor(1.0) / torch.tensor(value, dtype=torch.float32))


def group_extrema(weight: Tensor, group: int) -> tuple[Tensor, Tensor]:
    """Minimum and maximum of every row group; a narrower last group stands alone."""
    rows, width = weight.shape
    whole = width - width % group
    low, high = [], []
    if whole:
        blocks = weight[:, :whole].reshape(rows, -1, group)
        low.append(blocks.amin(-1))
        high.append(blocks.amax(-1))
    if whole < width:
        low.append(weight[:, whole:].amin(-1, keepdim=True))
        high.append(weight[:, whole:].amax(-1, keepdim=True))
    return torch.cat(low, 1), torch.cat(high, 1)


def nearest_codes(normalized: Tensor, values: Tensor) -> Tensor:
    return nearest_indices(normalized, values)


class Scaled(Quantizer):
    """A grid applied to row groups that each carry a scale and, for scalar grids, optionally
    an offset."""

    row_separable = True

    def __init__(self, grid: Grid, group: int | None = 128,
                 scale: "str | Callable[[Tensor], Tensor]" = "absmax", scale_fmt: "str | Grid" = "fp16",
                 asym: bool = False, *, search_steps: int = 20) -> None:
        if group is not None and group <= 0:
            raise ValueError("group must be positive or None")
        if not callable(scale) and scale not in {"absmax", "mse"}:
            raise ValueError("scale must be absmax, mse, or callable")
        if search_steps < 1:
            raise ValueError("search_steps must be positive")
        if asym and (grid.dim != 1 or grid.values is None):
            raise ValueError("asymmetric quantization requires an explicit scalar grid")
        if asym and (scale_fmt == "e8m0" or isinstance(scale_fmt, Grid)):
            raise ValueError("asymmetric offsets require a signed floating-point storage format")
        self.grid, self.group, self.scale, self.scale_fmt = grid, group, scale, scale_fmt
        self.asym, self.search_steps = asym, search_steps
        self._on_device: dict[torch.device, Tensor] = {}
        table = None if grid.values is None or grid.dim != 1 else grid.values.detach().cpu()
        self._value_minimum = 0.0 if table is None else float(table.min())
        self._value_maximum = 0.0 if table is None else float(table.max())
        span = self._value_maximum - self._value_minimum
        if asym and span <= 0:
            raise ValueError("asymmetric quantization requires at least two distinct grid values")
        self._magnitude_reciprocal = single_precision_reciprocal(
            1.0 if grid.values is None else float(grid.values.abs().max()))
        self._range_reciprocal = single_precision_reciprocal(span) if asym else 1.0

    # -- description ---------------------------------------------------------------------

    def values_on(self, device: torch.device) -> Tensor:
        table = self._on_device.get(device)
        if table is None:
            assert self.grid.values is not None
            table = self._on_device[device] = self.grid.values.to(device).contiguous()
        return table

    def reconstruct_activations(self, value: Tensor) -> Tensor:
        """Quantize-dequantize a two-dimensional activation tensor online (no codec state kept):
        one fused kernel on a HIP device, the rounder itself otherwise."""
        fused = (value.is_cuda and value.dim() == 2 and value.dtype in (torch.float32, torch.float16, torch.bfloat16)
                 and self.grid.dim == 1 and self.grid.values is not None and self.scale == "absmax"
                 and isinstance(self.scale_fmt, str) and self.scale_fmt in SCALE_FORMAT_BITS
                 and self.grid.values.numel() <= FUSED_CODEBOOK_LIMIT and self.grid.bits <= 8)
        if not fused:
            return self(value.float()).w.to(value.dtype)
        from mlkit_amd.kernels import scalar_encode

        assert isinstance(self.scale_fmt, str)
        return scalar_encode.reconstruct(
            value.contiguous(), self.values_on(value.device), self.group or value.shape[1], self.scale_fmt,
            self.asym, self.grid.integer, self._value_minimum, self._value_maximum,
            self._range_reciprocal if self.asym else self._magnitude_reciprocal)

    def logical_bits(self, shape: tuple[int, int]) -> float:
        rows, width = shape
        group = min(self.group or width, width)
        per_scale = self.scale_fmt.bits if isinstance(self.scale_fmt, Grid) else SCALE_FORMAT_BITS[self.scale_fmt]
        groups = rows * (-(-width // group))
        return self.grid.bits * rows * width / self.grid.dim + per_scale * groups * (2 if self.asym else 1)

    def __repr__(self) -> str:
        rule = self.scale if isinstance(self.scale, str) else getattr(self.scale, "__name__", type(self.scale).__name__)
        text = f"scaled({self.grid!r}, group={self.group}, scale={rule!r}"
        if self.scale_fmt != "fp16":
            text += f", scale_fmt={self.scale_fmt!r}"
        return text + (", asym=True)" if self.asym else ")")

    # -- fitting -------------------------------------------------------------------------

    def _kernel_path(self, weight: Tensor, table: Tensor | None) -> bool:
        """Whether the scales of ``weight`` can come from the fit / search kernels: scalar tables
        of up to 256 values, and vector grids whose scales follow the range (no search)."""
        if not (weight.is_cuda and isinstance(self.scale_fmt, str) and not callable(self.scale)):
            return False
        if self.grid.dim > 1:
            return self.grid.values is not None and self.scale == "absmax"
        return table is not None and table.numel() <= FUSED_CODEBOOK_LIMIT

    def _initial_scales(self, weight: Tensor, group: int) -> tuple[Tensor, Tensor | None]:
        rows, width = weight.shape
        if callable(self.scale) and not self.asym:
            if not bool(torch.isfinite(weight).all()):
                raise ValueError("scaled requires a finite floating-point weight matrix")
            blocks = functional.pad(weight, (0, -width % group)).reshape(-1, group)
            return self.scale(blocks).reshape(rows, -1), None
        low, high = group_extrema(weight, group)
        if not bool(torch.isfinite(low).all() and torch.isfinite(high).all()):
            raise ValueError("scaled requires a finite floating-point weight matrix")
        if self.asym:
            scales = (high - low).clamp_min(1e-12) * self._range_reciprocal
            return scales, low - self._value_minimum * scales
        return torch.maximum(high, -low).clamp_min(1e-12) * self._magnitude_reciprocal, None

    def _search_on_host(self, weight: Tensor, scales: Tensor, zero: Tensor | None, group: int) -> Tensor:
        rows, width = weight.shape
        blocks = functional.pad(weight, (0, -width % group)).reshape(rows, -1, group)
        occupied = (torch.arange(blocks.shape[1] * group, device=weight.device) < width).reshape(1, -1, group)
        centered = blocks if zero is None else blocks - zero[..., None]

        def error_of(candidate: Tensor) -> Tensor:
            normalized = centered / candidate[..., None]
            if self.grid.dim > 1:
                blocks_of = normalized.reshape(*normalized.shape[:-1], -1, self.grid.dim)
                rounded = self.grid(blocks_of).reshape_as(centered)
            else:
                rounded = self.grid(normalized)
            return ((rounded * candidate[..., None] - centered).square() * occupied).sum(-1)

        chosen, best = scales.clone(), error_of(scales)
        for fraction in torch.linspace(0.5, 1.0, self.search_steps).tolist():
            candidate, _ = store_scale(scales * fraction, self.scale_fmt)
            error = error_of(candidate)
            chosen = torch.where(error < best, candidate, chosen)
            best = torch.minimum(best, error)
        return chosen

    def fit(self, w: Tensor, ctx: Ctx) -> FittedRounder:
        if w.ndim != 2 or not w.is_floating_point():
            raise ValueError("scaled requires a finite floating-point weight matrix")
        rows, width = w.shape
        group = width if self.group is None else min(self.group, width)
        dimension, codebook = self.grid.dim, self.grid.values
        if group % dimension:
            raise ValueError("group width must be divisible by the vector grid dimension")
        lattice = self.grid.name == "e8p"
        if dimension > 1 and codebook is not None and not lattice:
            counted = ctx.cache.setdefault("_mlkit_vector_codebooks", set())
            if id(self.grid) not in counted:  # the codebook is side information, paid for once
                ctx.add_bits(codebook.numel() * codebook.element_size() * 8)
                counted.add(id(self.grid))
        weight = w.float()
        table = None if codebook is None or dimension != 1 else self.values_on(w.device)
        on_kernels = self._kernel_path(weight, table)
        if on_kernels:
            from mlkit_amd.kernels import scalar_encode

            assert isinstance(self.scale_fmt, str)
            weight = weight.contiguous()
            searching = self.scale == "mse"
            scales, zero = scalar_encode.fit_scales(
                weight, group, asym=self.asym,
                reciprocal=self._range_reciprocal if self.asym else self._magnitude_reciprocal,
                value_minimum=self._value_minimum, scale_format=self.scale_fmt, store_zero=not searching)
            if not bool(torch.isfinite(scales).all()):
                raise ValueError("scaled requires a finite floating-point weight matrix")
            scale_bits = SCALE_FORMAT_BITS[self.scale_fmt]
            if searching:
                assert table is not None
                fractions = torch.linspace(0.5, 1.0, self.search_steps, device=w.device)
                scales = scalar_encode.search_scales(
                    weight, scales, zero, table, fractions, group, None, self.scale_fmt,
                    integer=self.grid.integer, minimum=self._value_minimum, maximum=self._value_maximum)
                if zero is not None:
                    zero = store_scale(zero.abs().clamp_min(1e-12), self.scale_fmt)[0] * zero.sign()
        else:
            scales, zero = self._initial_scales(weight, group)
            scales, scale_bits = store_scale(scales, self.scale_fmt)
            if self.scale == "mse":
                scales = self._search_on_host(weight, scales, zero, group)
            if zero is not None:
                zero = store_scale(zero.abs().clamp_min(1e-12), self.scale_fmt)[0] * zero.sign()
        side_bits = scales.numel() * scale_bits * (2 if zero is not None else 1)
        metadata = {"code_bits": self.grid.bits, "scale_fmt": self.scale_fmt,
                    "trainable": ["scales"] + (["zero"] if zero is not None else [])}
        scalar = None
        if table is not None:
            scalar = ScalarRounding(grid=self.grid, scales=scales, zero=zero, group=group, values=table,
                                    bits=self.grid.bits * w.numel() + side_bits, metadata=metadata)

        vector = None
        vector_metadata = {"code_bits": self.grid.bits, "scale_fmt": self.scale_fmt, "trainable": ["scales"]}
        if dimension > 1 and codebook is not None and w.is_cuda:
            from mlkit_amd.quantization.lattice import device_table

            vector = VectorRounding(grid=self.grid, scales=scales, group=group,
                                    codebook=device_table(w.device) if lattice else self.values_on(w.device),
                                    codebook_size=codebook.shape[0], lattice=lattice,
                                    bits=self.grid.bits * w.numel() / dimension + side_bits,
                                    metadata=vector_metadata)

        def round_columns(value: Tensor, columns: slice) -> Q:
            start, stop, stride = columns.indices(width)
            if stride != 1 or stop - start != value.shape[1]:
                raise ValueError("rounder columns must describe a contiguous slice of its fitted region")
            bits = self.grid.bits * value.numel() / dimension + side_bits * value.shape[1] / width
            if scalar is not None:
                codes = self._scalar_codes(value, scalar, start, stop)
                return Q(bits=bits, codes=codes, decode=decode_scaled, codec="scaled", metadata=scalar.metadata,
                         params={"scales": scales, "values": scalar.values, "group": group, "offset": start,
                                 "zero": zero})
            index = torch.arange(start, stop, device=value.device) // group
            centered = value.float() if zero is None else value.float() - zero[:, index]
            normalized = centered / scales[:, index]
            if dimension == 1:
                rounded = self.grid(normalized)
            else:
                if value.shape[1] % dimension:
                    raise ValueError("column slices must align to the vector grid dimension")
                blocks = normalized.reshape(-1, dimension)
                if codebook is not None:
                    if lattice:
                        from mlkit_amd.quantization.lattice import nearest_e8p

                        codes = nearest_e8p(blocks, return_indices=True)
                    else:
                        codes = nearest(blocks, codebook, return_indices=True)
                    return Q(codes=codes.reshape(value.shape[0], -1).to(torch.int32), bits=bits,
                             decode=decode_vector_scaled, codec="vector_scaled", metadata=vector_metadata,
                             params={"scales": scales, "values": None if lattice else codebook.to(value.device),
                                     "dim": dimension, "group": group, "offset": start, "zero": zero})
                rounded = self.grid(blocks).reshape_as(value)
            restored = rounded * scales[:, index]
            return Q(restored if zero is None else restored + zero[:, index], bits=bits)

        return FittedRounder(round_columns, scalar=scalar, vector=vector)

    def _scalar_codes(self, value: Tensor, scalar: ScalarRounding, start: int, stop: int) -> Tensor:
        """Codes of the nearest grid values for columns ``start`` to ``stop`` of the fitted region."""
        if (value.is_cuda and start % scalar.group == 0 and self.grid.bits <= 8
                and scalar.values.numel() <= FUSED_CODEBOOK_LIMIT):
            from mlkit_amd.kernels import scalar_encode

            first = start // scalar.group
            count = -(-(stop - start) // scalar.group)
            scales = scalar.scales[:, first:first + count].contiguous()
            zero = None if scalar.zero is None else scalar.zero[:, first:first + count].contiguous()
            return scalar_encode.encode(value.float().contiguous(), scales, zero, scalar.values, scalar.group,
                                        None, integer=self.grid.integer, minimum=self._value_minimum,
                                        maximum=self._value_maximum)
        index = torch.arange(start, stop, device=value.device) // scalar.group
        centered = value.float() if scalar.zero is None else value.float() - scalar.zero[:, index]
        normalized = centered / scalar.scales[:, index]
        if self.grid.integer:
            codes = normalized.round().clamp(self._value_minimum, self._value_maximum) - self._value_minimum
        else:
            codes = nearest_codes(normalized, scalar.values)
        return codes.to(torch.uint8 if self.grid.bits <= 8 else torch.int32)


def scaled(grid: Grid, group: int | None = 128, scale: "str | Callable[[Tensor], Tensor]" = "absmax",
           scale_fmt: "str | Grid" = "fp16", asym: bool = False, **options: Any) -> Scaled:
    return Scaled(grid, group, scale, scale_fmt, asym, **options)


def int(bits: builtins.int = 4, group: builtins.int | None = 128, **options: Any) -> Scaled:  # noqa: A001
    return scaled(grid.int(bits), group=group, **options)


def nf4(group: builtins.int | None = 64, **options: Any) -> Scaled:
    return scaled(grid.values(NF4_VALUES, bits=4, name="nf4"), group=group, **options)


def mxfp4(group: builtins.int = 32, **options: Any) -> Scaled:
    return scaled(grid.fp("e2m1"), group=group, scale_fmt="e8m0", **options)
