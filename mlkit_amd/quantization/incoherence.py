"""Incoherence processing: an inner quantizer applied in a randomly rotated basis.

Same call surface and results as the reference's ``Incoherent`` / ``incoherent``
(/root/reference/src/mlkit/quantization/algorithms/incoherence.py:15-98): the weight is seen by
the inner quantizer as ``U W V^T`` with ``U``, ``V`` sign-randomised structured transforms of
the output and input side (signs from ``deterministic_signs`` of the layer seed and seed + 1),
calibration statistics move to the same basis, and a portable inner representation comes back
wrapped in the ``"basis"`` codec, which undoes the rotation on decode.

Here the two sides are objects (``_Side``) that know how to move a matrix into their basis and
back along either axis, so the quantizer itself reads as: rotate, describe the statistics in
the new basis, round, wrap or rotate back.  On a HIP device each move is one or two kernel
launches with the sign flips fused.
"""

from collections.abc import Callable
from typing import Any

from torch import Tensor

from mlkit_amd.quantization.codecs import compose, deterministic_signs, registered
from mlkit_amd.quantization.core import Ctx, Q, Quantizer, as_q, layer_seed
from mlkit_amd.quantization.transforms import rotate

SIDE_KINDS = (None, "rht")


class _Side:
    """One sign-randomised structured transform ``T diag(signs)`` of a given width."""

    def __init__(self, width: int, seed: int, device) -> None:
        self.seed = seed
        self.signs = deterministic_signs(width, seed, device)

    def along_columns(self, matrix: Tensor, back: bool = False) -> Tensor:
        """``matrix @ (T diag(signs))^T`` (every row transformed), or its inverse."""
        return rotate(matrix.contiguous(), inverse=back, signs=self.signs)

    def along_rows(self, matrix: Tensor, back: bool = False) -> Tensor:
        """``(T diag(signs)) @ matrix`` (every column transformed), or its inverse."""
        return self.along_columns(matrix.T, back).T

    def conjugate(self, symmetric: Tensor) -> Tensor:
        """``(T S) M (T S)^T`` for a square matrix over this side's width."""
        return self.along_rows(self.along_columns(symmetric))


def _statistics_in(side: _Side, ctx: Ctx, device) -> Callable[[str, Callable | None, str], Tensor]:
    """Calibration statistics as the inner quantizer must see them once the inputs are rotated
    by ``side``: everything is recomputed from the rotated inputs (or conjugated, for H)."""
    upstream = ctx._provider

    def provide(name: str, function: Callable | None, reduce: str) -> Tensor:
        if name == "H":
            return side.conjugate(ctx.H.to(device))
        rotated_inputs = side.along_columns(ctx.X.to(device))
        known = {"X": lambda: rotated_inputs, "act_absmean": lambda: rotated_inputs.abs().mean(0),
                 "act_absmax": lambda: rotated_inputs.abs().amax(0)}
        if name in known:
            return known[name]()
        if function is not None:
            return function(rotated_inputs)
        if upstream is None:
            raise KeyError(name)
        return upstream(name, function, reduce)

    return provide


class Incoherent(Quantizer):
    def __init__(self, inner: Callable[..., "Q | Tensor"], *, left: str | None = "rht", right: str | None = "rht",
                 train_signs: bool = False) -> None:
        if left not in SIDE_KINDS or right not in SIDE_KINDS:
            raise ValueError("incoherence transforms must be rht or None")
        self.inner, self.left, self.right, self.train_signs = inner, left, right, train_signs

    def __repr__(self) -> str:
        return f"incoherent({self.inner!r})"

    def __call__(self, w: Tensor, ctx: Ctx | None = None) -> Q:
        ctx = ctx or Ctx(device=w.device)
        base_seed = layer_seed(ctx.name, ctx._seed) % 2**32
        rows, columns = w.shape
        output_side = _Side(rows, base_seed, w.device) if self.left else None
        input_side = _Side(columns, base_seed + 1, w.device) if self.right else None

        in_basis = w.float()
        if output_side is not None:
            in_basis = output_side.along_rows(in_basis)
        if input_side is not None:
            in_basis = input_side.along_columns(in_basis)
        inner_ctx = ctx.replace() if input_side is None else ctx.derive(_statistics_in(input_side, ctx, w.device))
        rounded = as_q(self.inner(in_basis, inner_ctx))
        ctx.add_bits(inner_ctx.additional_bits)

        portable = rounded.codes is not None and registered(rounded.codec)
        if not portable:
            if self.train_signs:
                raise ValueError("trainable signs require an inner quantizer with a registered codec")
            restored = rounded.w
            if input_side is not None:
                restored = input_side.along_columns(restored, back=True)
            if output_side is not None:
                restored = output_side.along_rows(restored, back=True)
            return Q(restored, bits=rounded.bits)

        kept_signs = {"left_signs": output_side.signs if output_side is not None and self.train_signs else None,
                      "right_signs": input_side.signs if input_side is not None and self.train_signs else None}
        wrapped = compose(rounded, "basis", {
            "shape": (rows, columns),
            "left_seed": None if output_side is None else output_side.seed,
            "right_seed": None if input_side is None else input_side.seed % 2**32,
            **kept_signs,
        })
        for key, signs in kept_signs.items():  # trainable sign vectors are stored, as fp16
            if signs is not None:
                wrapped.metadata["trainable"].append(key)
                wrapped.metadata["parameter_formats"][key] = "fp16"
                ctx.add_bits(16 * signs.numel())
        return wrapped


def incoherent(inner: Callable[..., "Q | Tensor"], **options: Any) -> Incoherent:
    return Incoherent(inner, **options)
