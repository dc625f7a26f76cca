"""Incoherence processing: an inner quantizer applied in a randomly rotated basis.

Mirrors /root/reference/src/mlkit/quantization/algorithms/incoherence.py:15-98 (``Incoherent``,
``incoherent``): rows and columns are multiplied by hash-derived signs and rotated with the
structured transform before the inner quantizer sees them; calibration statistics are
rotated the same way; a portable inner representation is wrapped in the ``"basis"`` codec,
which rotates the reconstruction back on decode.  On a HIP device every rotation is one or
two kernel launches with the sign flips fused.
"""

from collections.abc import Callable
from typing import Any

from torch import Tensor

from mlkit_amd.quantization.codecs import compose, deterministic_signs, registered
from mlkit_amd.quantization.core import Ctx, Q, Quantizer, as_q, layer_seed
from mlkit_amd.quantization.transforms import rotate


def _rows(value: Tensor, signs: Tensor, inverse: bool = False) -> Tensor:
    """The transform along the first dimension."""
    return rotate(value.T.contiguous(), inverse=inverse, signs=signs).T


class Incoherent(Quantizer):
    def __init__(self, inner: Callable[..., "Q | Tensor"], *, left: str | None = "rht", right: str | None = "rht",
                 train_signs: bool = False) -> None:
        if left not in {None, "rht"} or right not in {None, "rht"}:
            raise ValueError("incoherence transforms must be rht or None")
        self.inner, self.left, self.right, self.train_signs = inner, left, right, train_signs

    def __repr__(self) -> str:
        return f"incoherent({self.inner!r})"

    def __call__(self, w: Tensor, ctx: Ctx | None = None) -> Q:
        ctx = ctx or Ctx(device=w.device)
        seed = layer_seed(ctx.name, ctx._seed) % 2**32
        left_signs = deterministic_signs(w.shape[0], seed, w.device) if self.left else None
        right_signs = deterministic_signs(w.shape[1], seed + 1, w.device) if self.right else None
        rotated = w.float()
        if left_signs is not None:
            rotated = _rows(rotated, left_signs)
        if right_signs is not None:
            rotated = rotate(rotated.contiguous(), signs=right_signs)
        inner_ctx = ctx.replace()
        if right_signs is not None:
            fallback = ctx._provider

            def rotated_statistic(name: str, fn: Callable | None, reduce: str) -> Tensor:
                if name == "H":
                    hessian = ctx.H.to(w.device) * right_signs[:, None] * right_signs[None, :]
                    return rotate(rotate(hessian.contiguous()).T.contiguous()).T
                inputs = rotate(ctx.X.to(w.device).contiguous(), signs=right_signs)
                if name == "X":
                    return inputs
                if name == "act_absmean":
                    return inputs.abs().mean(0)
                if name == "act_absmax":
                    return inputs.abs().amax(0)
                if fn is not None:
                    return fn(inputs)
                if fallback is not None:
                    return fallback(name, fn, reduce)
                raise KeyError(name)

            inner_ctx = ctx.derive(rotated_statistic)
        quantized = as_q(self.inner(rotated, inner_ctx))
        ctx.add_bits(inner_ctx.additional_bits)
        if quantized.codes is not None and registered(quantized.codec):
            result = compose(quantized, "basis", {
                "shape": tuple(w.shape),
                "left_seed": seed if self.left else None,
                "right_seed": (seed + 1) % 2**32 if self.right else None,
                "left_signs": left_signs if self.train_signs else None,
                "right_signs": right_signs if self.train_signs else None,
            })
            if self.train_signs:
                for key, signs in (("left_signs", left_signs), ("right_signs", right_signs)):
                    if signs is not None:
                        result.metadata["trainable"].append(key)
                        result.metadata["parameter_formats"][key] = "fp16"
                        ctx.add_bits(16 * signs.numel())
            return result
        if self.train_signs:
            raise ValueError("trainable signs require an inner quantizer with a registered codec")
        restored = quantized.w
        if right_signs is not None:
            restored = rotate(restored.contiguous(), inverse=True, signs=right_signs)
        if left_signs is not None:
            restored = _rows(restored, left_signs, inverse=True)
        return Q(restored, bits=quantized.bits)


def incoherent(inner: Callable[..., "Q | Tensor"], **options: Any) -> Incoherent:
    return Incoherent(inner, **options)
