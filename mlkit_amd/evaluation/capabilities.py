"""What a quantizer qualifies for: fused kernels, checkpoint form, packed execution.

Mirrors /root/reference/src/mlkit/evaluation/capability_report.py:24-133 (``Capabilities``,
``capabilities``, ``error_feedback_path``, ``packed_inference_path``,
``online_activation_path``) with the same field names and the same report strings for the
scalar formats this package implements.
"""

from dataclasses import dataclass, fields
from typing import Any

import torch
from torch import Tensor

from mlkit_amd.inference.packed_linear import packed_compatible
from mlkit_amd.kernels.packed_linear import layout_for
from mlkit_amd.quantization.codecs import registered
from mlkit_amd.quantization.core import Ctx, FittedRounder, FunctionQuantizer, Q, Quantizer, as_q
from mlkit_amd.quantization.feedback import FUSED_CODEBOOK_LIMIT
from mlkit_amd.quantization.scaled import SCALE_FORMAT_BITS, Scaled


def _shown(value: Any) -> str:
    if value is None:
        return "unknown"
    return f"{value:.4f}" if isinstance(value, float) else str(value)


@dataclass
class Capabilities:
    """``checkpoint``: codes or dense reconstruction; ``error_feedback``: how gptq / ldlq round
    with this inner format; ``packed_inference``: whether ``optimize`` executes the codes
    without reconstructing the weight."""

    quantizer: str
    bits_per_weight: float | None
    codec: str | None
    checkpoint: str
    error_feedback: str
    packed_inference: str
    online_activations: str

    def __str__(self) -> str:
        labels = [field.name.replace("_", " ") for field in fields(self)]
        pad = max(map(len, labels))
        return "\n".join(f"{label.ljust(pad)}  {_shown(getattr(self, field.name))}"
                         for label, field in zip(labels, fields(self), strict=True))


def error_feedback_path(quantization: Any, weight: Tensor) -> str:
    if isinstance(quantization, FunctionQuantizer) or not isinstance(quantization, Quantizer):
        return "reference rounding; the function is called on every column block"
    if type(quantization).fit is Quantizer.fit:
        return "not an inner format; it does not implement Quantizer.fit"
    context = Ctx("capabilities", X=weight.new_zeros((1, weight.shape[1])))
    with torch.no_grad():
        rounder = quantization.fit(weight, context)
    scalar = rounder.scalar if isinstance(rounder, FittedRounder) else None
    if scalar is not None and scalar.grid.bits <= 8 and scalar.values.numel() <= FUSED_CODEBOOK_LIMIT:
        return "fused scalar kernel at step=1"
    return "reference rounding with the fitted rounder"


def packed_inference_path(result: Q, input_width: int) -> str:
    if not registered(result.codec) or result.codec not in {"scaled", "feedback"} or not packed_compatible(result):
        return "no; dense weights"
    if layout_for(result.metadata["code_bits"], input_width, result.params["group"]) is None:
        return "packed storage with dense execution; rows or groups split a packing word"
    return "fused kernel"


def online_activation_path(quantization: Any) -> str:
    if not isinstance(quantization, Scaled):
        return "reference rounding; not restorable from a checkpoint"
    fused = (quantization.grid.dim == 1 and quantization.grid.values is not None and quantization.scale == "absmax"
             and isinstance(quantization.scale_fmt, str) and quantization.scale_fmt in SCALE_FORMAT_BITS)
    return "fused kernel" if fused else "reference rounding"


def capabilities(quantization: Any, shape: tuple[int, int] = (64, 256), *, device: str = "cuda") -> Capabilities:
    """Round a seeded random matrix with ``quantization`` and report what it qualifies for.

    The bit cost includes side information and therefore depends on ``shape``.
    """
    generator = torch.Generator(device=device).manual_seed(0)
    weight = torch.randn(shape, device=device, generator=generator)
    inputs = torch.randn((4 * shape[1], shape[1]), device=device, generator=generator)
    context = Ctx("capabilities", X=inputs)
    with torch.no_grad():
        result = as_q(quantization(weight, context))
        restored = result.w
    if restored.shape != weight.shape or not bool(torch.isfinite(restored).all()):
        raise ValueError("the quantizer returned an invalid reconstruction")
    bits = None if result.bits is None else result.bits + context.additional_bits
    portable = result.codes is not None and registered(result.codec)
    return Capabilities(
        quantizer=repr(quantization),
        bits_per_weight=None if bits is None else bits / weight.numel(),
        codec=result.codec,
        checkpoint="codes with a registered codec" if portable else "dense reconstruction",
        error_feedback=error_feedback_path(quantization, weight),
        packed_inference=packed_inference_path(result, shape[1]),
        online_activations=online_activation_path(quantization),
    )
