"""What a quantizer qualifies for: fused kernels, checkpoint form, packed execution.

Same fields and report strings as the reference's capability report
(/root/reference/src/mlkit/evaluation/capability_report.py:24-133: ``Capabilities``,
``capabilities``, ``error_feedback_path``, ``packed_inference_path``,
``online_activation_path``), for the scalar formats this package implements.  Each of the
three "path" questions is answered by walking a short list of (condition, answer) rules, the
first that applies wins; ``capabilities`` rounds a seeded random matrix once and asks them.
"""

from dataclasses import dataclass, fields
from typing import Any

import torch
from torch import Tensor

from mlkit_amd.inference.packed_linear import packed_compatible
from mlkit_amd.kernels.packed_linear import layout_for
from mlkit_amd.quantization.codecs import registered
from mlkit_amd.quantization.core import Ctx, FittedRounder, FunctionQuantizer, Q, Quantizer, as_q
from mlkit_amd.quantization.feedback import FUSED_CODEBOOK_LIMIT, FUSED_VECTOR_CODEBOOK_LIMIT, FUSED_VECTOR_DIMENSIONS
from mlkit_amd.quantization.scaled import SCALE_FORMAT_BITS, Scaled

FUSED = "fused kernel"


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
        rows = []
        for field in fields(self):
            value = getattr(self, field.name)
            text = "unknown" if value is None else (f"{value:.4f}" if isinstance(value, float) else str(value))
            rows.append((field.name.replace("_", " "), text))
        width = max(len(label) for label, _ in rows)
        return "\n".join(f"{label:<{width}}  {text}" for label, text in rows)


def _fitted_state(quantization: Quantizer, weight: Tensor):
    """The scalar and vector rounding states the quantizer fits on ``weight`` (None where it fits none)."""
    with torch.no_grad():
        fitted = quantization.fit(weight, Ctx("capabilities", X=weight.new_zeros((1, weight.shape[1]))))
    return (fitted.scalar, fitted.vector) if isinstance(fitted, FittedRounder) else (None, None)


def error_feedback_path(quantization: Any, weight: Tensor) -> str:
    plain_function = isinstance(quantization, FunctionQuantizer) or not isinstance(quantization, Quantizer)
    if plain_function:
        return "reference rounding; the function is called on every column block"
    if type(quantization).fit is Quantizer.fit:
        return "not an inner format; it does not implement Quantizer.fit"
    scalar, vector = _fitted_state(quantization, weight)
    if scalar is not None and scalar.grid.bits <= 8 and scalar.values.numel() <= FUSED_CODEBOOK_LIMIT:
        return "fused scalar kernel at step=1"
    if (vector is not None and vector.grid.dim in FUSED_VECTOR_DIMENSIONS
            and vector.codebook_size <= FUSED_VECTOR_CODEBOOK_LIMIT):
        return f"fused vector kernel at step={vector.grid.dim}"
    return "reference rounding with the fitted rounder"


def packed_inference_path(result: Q, input_width: int) -> str:
    scalar_codes = registered(result.codec) and result.codec in ("scaled", "feedback") and packed_compatible(result)
    if not scalar_codes:
        return "no; dense weights"
    whole_words = layout_for(result.metadata["code_bits"], input_width, result.params["group"]) is not None
    return FUSED if whole_words else "packed storage with dense execution; rows or groups split a packing word"


def online_activation_path(quantization: Any) -> str:
    if not isinstance(quantization, Scaled):
        return "reference rounding; not restorable from a checkpoint"
    requirements = (
        quantization.grid.dim == 1,
        quantization.grid.values is not None,
        quantization.scale == "absmax",
        isinstance(quantization.scale_fmt, str) and quantization.scale_fmt in SCALE_FORMAT_BITS,
    )
    return FUSED if all(requirements) else "reference rounding"


def capabilities(quantization: Any, shape: tuple[int, int] = (64, 256), *, device: str = "cuda") -> Capabilities:
    """Round a seeded random matrix with ``quantization`` and report what it qualifies for.

    The bit cost includes side information and therefore depends on ``shape``.
    """
    rows, width = shape
    generator = torch.Generator(device=device).manual_seed(0)
    weight = torch.randn((rows, width), device=device, generator=generator)
    context = Ctx("capabilities", X=torch.randn((4 * width, width), device=device, generator=generator))
    with torch.no_grad():
        result = as_q(quantization(weight, context))
        reconstruction = result.w
    if reconstruction.shape != weight.shape or not bool(torch.isfinite(reconstruction).all()):
        raise ValueError("the quantizer returned an invalid reconstruction")
    total_bits = None if result.bits is None else result.bits + context.additional_bits
    stored_as_codes = result.codes is not None and registered(result.codec)
    return Capabilities(
        quantizer=repr(quantization),
        bits_per_weight=None if total_bits is None else total_bits / weight.numel(),
        codec=result.codec,
        checkpoint="codes with a registered codec" if stored_as_codes else "dense reconstruction",
        error_feedback=error_feedback_path(quantization, weight),
        packed_inference=packed_inference_path(result, width),
        online_activations=online_activation_path(quantization),
    )
