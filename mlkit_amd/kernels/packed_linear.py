"""Fused decode + matrix-vector product of packed scalar codes, and packed -> dense decode.

Same call surface as the reference's ``kernels/packed_linear.py`` (``PackedLayout``,
``layout_for``, ``matrix_vector``, ``decode``; /root/reference/src/mlkit/kernels/
packed_linear.py:43-79,181-226,279-313); the launches go to ``mk_packed_matvec`` and
``mk_packed_decode`` of ``libmlkit_amd.so`` on the current HIP stream.
"""

import math
from dataclasses import dataclass

import torch
from torch import Tensor

from mlkit_amd import native

ROW_TILE = 8
MAXIMUM_TILE_CODES = 128
MINIMUM_TILE_CODES = 16
MAXIMUM_SAMPLE_TILE = 8
MAXIMUM_CODE_BITS = 8


@dataclass(frozen=True)
class PackedLayout:
    """Word structure of a packed stream: ``codes_per_word`` codes in ``bytes_per_word`` bytes.

    ``tile_words`` is the reference's kernel tile (largest power-of-two count of words
    inside a scale group, at most 128 codes); the HIP kernels choose their own tiling and
    keep the field for API parity and for the "fused or not" decision.
    """

    bits: int
    bytes_per_word: int
    codes_per_word: int
    tile_words: int

    @property
    def tile_codes(self) -> int:
        return self.codes_per_word * self.tile_words

    def row_bytes(self, input_width: int) -> int:
        return (input_width // self.codes_per_word) * self.bytes_per_word

    def tiles_per_row(self, input_width: int) -> int:
        return -(-input_width // self.tile_codes)


def layout_for(bits: int, input_width: int, group: int) -> PackedLayout | None:
    """The layout of a layer, or ``None`` when a row or a scale group splits a packing word."""
    if bits < 1 or bits > MAXIMUM_CODE_BITS:
        return None
    common = math.gcd(bits, 8)
    codes_per_word = 8 // common
    if input_width % codes_per_word or group % codes_per_word:
        return None
    words_per_group = group // codes_per_word
    tile_words = min(MAXIMUM_TILE_CODES // codes_per_word, words_per_group & -words_per_group)
    if tile_words * codes_per_word < MINIMUM_TILE_CODES:
        return None
    return PackedLayout(bits, bits // common, codes_per_word, tile_words)


def sample_tile_for(samples: int) -> int:
    """Input rows one workgroup multiplies against each decoded weight (a power of two up to 8)."""
    tile = 1
    while tile < samples and tile < MAXIMUM_SAMPLE_TILE:
        tile *= 2
    return tile


def matrix_vector(
    inputs: Tensor,
    packed: Tensor,
    scales: Tensor,
    values: Tensor,
    zeros: Tensor | None,
    bias: Tensor | None,
    output: Tensor,
    group: int,
    layout: PackedLayout,
    *,
    uniform_grid: bool = False,
    grid_minimum: float = 0.0,
    grid_step: float = 1.0,
) -> None:
    """``output[m, n] = sum_k dequant(code[n, k]) * inputs[m, k] (+ bias[n])`` on the current stream."""
    device = native.require_device(inputs, packed, scales, values, zeros, bias, output)
    samples, input_width = inputs.shape
    output_width = output.shape[-1]
    if not inputs.is_contiguous() or not output.is_contiguous():
        raise ValueError("packed matrix-vector inputs and outputs must be contiguous")
    if output.dtype != inputs.dtype or output.shape[0] != samples:
        raise ValueError("output must have the dtype and row count of the inputs")
    if packed.dtype != torch.uint8 or packed.numel() != output_width * layout.row_bytes(input_width):
        raise ValueError("packed byte count does not match the layer shape and precision")
    if zeros is not None and zeros.dtype != scales.dtype:
        raise ValueError("zeros must have the dtype of scales")
    status = native.library().mk_packed_matvec(
        inputs.data_ptr(), native.dtype_code(inputs), packed.data_ptr(), scales.data_ptr(),
        native.dtype_code(scales), values.data_ptr(), values.numel(), native.pointer(zeros),
        native.pointer(bias), 0 if bias is None else native.dtype_code(bias), output.data_ptr(),
        samples, output_width, input_width, group, layout.bits, int(uniform_grid),
        grid_minimum, grid_step, native.current_stream(device),
    )
    native.check(status)


def decode(
    packed: Tensor,
    scales: Tensor,
    values: Tensor,
    zeros: Tensor | None,
    output: Tensor,
    group: int,
    layout: PackedLayout,
    uniform_grid: bool,
    grid_minimum: float,
    grid_step: float,
) -> None:
    """Reconstruct the dense ``[out_features, in_features]`` weight from word-aligned codes."""
    device = native.require_device(packed, scales, values, zeros, output)
    output_width, input_width = output.shape
    if not output.is_contiguous():
        raise ValueError("decode output must be contiguous")
    if packed.dtype != torch.uint8 or packed.numel() != output_width * layout.row_bytes(input_width):
        raise ValueError("packed byte count does not match the layer shape and precision")
    status = native.library().mk_packed_decode(
        packed.data_ptr(), scales.data_ptr(), native.dtype_code(scales), values.data_ptr(),
        values.numel(), native.pointer(zeros), output.data_ptr(), native.dtype_code(output),
        output_width, input_width, group, layout.bits, int(uniform_grid), grid_minimum, grid_step,
        native.current_stream(device),
    )
    native.check(status)


@torch.library.custom_op("mlkit_amd::packed_matvec", mutates_args=())
def packed_matvec_op(
    inputs: Tensor,
    packed: Tensor,
    scales: Tensor,
    values: Tensor,
    zeros: Tensor | None,
    bias: Tensor | None,
    output_width: int,
    group: int,
    bits: int,
    uniform_grid: bool,
    grid_minimum: float,
    grid_step: float,
) -> Tensor:
    """The fused matvec as a traceable operator: what a compiled graph holds in place of the
    ``ctypes`` call (the reference lets the compiler capture its Triton launch instead,
    inference/packed_linear.py:161-176).  It only enqueues on the current stream, so
    ``mode="reduce-overhead"`` can capture it into a HIP graph."""
    device = native.require_device(inputs, packed, scales, values, zeros, bias)
    output = inputs.new_empty((inputs.shape[0], output_width))
    status = native.library().mk_packed_matvec(
        inputs.data_ptr(), native.dtype_code(inputs), packed.data_ptr(), scales.data_ptr(),
        native.dtype_code(scales), values.data_ptr(), values.numel(), native.pointer(zeros),
        native.pointer(bias), 0 if bias is None else native.dtype_code(bias), output.data_ptr(),
        inputs.shape[0], output_width, inputs.shape[1], group, bits, int(uniform_grid), grid_minimum, grid_step,
        native.current_stream(device),
    )
    native.check(status)
    return output


@packed_matvec_op.register_fake
def _packed_matvec_shape(inputs, packed, scales, values, zeros, bias, output_width, group, bits, uniform_grid,
                         grid_minimum, grid_step):
    return inputs.new_empty((inputs.shape[0], output_width))
