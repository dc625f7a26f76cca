"""Fused decode + matrix-vector product of packed scalar codes, and packed -> dense decode.

Same call surface as the reference's ``kernels/packed_linear.py`` (``PackedLayout``,
``layout_for``, ``matrix_vector``, ``decode``; /root/reference/src/mlkit/kernels/
packed_linear.py:43-79,181-226,279-313); the launches go to ``mk_packed_matvec`` and
``mk_packed_decode`` of ``libmlkit_amd.so`` on the current HIP stream.
"""

import ctypes
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


class GroupLaunch:
    """Bound arguments of ``mk_packed_matvec_group`` for sibling layers that read the same
    activations: the host arrays of device pointers are built once and reused by every call."""

    def __init__(self, packed: list[Tensor], scales: list[Tensor], values: Tensor, zeros: list[Tensor | None],
                 bias: list[Tensor | None], output_widths: list[int], input_width: int, group: int, layout: PackedLayout,
                 *, uniform_grid: bool, grid_minimum: float, grid_step: float) -> None:
        count = len(packed)
        if not 1 <= count <= 8 or not (len(scales) == len(zeros) == len(bias) == len(output_widths) == count):
            raise ValueError("a launch group holds one to eight matrices with one entry per matrix in every list")
        self.device = native.require_device(values, *packed, *scales, *zeros, *bias)
        with_zeros = zeros[0] is not None
        for index in range(count):
            if packed[index].dtype != torch.uint8 or packed[index].numel() != output_widths[index] * layout.row_bytes(input_width):
                raise ValueError("packed byte count does not match the layer shape and precision")
            if scales[index].dtype != scales[0].dtype or (zeros[index] is not None) != with_zeros:
                raise ValueError("the matrices of a launch group share the scale dtype and the use of offsets")
            if zeros[index] is not None and zeros[index].dtype != scales[0].dtype:
                raise ValueError("zeros must have the dtype of scales")
        bias_dtypes = {entry.dtype for entry in bias if entry is not None}
        if len(bias_dtypes) > 1:
            raise ValueError("the biases of a launch group share one dtype")
        pointers = ctypes.c_void_p * count
        self.keep = (packed, scales, values, zeros, bias)
        self.count = count
        self.output_widths = list(output_widths)
        self.input_width = input_width
        self._x = pointers()
        self._y = pointers()
        self._constant = (
            pointers(*[entry.data_ptr() for entry in packed]), pointers(*[entry.data_ptr() for entry in scales]),
            native.dtype_code(scales[0]), values.data_ptr(), values.numel(),
            pointers(*[native.pointer(entry) for entry in zeros]) if with_zeros else None,
            pointers(*[native.pointer(entry) for entry in bias]) if bias_dtypes else None,
            native.DTYPE_CODES[next(iter(bias_dtypes))] if bias_dtypes else 0,
        )
        self._widths = (ctypes.c_int * count)(*output_widths)
        self._tail = (input_width, group, layout.bits, int(uniform_grid), grid_minimum, grid_step)

    def __call__(self, inputs: "Tensor | list[Tensor]", outputs: list[Tensor], stream: int | None = None) -> None:
        """``outputs[i][m, n] = sum_k dequant(code_i[n, k]) * inputs_i[m, k] (+ bias_i[n])`` on the current
        stream.  ``inputs`` is one tensor every matrix reads, or one tensor per matrix (the same
        shape and dtype: e.g. the experts of a mixture-of-experts layer)."""
        shared = isinstance(inputs, Tensor)
        each = [inputs] * self.count if shared else list(inputs)
        if len(each) != self.count or len(outputs) != self.count:
            raise ValueError("one input (or one shared input) and one output per matrix of the group")
        first = each[0]
        samples = first.shape[0]
        for index, (entry, output) in enumerate(zip(each, outputs)):
            if (not entry.is_cuda or entry.device != self.device or not entry.is_contiguous()
                    or tuple(entry.shape) != (samples, self.input_width) or entry.dtype != first.dtype):
                raise ValueError("grouped packed matvec needs contiguous inputs of one shape and dtype, of the layers' "
                                 "width, on their device")
            if (output.dtype != first.dtype or tuple(output.shape) != (samples, self.output_widths[index])
                    or not output.is_contiguous() or output.device != self.device):
                raise ValueError("outputs must be contiguous [samples, output_width] tensors of the inputs' dtype")
            self._x[index] = entry.data_ptr()
            self._y[index] = output.data_ptr()
        status = native.library().mk_packed_matvec_group(
            self._x, native.dtype_code(first), self.count, *self._constant, self._y, self._widths, samples,
            *self._tail, native.current_stream(self.device) if stream is None else stream)
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
