"""A linear layer (and a tied embedding) that execute packed scalar-grid codes.

Mirrors /root/reference/src/mlkit/inference/packed_linear.py: ``PackedLinear`` (:41-245),
``PackedEmbedding`` (:248-287), ``packed_compatible`` (:290-304) -- same buffers
(``packed``, ``scales``, ``values``, ``zeros``, ``bias``; ``_dense_weight`` non-persistent),
attributes and error messages.  Up to ``maximum_fused_rows`` input rows go to
``mk_packed_matvec``; larger inputs decode the weight once (``mk_packed_decode``) and use an
ordinary matrix product.
"""

from collections.abc import Callable

import torch
import torch.nn.functional as functional
from torch import Tensor, nn

from mlkit_amd import native
from mlkit_amd.kernels.packed_linear import MAXIMUM_CODE_BITS, decode, layout_for, packed_matvec_op
from mlkit_amd.quantization.bitstream import pack, unpack
from mlkit_amd.quantization.codecs import decode_scaled
from mlkit_amd.quantization.core import Q

SCALE_STORAGE_DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16}
MAXIMUM_FUSED_ROWS = 8


def preserve_input_processing(original: nn.Module, replacement: nn.Module) -> None:
    """Carry online input transforms (forward pre-hooks and their ``_mlkit_`` buffers) over to
    the layer that replaces ``original`` (models/module_utilities.py:19-25 in the reference)."""
    replacement._forward_pre_hooks = original._forward_pre_hooks.copy()
    replacement._forward_pre_hooks_with_kwargs = original._forward_pre_hooks_with_kwargs.copy()
    for name, value in original.named_buffers(recurse=False):
        if name.startswith("_mlkit_"):
            replacement.register_buffer(name, value.detach().clone())


class PackedLinear(nn.Module):
    """Exact scalar-grid codes of one to eight bits with fused decode for short inputs.

    A layer whose rows or scale groups split a packing word keeps its packed storage and
    always reconstructs the dense weight (``layout is None``, ``maximum_fused_rows == 0``).
    """

    packed: Tensor
    scales: Tensor
    values: Tensor
    zeros: Tensor | None
    bias: Tensor | None
    _dense_weight: Tensor | None

    def __init__(self, original: nn.Linear, quantized: Q, *, cache_dense: bool = False) -> None:
        super().__init__()
        if not packed_compatible(quantized):
            raise ValueError(
                "PackedLinear requires a complete scalar-grid codec of at most eight bits in "
                "its original column order with refit boundaries aligned to scale groups")
        assert quantized.codes is not None
        device = original.weight.device
        if device.type != "cuda":
            raise ValueError("PackedLinear requires CUDA weights")
        native.library()  # fail here, not at the first forward, when the kernels are not built
        self.in_features, self.out_features = original.in_features, original.out_features
        self.group = quantized.params["group"]
        self.code_bits = int(quantized.metadata["code_bits"])
        self.storage_dtype = original.weight.dtype
        self.cache_dense = cache_dense
        scales = quantized.params["scales"]
        side_dtype = SCALE_STORAGE_DTYPES.get(str(quantized.metadata.get("scale_fmt")), scales.dtype)
        zero = quantized.params.get("zero")
        self.register_buffer("packed", pack(quantized.codes, self.code_bits).to(device))
        self.register_buffer("scales", scales.to(device=device, dtype=side_dtype).contiguous())
        self.register_buffer("values", quantized.params["values"].to(device=device, dtype=torch.float32).contiguous())
        self.register_buffer("zeros", None if zero is None else zero.to(device=device, dtype=side_dtype).contiguous())
        self.register_buffer("bias", None if original.bias is None else original.bias.detach().clone())
        self.register_buffer("_dense_weight", None, persistent=False)
        table = quantized.params["values"].detach().cpu().float()
        steps = table.diff()
        self.uniform_grid = bool(len(steps) and torch.allclose(steps, steps[0].expand_as(steps)))
        self.grid_minimum = float(table[0])
        self.grid_step = float(steps[0]) if len(steps) else 1.0
        self.layout = layout_for(self.code_bits, self.in_features, self.group)
        self.maximum_fused_rows = 0 if self.layout is None else MAXIMUM_FUSED_ROWS
        self._launch: tuple | None = None
        preserve_input_processing(original, self)

    def _apply(self, fn: Callable[[Tensor], Tensor], recurse: bool = True) -> "PackedLinear":
        self._launch = None
        self._dense_weight = None
        return super()._apply(fn, recurse)

    @property
    def weight(self) -> Tensor:
        if self._dense_weight is not None:
            return self._dense_weight
        if self.layout is None:
            codes = unpack(self.packed, self.code_bits, (self.out_features, self.in_features))
            dense = decode_scaled(codes, scales=self.scales.float(), values=self.values, group=self.group,
                                  zero=None if self.zeros is None else self.zeros.float()).to(self.storage_dtype)
        else:
            dense = torch.empty((self.out_features, self.in_features), device=self.packed.device,
                                dtype=self.storage_dtype)
            decode(self.packed, self.scales, self.values, self.zeros, dense, self.group, self.layout,
                   self.uniform_grid, self.grid_minimum, self.grid_step)
        if self.cache_dense:
            self._dense_weight = dense
        return dense

    def forward(self, inputs: Tensor) -> Tensor:
        width = self.in_features
        shape = inputs.shape
        if shape[-1] != width:
            raise ValueError("input width does not match the packed linear")
        if not inputs.is_cuda:
            raise ValueError("packed inference requires CUDA inputs")
        rows = inputs.numel() // width
        if rows > self.maximum_fused_rows or rows == 0 or inputs.dtype not in native.DTYPE_CODES:
            return functional.linear(inputs, self.weight.to(inputs.dtype), self.bias)
        if inputs.requires_grad and torch.is_grad_enabled():
            raise RuntimeError("packed CUDA inference does not support autograd")
        flat = inputs.reshape(rows, width)
        if not flat.is_contiguous():
            flat = flat.contiguous()
        if torch.compiler.is_compiling():
            output = packed_matvec_op(flat, self.packed, self.scales, self.values, self.zeros, self.bias,
                                      self.out_features, self.group, self.code_bits, self.uniform_grid,
                                      self.grid_minimum, self.grid_step)
        else:
            output = inputs.new_empty((rows, self.out_features))
            self._matvec(flat, output, rows)
        return output.view(shape[:-1] + (self.out_features,))

    def _matvec(self, inputs: Tensor, output: Tensor, rows: int) -> None:
        """One call into the C ABI.  The layer's constant arguments are bound once and kept
        for as long as all five buffers stay where they were: the key is every buffer's
        address, so a moved, cast, reassigned or reloaded ``scales`` / ``zeros`` / ``bias`` /
        ``values`` / ``packed`` rebuilds them."""
        buffers = self._buffers
        packed, scales, values = buffers["packed"], buffers["scales"], buffers["values"]
        zeros, bias = buffers["zeros"], buffers["bias"]
        key = (packed.data_ptr(), scales.data_ptr(), values.data_ptr(),
               0 if zeros is None else zeros.data_ptr(), 0 if bias is None else bias.data_ptr(),
               scales.dtype, None if bias is None else bias.dtype)
        launch = self._launch
        if launch is None or launch[0] != key:
            launch = self._launch = (
                key,
                (key[0], key[1], native.dtype_code(scales), key[2], values.numel(), native.pointer(zeros),
                 native.pointer(bias), 0 if bias is None else native.dtype_code(bias)),
                (self.out_features, self.in_features, self.group, self.code_bits, int(self.uniform_grid),
                 self.grid_minimum, self.grid_step),
            )
        _, tensors, constants = launch
        status = native.library().mk_packed_matvec(
            inputs.data_ptr(), native.DTYPE_CODES[inputs.dtype], *tensors, output.data_ptr(), rows, *constants,
            native.current_stream(inputs.device))
        if status:
            native.check(status)


class PackedEmbedding(nn.Module):
    """An embedding table read from the packed codes of a tied output projection.

    Row ``i`` of the projection is the embedding of token ``i``; only requested rows are
    decoded.  The projection is referenced without being registered: it already belongs to
    the model as its output head.
    """

    def __init__(self, projection: PackedLinear, original: nn.Embedding) -> None:
        super().__init__()
        if projection.layout is None:
            raise ValueError("a packed embedding requires rows that hold whole packing words")
        self._projection = (projection,)
        self.num_embeddings = projection.out_features
        self.embedding_dim = projection.in_features
        self.padding_idx = original.padding_idx

    @property
    def projection(self) -> PackedLinear:
        return self._projection[0]

    @property
    def weight(self) -> Tensor:
        return self.projection.weight

    def forward(self, indices: Tensor) -> Tensor:
        head = self.projection
        rows = indices.reshape(-1)
        taken = head.packed.view(self.num_embeddings, -1)[rows]
        codes = unpack(taken.reshape(-1), head.code_bits, (rows.numel(), self.embedding_dim))
        embedded = decode_scaled(codes, scales=head.scales[rows].float(), values=head.values, group=head.group,
                                 zero=None if head.zeros is None else head.zeros[rows].float())
        return embedded.to(head.storage_dtype).view(*indices.shape, self.embedding_dim)


def packed_compatible(quantized: Q) -> bool:
    """A complete scalar codec of at most eight bits, unpermuted, with refit regions that are
    whole scale groups."""
    if quantized.codec not in {"scaled", "feedback"}:
        return False
    group = quantized.params["group"]
    code_bits = quantized.metadata.get("code_bits")
    return (isinstance(code_bits, int) and 1 <= code_bits <= MAXIMUM_CODE_BITS
            and quantized.codes is not None
            and quantized.params["values"].numel() <= 2**code_bits
            and quantized.params.get("offset", 0) == 0
            and quantized.params.get("permutation") is None
            and quantized.params.get("refit", group) % group == 0)
