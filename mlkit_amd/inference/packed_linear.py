"""A linear layer (and a tied embedding) that execute packed scalar-grid codes.

Drop-in for /root/reference/src/mlkit/inference/packed_linear.py: ``PackedLinear`` (:41-245),
``PackedEmbedding`` (:248-287), ``packed_compatible`` (:290-304) -- the same buffers
(``packed``, ``scales``, ``values``, ``zeros``, ``bias``; ``_dense_weight`` non-persistent),
attributes and error messages.

How a call is served here:

* up to ``maximum_fused_rows`` input rows: one ``mk_packed_matvec`` launch, or, when the layer
  has absorbed its online input rotation, one ``mk_rotated_packed_matvec`` call (rotation
  kernel and matvec enqueued back to back, the rotated activations staying in a small buffer
  of the layer);
* more rows, or a layout without a fused kernel: the weight is decoded once
  (``mk_packed_decode``) and an ordinary matrix product follows;
* a tied embedding decodes only the requested rows (``mk_packed_decode_rows``).
"""

import copy
from collections.abc import Callable
from dataclasses import dataclass

import torch
import torch.nn.functional as functional
from torch import Tensor, nn

from mlkit_amd import native
from mlkit_amd.kernels.packed_linear import (MAXIMUM_CODE_BITS, GroupLaunch, PackedLayout, decode, layout_for,
                                             packed_matvec_op)
from mlkit_amd.quantization.bitstream import pack, unpack
from mlkit_amd.quantization.codecs import decode_scaled
from mlkit_amd.quantization.core import Q

SCALE_STORAGE_DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16}
MAXIMUM_FUSED_ROWS = 8
_LAUNCH_BUFFERS = frozenset({"packed", "scales", "values", "zeros", "bias"})


def preserve_input_processing(original: nn.Module, replacement: nn.Module) -> None:
    """Carry online input transforms (forward pre-hooks and their ``_mlkit_`` buffers) over to
    the layer that replaces ``original`` (models/module_utilities.py:19-25 in the reference)."""
    replacement._forward_pre_hooks = original._forward_pre_hooks.copy()
    replacement._forward_pre_hooks_with_kwargs = original._forward_pre_hooks_with_kwargs.copy()
    for name, value in original.named_buffers(recurse=False):
        if name.startswith("_mlkit_"):
            replacement.register_buffer(name, value.detach().clone())


def packed_compatible(quantized: Q) -> bool:
    """Whether ``quantized`` can be held as a packed stream: a complete ``scaled`` / ``feedback``
    codec of one to eight bits whose table fits the code width, in natural column order, with
    no code offset and refit regions made of whole scale groups."""
    if quantized.codec not in ("scaled", "feedback") or quantized.codes is None:
        return False
    parameters = quantized.params
    width = quantized.metadata.get("code_bits")
    if not isinstance(width, int) or not 1 <= width <= MAXIMUM_CODE_BITS:
        return False
    if parameters["values"].numel() > (1 << width):
        return False
    if parameters.get("permutation") is not None or parameters.get("offset", 0) != 0:
        return False
    group = parameters["group"]
    return parameters.get("refit", group) % group == 0


@dataclass(frozen=True)
class _Grid:
    """The value table as the kernels see it: affine grids need no table lookup."""

    uniform: bool
    minimum: float
    step: float

    @staticmethod
    def of(values: Tensor) -> "_Grid":
        table = values.detach().float().cpu()
        if table.numel() < 2:
            return _Grid(False, float(table[0]) if table.numel() else 0.0, 1.0)
        gaps = table[1:] - table[:-1]
        return _Grid(bool(torch.allclose(gaps, gaps[0].expand_as(gaps))), float(table[0]), float(gaps[0]))


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

    def __init__(self, original: nn.Linear, quantized: Q, *, cache_dense: bool = False,
                 overflow: Tensor | None = None) -> None:
        """``overflow``: a one-element int32 tensor on the layer's device that collects the range check of
        the codes (see ``pack``); the caller looks at it once for all the layers it builds.  Without it the
        check is made here, which synchronises."""
        super().__init__()
        if not packed_compatible(quantized):
            raise ValueError(
                "PackedLinear requires a complete scalar-grid codec of at most eight bits in "
                "its original column order with refit boundaries aligned to scale groups")
        device = original.weight.device
        if device.type != "cuda":
            raise ValueError("PackedLinear requires CUDA weights")
        native.library()  # a missing kernel library is reported here, not at the first forward
        parameters, metadata = quantized.params, quantized.metadata
        self.in_features, self.out_features = original.in_features, original.out_features
        self.group: int = parameters["group"]
        self.code_bits = int(metadata["code_bits"])
        self.storage_dtype = original.weight.dtype
        self.cache_dense = cache_dense
        # Side information is kept in the 16-bit format it was rounded to, when there is one.
        side_dtype = SCALE_STORAGE_DTYPES.get(str(metadata.get("scale_fmt")), parameters["scales"].dtype)

        def resident(tensor: Tensor | None, dtype: torch.dtype) -> Tensor | None:
            return None if tensor is None else tensor.detach().to(device=device, dtype=dtype).contiguous()

        if overflow is not None and overflow.device != device:
            overflow = None
        self.register_buffer("packed", pack(quantized.codes.to(device), self.code_bits, overflow=overflow))
        self.register_buffer("scales", resident(parameters["scales"], side_dtype))
        self.register_buffer("values", resident(parameters["values"], torch.float32))
        self.register_buffer("zeros", resident(parameters.get("zero"), side_dtype))
        self.register_buffer("bias", None if original.bias is None else original.bias.detach().clone())
        self.register_buffer("_dense_weight", None, persistent=False)
        grid = _Grid.of(parameters["values"])
        self.uniform_grid, self.grid_minimum, self.grid_step = grid.uniform, grid.minimum, grid.step
        self.layout: PackedLayout | None = layout_for(self.code_bits, self.in_features, self.group)
        self.maximum_fused_rows = MAXIMUM_FUSED_ROWS if self.layout is not None else 0
        self._launch: tuple | None = None
        self._rotation = None          # an absorbed OnlineRotation
        self._rotation_launch: tuple | None = None
        self._siblings: SiblingLaunch | None = None
        preserve_input_processing(original, self)
        self._absorb_rotation_hook()

    # -- online input rotation ---------------------------------------------------------------

    def absorb_input_rotation(self, rotation) -> None:
        """Run ``rotation`` (an ``OnlineRotation``) on the inputs inside ``forward`` instead of
        in a forward pre-hook: short inputs then take one library call for rotation + matvec."""
        self._rotation = rotation
        self._rotation_launch = None

    def _absorb_rotation_hook(self) -> None:
        """A carried-over ``RotateInputs`` pre-hook is taken in when it is the only pre-hook
        (so the order in which input transforms apply cannot change)."""
        from mlkit_amd.conversion import RotateInputs

        hooks = self._forward_pre_hooks
        if len(hooks) == 1 and not self._forward_pre_hooks_with_kwargs:
            (key, hook), = hooks.items()
            if isinstance(hook, RotateInputs):
                del hooks[key]
                self.absorb_input_rotation(hook.rotation)

    # -- module plumbing ---------------------------------------------------------------------

    def __setattr__(self, name: str, value) -> None:
        if name in _LAUNCH_BUFFERS:   # a replaced buffer: bound launch arguments are stale
            self.__dict__["_launch"] = None
            siblings = self.__dict__.get("_siblings")
            if siblings is not None:
                siblings.reset()
        super().__setattr__(name, value)

    def register_buffer(self, name: str, tensor, persistent: bool = True) -> None:
        if name in _LAUNCH_BUFFERS and "_siblings" in self.__dict__:
            self.__dict__["_launch"] = None
            if self.__dict__["_siblings"] is not None:
                self.__dict__["_siblings"].reset()
        super().register_buffer(name, tensor, persistent)

    def __getstate__(self) -> dict:
        """Bound launch arguments hold raw device addresses: a pickled or deep-copied layer (both go through
        here) binds its own on first use."""
        state = self.__dict__.copy()
        state["_launch"] = state["_rotation_launch"] = None
        return state

    def _apply(self, fn: Callable[[Tensor], Tensor], recurse: bool = True) -> "PackedLinear":
        self._launch = self._rotation_launch = None
        self._dense_weight = None
        if self._siblings is not None:
            self._siblings.reset()
        return super()._apply(fn, recurse)

    @property
    def weight(self) -> Tensor:
        """The dense ``[out_features, in_features]`` weight in the storage dtype."""
        cached = self._dense_weight
        if cached is not None:
            return cached
        shape = (self.out_features, self.in_features)
        if self.layout is not None:
            dense = torch.empty(shape, device=self.packed.device, dtype=self.storage_dtype)
            decode(self.packed, self.scales, self.values, self.zeros, dense, self.group, self.layout,
                   self.uniform_grid, self.grid_minimum, self.grid_step)
        else:  # rows or groups split a packing word: unpack the stream, then the scalar decoder
            offsets = self.zeros.float() if self.zeros is not None else None
            dense = decode_scaled(unpack(self.packed, self.code_bits, shape), scales=self.scales.float(),
                                  values=self.values, group=self.group, zero=offsets).to(self.storage_dtype)
        if self.cache_dense:
            self._dense_weight = dense
        return dense

    # -- forward -----------------------------------------------------------------------------

    def forward(self, inputs: Tensor) -> Tensor:
        if inputs.shape[-1] != self.in_features:
            raise ValueError("input width does not match the packed linear")
        if not inputs.is_cuda:
            raise ValueError("packed inference requires CUDA inputs")
        rows = inputs.numel() // self.in_features
        fused = 0 < rows <= self.maximum_fused_rows and inputs.dtype in native.DTYPE_CODES
        compiling = torch.compiler.is_compiling()
        rotate_here = False
        if self._rotation is not None:
            if fused and not compiling and self._rotation_arguments(inputs) is not None:
                rotate_here = True
            else:
                inputs = self._rotation(inputs)   # the general path: rotate, then as an unrotated layer
        if not fused:
            return functional.linear(inputs, self.weight.to(inputs.dtype), self.bias)
        if inputs.requires_grad and torch.is_grad_enabled():
            raise RuntimeError("packed CUDA inference does not support autograd")
        flat = inputs.reshape(rows, self.in_features)
        if not flat.is_contiguous():
            flat = flat.contiguous()
        if compiling:
            output = packed_matvec_op(flat, self.packed, self.scales, self.values, self.zeros, self.bias,
                                      self.out_features, self.group, self.code_bits, self.uniform_grid,
                                      self.grid_minimum, self.grid_step)
        elif self._siblings is not None and not rotate_here:
            output = self._siblings.output_for(self, inputs, flat)
        else:
            output = inputs.new_empty((rows, self.out_features))
            self._matvec(flat, output, rows, rotate_here)
        return output.view(inputs.shape[:-1] + (self.out_features,))

    # -- grouped launches with sibling layers ------------------------------------------------

    @property
    def groupable(self) -> bool:
        """Whether this layer may share a launch with siblings: a fused layout, no input
        transform of its own."""
        return (self.layout is not None and self._rotation is None and not self._forward_pre_hooks
                and not self._forward_pre_hooks_with_kwargs)

    @property
    def group_key(self) -> tuple:
        """What sibling layers must have in common to share a launch."""
        return (self.in_features, self.group, self.code_bits, self.uniform_grid, self.grid_minimum, self.grid_step,
                tuple(self.values.tolist()), self.scales.dtype, self.zeros is None,
                None if self.bias is None else self.bias.dtype, self.packed.device)

    def _bound_arguments(self) -> tuple:
        """The layer's constant launch arguments, bound once and kept for as long as all five
        buffers stay where they were: the key is every buffer's address and dtype, so a moved,
        cast, reassigned or reloaded buffer rebuilds them."""
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
        return launch

    def _rotation_arguments(self, inputs: Tensor) -> tuple | None:
        """``(key, rotated buffer, leading arguments of mk_rotated_packed_matvec, keep)`` for
        this device and input dtype, or None when the rotation kernels do not take the width."""
        key = (inputs.device, inputs.dtype)
        bound = self._rotation_launch
        if bound is not None and bound[0] == key and bound[1] is not None:
            # the bound pointers are addresses of the `keep` tensors: a copied or reloaded layer carries copies
            # of those tensors (or none), never the addresses
            _, _, basis, signs, _ = bound[2]
            keep = bound[3]
            if keep[0].data_ptr() != signs or (basis is not None and (len(keep) < 2 or keep[1].data_ptr() != basis)):
                bound = None
        if bound is None or bound[0] != key:
            arguments = self._rotation.launch_arguments(self.in_features, inputs.device)
            if arguments is None:
                bound = self._rotation_launch = (key, None, None, None)
            else:
                order, power, basis, signs, scale, keep = arguments
                rotated = torch.empty((MAXIMUM_FUSED_ROWS, self.in_features), dtype=inputs.dtype, device=inputs.device)
                bound = self._rotation_launch = (key, rotated, (order, power, basis, signs, scale), keep)
        return None if bound[1] is None else bound

    def _matvec(self, inputs: Tensor, output: Tensor, rows: int, rotate: bool = False) -> None:
        """One call into the C ABI on the current stream."""
        _, tensors, constants = self._bound_arguments()
        stream = native.current_stream(inputs.device)
        code = native.DTYPE_CODES[inputs.dtype]
        if rotate:
            _, rotated, rotation, _ = self._rotation_arguments(inputs)
            status = native.library().mk_rotated_packed_matvec(
                inputs.data_ptr(), code, rotated.data_ptr(), *rotation, *tensors, output.data_ptr(), rows, *constants,
                stream)
        else:
            status = native.library().mk_packed_matvec(inputs.data_ptr(), code, *tensors, output.data_ptr(), rows,
                                                       *constants, stream)
        if status:
            native.check(status)


class SiblingLaunch:
    """Packed layers that read the same activations, multiplied by one launch.

    The first member whose ``forward`` sees an input runs ``mk_packed_matvec_group`` for all
    members and keeps the others' outputs; each other member, called with the *same tensor*
    (same object, or same memory, shape and version), takes its output from there, once.  The
    kept input is referenced for as long as outputs are pending, so its memory cannot be
    handed to another tensor meanwhile; an in-place change is noticed through the tensor's
    version counter where one exists (not under ``torch.inference_mode``: there the model must
    not modify the shared input between the sibling calls).  Anything else -- another input, a
    member called twice -- simply starts a new grouped launch, so results never depend on the
    cache being hit.  A member that is called with another input while its output of the last
    grouped launch still waits does not share its siblings' input: it leaves the group."""

    MAXIMUM = 8

    def __init__(self, layers: list[PackedLinear]) -> None:
        self.layers = tuple(layers)
        for layer in self.layers:
            layer._siblings = self
        self._launch: GroupLaunch | None = None
        self._pending: tuple | None = None

    def reset(self) -> None:
        self._launch = None
        self._pending = None

    def __getstate__(self) -> dict:
        return {"layers": self.layers, "_launch": None, "_pending": None}

    def _release(self, layer: "PackedLinear") -> None:
        """Take ``layer`` out of the group; a group of one is dissolved."""
        layer._siblings = None
        self.layers = tuple(member for member in self.layers if member is not layer)
        self._launch = None
        if self._pending is not None:
            self._pending[2].pop(id(layer), None)
            if not self._pending[2]:
                self._pending = None
        if len(self.layers) == 1:
            self.layers[0]._siblings = None
            self.layers = ()
            self._pending = None

    def __deepcopy__(self, memo: dict) -> "SiblingLaunch":
        """A copy links the copied layers and binds its own launch arguments on first use."""
        clone = SiblingLaunch.__new__(SiblingLaunch)
        memo[id(self)] = clone
        clone.layers = tuple(copy.deepcopy(layer, memo) for layer in self.layers)
        clone._launch = None
        clone._pending = None
        return clone

    @staticmethod
    def _version(tensor: Tensor) -> int | None:
        try:
            return tensor._version
        except RuntimeError:  # inference tensors keep no version counter
            return None

    def _bound(self) -> GroupLaunch:
        if self._launch is None:
            first = self.layers[0]
            self._launch = GroupLaunch(
                [layer.packed for layer in self.layers], [layer.scales for layer in self.layers], first.values,
                [layer.zeros for layer in self.layers], [layer.bias for layer in self.layers],
                [layer.out_features for layer in self.layers], first.in_features, first.group, first.layout,
                uniform_grid=first.uniform_grid, grid_minimum=first.grid_minimum, grid_step=first.grid_step)
        return self._launch

    def output_for(self, layer: PackedLinear, original: Tensor, flat: Tensor) -> Tensor:
        pending = self._pending
        if pending is not None:
            kept, version, outputs = pending
            # without a version counter only the very same tensor object counts as the same input
            same = kept is original or (version is not None and kept.data_ptr() == original.data_ptr()
                                        and kept.shape == original.shape and kept.dtype == original.dtype
                                        and kept.stride() == original.stride())
            if same and version == self._version(original) and id(layer) in outputs:
                output = outputs.pop(id(layer))
                if not outputs:
                    self._pending = None
                return output
            if id(layer) in outputs and kept is not original and kept.data_ptr() != original.data_ptr():
                # an output of this layer is still waiting and it is called with a tensor that lives elsewhere: it
                # does not read what its siblings read (an output projection beside q / k / v).  It leaves the
                # group; its share of every grouped launch was wasted work.
                self._release(layer)
                output = flat.new_empty((flat.shape[0], layer.out_features))
                layer._matvec(flat, output, flat.shape[0])
                return output
        rows = flat.shape[0]
        results = [flat.new_empty((rows, member.out_features)) for member in self.layers]
        self._bound()(flat, results)
        outputs = {id(member): result for member, result in zip(self.layers, results)}
        mine = outputs.pop(id(layer))
        self._pending = (original, self._version(original), outputs) if outputs else None
        return mine


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
        device = head.packed.device
        tokens = indices.reshape(-1).to(device=device, dtype=torch.int64).contiguous()
        embedded = torch.empty((tokens.numel(), self.embedding_dim), dtype=head.storage_dtype, device=device)
        if tokens.numel():
            native.check(native.library().mk_packed_decode_rows(
                head.packed.data_ptr(), head.scales.data_ptr(), native.dtype_code(head.scales), head.values.data_ptr(),
                head.values.numel(), native.pointer(head.zeros), tokens.data_ptr(), tokens.numel(), embedded.data_ptr(),
                native.dtype_code(embedded), self.num_embeddings, self.embedding_dim, head.group, head.code_bits,
                int(head.uniform_grid), head.grid_minimum, head.grid_step, native.current_stream(device)))
        return embedded.view(*indices.shape, self.embedding_dim)
