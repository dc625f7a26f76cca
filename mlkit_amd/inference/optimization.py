"""Choosing how a converted model executes: dense weights, or packed codes.

``optimize`` has the call surface and results of the reference's
(/root/reference/src/mlkit/inference/optimization.py:11-100): ``backend`` is ``"auto"``,
``"dense"`` or ``"packed"``; a packed-compatible ``nn.Linear`` becomes a ``PackedLinear``, an
embedding tied to a packed head becomes a ``PackedEmbedding``; ``execution_backend`` reads
``"dense"``, ``"packed:<layers>"`` and gains ``"+compiled"``.

The work is split in three steps: plan the replacements from the codec state, build the
result (in place, or as a copy that never duplicates the dense layers being replaced), and
optionally link sibling layers into grouped launches (``group_siblings``, an addition of this
package).
"""

import copy
from collections import defaultdict

import torch
from torch import nn

from mlkit_amd.inference.packed_linear import PackedEmbedding, PackedLinear, SiblingLaunch, packed_compatible
from mlkit_amd.models import Model, QModel
from mlkit_amd.quantization.bitstream import check_overflow

BACKENDS = ("auto", "dense", "packed")


def _planned_replacements(model: QModel, cache_dense: bool) -> tuple[dict[str, nn.Module], int]:
    """``{module name: packed module}`` for every layer that can execute its codes, and the
    number of packed linear layers among them."""
    module = model.module
    # one range check of the codes per device for the whole model instead of one read-back per layer
    flags: dict[torch.device, torch.Tensor] = {}

    def flag_on(device: torch.device) -> "torch.Tensor | None":
        if device.type != "cuda":
            return None
        if device not in flags:
            flags[device] = torch.zeros(1, dtype=torch.int32, device=device)
        return flags[device]

    planned: dict[str, nn.Module] = {
        name: PackedLinear(module.get_submodule(name), state, cache_dense=cache_dense,
                           overflow=flag_on(module.get_submodule(name).weight.device))
        for name, state in model.quantized.items()
        if isinstance(module.get_submodule(name), nn.Linear) and packed_compatible(state)
    }
    for flag in flags.values():
        check_overflow(flag)
    linear_layers = len(planned)
    # An input embedding that shares the weight of a packed head reads the head's codes.
    for parameter, head_name in model.tied_weights.items():
        head = planned.get(head_name)
        owner_name = parameter.rsplit(".", 1)[0] if "." in parameter else ""
        owner = module.get_submodule(owner_name)
        if isinstance(head, PackedLinear) and head.layout is not None and isinstance(owner, nn.Embedding):
            planned[owner_name] = PackedEmbedding(head, owner)
    return planned, linear_layers


def _with_replacements(model: QModel, planned: dict[str, nn.Module], inplace: bool) -> QModel:
    if inplace:
        for name, replacement in planned.items():
            if name == "":
                model.module = replacement
            else:
                model.module.set_submodule(name, replacement)
        return model
    # A copy in which every replaced layer is "already copied" as its replacement: the dense
    # weights about to be dropped are never duplicated.
    already = {id(model.module.get_submodule(name)): replacement for name, replacement in planned.items()}
    result = copy.deepcopy(model, already)
    for layer in result.module.modules():
        if isinstance(layer, PackedLinear) and layer._forward_pre_hooks:
            layer._forward_pre_hooks = copy.deepcopy(layer._forward_pre_hooks, already)  # hooks bound to the copy
    return result


def _link_siblings(module: nn.Module) -> int:
    """Packed linear layers that sit side by side under one parent and take the same input
    width and codec are linked so that the first of them to see an input multiplies it for all
    of them in one launch (``mk_packed_matvec_group``).  Returns the number of groups."""
    families: dict[tuple, list[PackedLinear]] = defaultdict(list)
    for name, layer in module.named_modules():
        if isinstance(layer, PackedLinear) and layer.groupable:
            families[(name.rpartition(".")[0], *layer.group_key)].append(layer)
    groups = 0
    for layers in families.values():
        for first in range(0, len(layers) - 1, SiblingLaunch.MAXIMUM):
            members = layers[first:first + SiblingLaunch.MAXIMUM]
            if len(members) > 1:
                SiblingLaunch(members)
                groups += 1
    return groups


def optimize(model: "Model | nn.Module", backend: str = "auto", *, compile: bool = False,
             mode: str = "reduce-overhead", cache_dense: bool = False, inplace: bool = False,
             group_siblings: bool = False) -> Model:
    """Keep every reconstruction while choosing how it executes.

    Packed execution covers scalar ``Q`` codecs of one to eight bits; other layers stay dense.
    ``group_siblings`` (off by default) lets packed layers under one parent that read the same
    activations (attention q / k / v, MLP gate / up) share one kernel launch; it relies on the
    model handing those layers the very same tensor, unmodified between their calls.
    """
    if backend not in BACKENDS:
        raise ValueError("backend must be auto, dense, or packed")
    wrapped = model if isinstance(model, Model) else Model(model)
    has_codes = isinstance(wrapped, QModel)
    chosen = backend if backend != "auto" else ("packed" if has_codes else "dense")
    if chosen == "packed":
        if not has_codes:
            raise ValueError("packed inference requires a QModel with codec state")
        planned, linear_layers = _planned_replacements(wrapped, cache_dense)
        result = _with_replacements(wrapped, planned, inplace)
        result.execution_backend = f"packed:{linear_layers}"
        if group_siblings:
            _link_siblings(result.module)
    else:
        result = wrapped if inplace else copy.deepcopy(wrapped)
        result.execution_backend = "dense"
    if compile:
        result.module.compile(mode=mode)
        result.execution_backend += "+compiled"
    return result
