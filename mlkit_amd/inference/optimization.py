"""Selection of dense or packed execution for a converted model.

Mirrors /root/reference/src/mlkit/inference/optimization.py:11-100 (``optimize``): same
arguments, the same replacement rules (a packed-compatible ``nn.Linear`` becomes a
``PackedLinear``; an embedding tied to a packed head becomes a ``PackedEmbedding``) and the
same ``execution_backend`` strings (``"dense"``, ``"packed:<n>"``, ``+compiled``).
"""

import copy

from torch import nn

from mlkit_amd.inference.packed_linear import PackedEmbedding, PackedLinear, packed_compatible
from mlkit_amd.models import Model, QModel


def optimize(model: "Model | nn.Module", backend: str = "auto", *, compile: bool = False,
             mode: str = "reduce-overhead", cache_dense: bool = False, inplace: bool = False) -> Model:
    """Keep every reconstruction while choosing how it executes.

    Packed execution covers scalar ``Q`` codecs of one to eight bits; other layers stay dense.
    """
    if backend not in {"auto", "dense", "packed"}:
        raise ValueError("backend must be auto, dense, or packed")
    wrapped = model if isinstance(model, Model) else Model(model)
    if backend == "auto":
        backend = "packed" if isinstance(wrapped, QModel) else "dense"
    if backend == "dense":
        converted = wrapped if inplace else copy.deepcopy(wrapped)
        converted.execution_backend = "dense"
    else:
        if not isinstance(wrapped, QModel):
            raise ValueError("packed inference requires a QModel with codec state")
        swaps: dict[str, nn.Module] = {}
        for name, quantized in wrapped.quantized.items():
            layer = wrapped.module.get_submodule(name)
            if isinstance(layer, nn.Linear) and packed_compatible(quantized):
                swaps[name] = PackedLinear(layer, quantized, cache_dense=cache_dense)
        packed_layers = len(swaps)
        for parameter_name, layer_name in wrapped.tied_weights.items():
            owner_name = parameter_name.rpartition(".")[0]
            owner = wrapped.module.get_submodule(owner_name)
            head = swaps.get(layer_name)
            if isinstance(owner, nn.Embedding) and isinstance(head, PackedLinear) and head.layout is not None:
                swaps[owner_name] = PackedEmbedding(head, owner)
        if inplace:
            for name, replacement in swaps.items():
                if name:
                    wrapped.module.set_submodule(name, replacement)
                else:
                    wrapped.module = replacement
            converted = wrapped
        else:
            # deepcopy with the replaced modules pre-seeded in the memo: the copy holds the
            # packed layers instead of copies of the dense ones
            memo = {id(wrapped.module.get_submodule(name)): replacement for name, replacement in swaps.items()}
            converted = copy.deepcopy(wrapped, memo)
            for layer in converted.module.modules():
                if isinstance(layer, PackedLinear):
                    layer._forward_pre_hooks = copy.deepcopy(layer._forward_pre_hooks, memo)
        converted.execution_backend = f"packed:{packed_layers}"
    if compile:
        converted.module.compile(mode=mode)
        converted.execution_backend += "+compiled"
    return converted
