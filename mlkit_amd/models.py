"""Minimal model wrappers: what ``optimize`` and the checkpoint functions need.

``Model`` / ``QModel`` keep the attribute names of the reference's wrappers
(/root/reference/src/mlkit/models/model.py:18-166: ``module``, ``quantized``,
``tied_weights``, ``execution_backend``, ``bpw``) without its architecture adapters,
calibration engine or reports, which are outside this package's path.  ``quantize`` rounds
every ``nn.Linear`` of a module with one quantizer, collecting layer inputs for calibrated
quantizers from the batches it is given.
"""

import copy
from collections.abc import Callable, Iterable
from typing import Any

import torch
from torch import Tensor, nn

from mlkit_amd.quantization.core import Ctx, Q, as_q


class Model(nn.Module):
    def __init__(self, module: nn.Module, tokenizer: Any = None, *, name: str | None = None) -> None:
        super().__init__()
        self.module = module.cuda()
        self.tokenizer = tokenizer
        self.name = name or type(module).__name__
        self.execution_backend = "dense"

    def forward(self, *args: Any, **kwargs: Any) -> Any:
        device = self.device
        move = lambda value: value.to(device) if isinstance(value, Tensor) else value  # noqa: E731
        return self.module(*[move(a) for a in args], **{k: move(v) for k, v in kwargs.items()})

    @property
    def device(self) -> torch.device:
        tensor = next(self.module.parameters(), None)
        if tensor is None:
            tensor = next(self.module.buffers(), None)
        return torch.device("cuda") if tensor is None else tensor.device

    @property
    def storage_bytes(self) -> int:
        """Bytes of the distinct parameter and buffer storages of the module."""
        storages = {}
        for tensor in [*self.module.parameters(), *self.module.buffers()]:
            storage = tensor.untyped_storage()
            storages[(tensor.device, storage.data_ptr())] = storage.nbytes()
        return sum(storages.values())


class QModel(Model):
    """A converted model with the representation of every rounded layer.

    ``tied_weights`` maps the name of a parameter that shares a rounded weight (a tied input
    embedding) to the name of the layer that owns its codes.
    """

    def __init__(self, *args: Any, **kwargs: Any) -> None:
        super().__init__(*args, **kwargs)
        self.quantized: dict[str, Q] = {}
        self.tied_weights: dict[str, str] = {}

    @property
    def transforms(self) -> list[dict[str, Any]]:
        """Descriptors of the online transforms installed on the module (rotations)."""
        return list(getattr(self.module, "_mlkit_transforms", []))

    @property
    def bpw(self) -> float | None:
        if not self.quantized or any(q.bits is None for q in self.quantized.values()):
            return None
        bits = sum(float(q.bits) for q in self.quantized.values())
        return bits / sum(self.module.get_submodule(name).weight.numel() for name in self.quantized)

    model_bpw = bpw

    def save(self, path: Any, *, overwrite: bool = False) -> None:
        from mlkit_amd.checkpoints import save

        save(self, path, overwrite=overwrite)


CHUNKED_CONVERSION_ELEMENTS = 2**26
ROW_CHUNK_ELEMENTS = 2**25


def _round_layer(weight: Tensor, quantization: Callable[..., "Q | Tensor"], context: Ctx) -> Q:
    """One layer through its quantizer; very large row-separable layers go in row chunks
    whose representations are joined (the 151936-row output heads)."""
    chunked = weight.numel() > CHUNKED_CONVERSION_ELEMENTS and getattr(quantization, "row_separable", False)
    if not chunked:
        return as_q(quantization(weight, context))
    from mlkit_amd.quantization.codecs import concatenate_rows

    rows = max(1, ROW_CHUNK_ELEMENTS // weight.shape[1])
    parts = [as_q(quantization(weight[start:start + rows], context)) for start in range(0, weight.shape[0], rows)]
    return concatenate_rows(parts)


def quantize(model: "Model | nn.Module", quantization: Callable[..., "Q | Tensor"],
             calib: Iterable[Any] | None = None, *, head: Callable[..., "Q | Tensor"] | None = None,
             skip: Iterable[str] = (), seed: int = 0, cache_dir: Any = None) -> QModel:
    """Round every ``nn.Linear`` of a copy of ``model`` and record its ``Q``.

    ``calib`` is an iterable of positional-argument tuples (or single tensors) the module is
    called with once; each layer's flattened inputs become ``Ctx.X``.  A linear layer whose
    weight is tied to an embedding (an output head) is left alone unless ``head`` gives the
    quantizer for it.  ``cache_dir`` is accepted for call compatibility and unused.
    """
    source = model.module if isinstance(model, Model) else model
    converted = QModel(copy.deepcopy(source).eval(), getattr(model, "tokenizer", None),
                       name=getattr(model, "name", None) or type(source).__name__)
    module = converted.module
    embedded = {id(layer.weight) for layer in module.modules() if isinstance(layer, nn.Embedding)}
    skipped = set(skip)
    layers: dict[str, tuple[nn.Linear, Callable[..., "Q | Tensor"]]] = {}
    for name, layer in module.named_modules():
        if not isinstance(layer, nn.Linear) or name in skipped:
            continue
        if id(layer.weight) in embedded:
            if head is not None:
                layers[name] = (layer, head)
        else:
            layers[name] = (layer, quantization)
    seen: dict[str, list[Tensor]] = {name: [] for name in layers}
    if calib is not None:
        hooks = [layer.register_forward_pre_hook(
            lambda _, inputs, key=name: seen[key].append(inputs[0].detach().reshape(-1, inputs[0].shape[-1])))
            for name, (layer, _) in layers.items()]
        with torch.no_grad():
            for batch in calib:
                converted(*batch) if isinstance(batch, (tuple, list)) else converted(batch)
        for hook in hooks:
            hook.remove()
    owners = {id(layer.weight): name for name, (layer, _) in layers.items()}
    for name, parameter in module.named_parameters(remove_duplicate=False):
        owner = owners.get(id(parameter))
        if owner is not None and name != (f"{owner}.weight" if owner else "weight"):
            converted.tied_weights[name] = owner
    for name, (layer, chosen) in layers.items():
        inputs = torch.cat(seen[name]) if seen[name] else None
        context = Ctx(name, module=layer, X=inputs, seed=seed, device=layer.weight.device)
        with torch.no_grad():
            result = _round_layer(layer.weight.detach(), chosen, context)
            layer.weight.copy_(result.w.to(layer.weight.dtype))
        if result.bits is not None:
            result.bits = result.bits + context.additional_bits
        converted.quantized[name] = result
    # captured factorisations (a width x width buffer each) served this pass; the model that is served next
    # should not find their memory taken
    from mlkit_amd.quantization.feedback import clear_factor_graphs

    clear_factor_graphs()
    return converted
