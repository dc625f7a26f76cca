"""Checkpoint layout: a versioned JSON manifest beside one safetensors file.

The same layout as the reference's checkpoints (/root/reference/src/mlkit/checkpoints/
manifest.py:3-5, saving.py:23-157, loading.py:37-180): a layer with a registered codec
stores its packed code stream (``<layer>.codes``) and its parameters (``<layer>.params.<p>``,
in their declared storage format, identical tensors stored once); other layers store the
dense reconstruction; everything else of the module's state is stored as ``state.<name>``,
without the buffers of packed layers, which are rebuilt from the codes.
"""

import hashlib
import json
import shutil
import tempfile
from collections.abc import Callable
from pathlib import Path
from typing import Any

import torch
from safetensors.torch import load_file, save_file
from torch import Tensor, nn

from mlkit_amd.models import QModel
from mlkit_amd.quantization.bitstream import pack, unpack
from mlkit_amd.quantization.codecs import decoder, registered
from mlkit_amd.quantization.core import Q

FORMAT_VERSION = 1
MANIFEST_FILE = "mlkit.json"
WEIGHTS_FILE = "weights.safetensors"
_NARROW_STORAGE = {torch.float16, torch.bfloat16, torch.float8_e4m3fn}
_JSON_TYPES = (str, int, float, bool, list, dict, type(None))


def _weight_name(layer: str) -> str:
    return f"{layer}.weight" if layer else "weight"


def _stored_parameter(name: str, value: Tensor, metadata: dict[str, Any]) -> tuple[Tensor, dict[str, Any]]:
    """A parameter in its storage form and the descriptor that restores it."""
    descriptor: dict[str, Any] = {"encoding": None}
    width = metadata.get("parameter_bits", {}).get(name)
    if width is not None:
        descriptor.update(encoding="packed", bits=width, shape=list(value.shape))
        return pack(value, width), descriptor
    fmt = metadata.get("parameter_formats", {}).get(name)
    if name in {"scales", "zero"}:
        fmt = metadata.get("scale_fmt", "fp32")
    if fmt == "fp16":
        value = value.half()
    elif fmt == "bf16":
        value = value.bfloat16()
    elif fmt == "fp8":
        value = value.to(torch.float8_e4m3fn)
    elif fmt == "e8m0":
        value = (value.float().log2().round() + 127).to(torch.uint8)
        descriptor["encoding"] = "e8m0"
    return value, descriptor


def describe_layers(quantized: dict[str, Q]) -> tuple[dict[str, Tensor], dict[str, Any]]:
    """Tensors and manifest entries of the rounded layers."""
    tensors: dict[str, Tensor] = {}
    layers: dict[str, Any] = {}
    stored_once: dict[tuple, str] = {}
    for layer, q in quantized.items():
        if not (registered(q.codec) and q.codes is not None):
            tensors[f"{layer}.reconstruction"] = q.w.detach().cpu().contiguous()
            layers[layer] = {"codec": None, "bits": q.bits}
            continue
        width = q.metadata.get("code_bits")
        if width is None:
            width = max(1, int(q.codes.max()).bit_length())
        tensors[f"{layer}.codes"] = pack(q.codes.cpu(), width)
        params: dict[str, Any] = {}
        for name, value in q.params.items():
            if not isinstance(value, Tensor):
                params[name] = {"value": value}
                continue
            stored, descriptor = _stored_parameter(name, value, q.metadata)
            stored = stored.detach().cpu().contiguous()
            digest = hashlib.sha256(stored.reshape(-1).view(torch.uint8).numpy().tobytes()).digest()
            key = (str(stored.dtype), tuple(stored.shape), digest)
            identifier = stored_once.setdefault(key, f"{layer}.params.{name}")
            if identifier == f"{layer}.params.{name}":
                tensors[identifier] = stored.clone()
            params[name] = {"tensor": identifier, **descriptor}
        layers[layer] = {"codec": q.codec, "shape": list(q.codes.shape), "code_bits": width, "bits": q.bits,
                         "params": params,
                         "metadata": {k: v for k, v in q.metadata.items() if isinstance(v, _JSON_TYPES)}}
    return tensors, layers


def _restored_parameter(tensors: dict[str, Tensor], descriptor: dict[str, Any]) -> Any:
    if "tensor" not in descriptor:
        return descriptor["value"]
    value = tensors[descriptor["tensor"]]
    if descriptor.get("encoding") == "e8m0":
        return torch.pow(2.0, value.float() - 127)
    if descriptor.get("encoding") == "packed":
        return unpack(value, descriptor["bits"], tuple(descriptor["shape"]))
    return value.float() if value.dtype in _NARROW_STORAGE else value


def restore_layer(tensors: dict[str, Tensor], name: str, entry: dict[str, Any]) -> Q:
    """The representation of one rounded layer, on the device of its tensors."""
    if entry["codec"] is None:
        return Q(tensors[f"{name}.reconstruction"], bits=entry["bits"])
    codes = unpack(tensors[f"{name}.codes"], entry["code_bits"], tuple(entry["shape"]))
    params = {key: _restored_parameter(tensors, value) for key, value in entry["params"].items()}
    return Q(codes=codes, params=params, decode=decoder(entry["codec"]), codec=entry["codec"], bits=entry["bits"],
             metadata={**entry.get("metadata", {}), "code_bits": entry["code_bits"]})


class _StateCollector:
    """The part of a module's state a checkpoint stores as ``state.<name>``: everything except
    the rounded weights (they come back from the codes), parameters tied to them, and the
    derived buffers of packed layers.  Tensors that are views of the same memory are stored
    once; the other names are recorded as aliases of the first."""

    DERIVED_BUFFERS = frozenset({"packed", "scales", "values", "zeros"})

    def __init__(self, model: QModel) -> None:
        self.rounded = set(model.quantized)
        self.skipped = {_weight_name(name) for name in model.quantized} | set(model.tied_weights)
        self.tensors: dict[str, Tensor] = {}
        self.aliases: dict[str, str] = {}
        self._owner_of_memory: dict[tuple, str] = {}

    def wanted(self, name: str) -> bool:
        if name in self.skipped:
            return False
        module_name, _, leaf = name.rpartition(".")
        return not (module_name in self.rounded and leaf in self.DERIVED_BUFFERS)

    def add(self, name: str, value: Tensor) -> None:
        memory = (value.device, value.data_ptr(), value.dtype, tuple(value.shape), tuple(value.stride()))
        owner = self._owner_of_memory.get(memory)
        if owner is None:
            self._owner_of_memory[memory] = name
            self.tensors[f"state.{name}"] = value.detach().cpu().contiguous().clone()
        else:
            self.aliases[name] = owner


def _manifest(model: QModel, layers: dict[str, Any], aliases: dict[str, str], tensors: dict[str, Tensor]) -> dict[str, Any]:
    reference_parameter = next(model.module.parameters(), None)
    dtype = torch.float32 if reference_parameter is None else reference_parameter.dtype
    return {
        "format_version": FORMAT_VERSION, "name": model.name, "architecture": "external",
        "dtype": str(dtype).removeprefix("torch."), "layers": layers, "reports": [], "pass_reports": [],
        "stability_reports": {}, "logical_bpw": model.bpw, "model_bpw": model.model_bpw,
        "parameter_accounting": None, "transforms": list(model.transforms), "activations": {}, "kv": None,
        "state_aliases": aliases, "tied_weights": model.tied_weights,
        "tensor_bytes": sum(tensor.numel() * tensor.element_size() for tensor in tensors.values()),
    }


def _publish(staged: Path, destination: Path) -> None:
    """Move a fully written checkpoint directory into place.  An existing checkpoint is set
    aside under a fresh name first and removed only after the new one is in place; if the new
    one cannot be moved in, the old one returns."""
    if not destination.exists():
        staged.rename(destination)
        return
    aside = Path(tempfile.mkdtemp(prefix=f".{destination.name}.replaced_", dir=destination.parent))
    aside.rmdir()                      # only the unique name is wanted
    destination.rename(aside)
    try:
        staged.rename(destination)
    except BaseException:
        aside.rename(destination)
        raise
    shutil.rmtree(aside, ignore_errors=True)


def save(model: QModel, path: "str | Path", *, overwrite: bool = False) -> None:
    """Write ``mlkit.json`` + ``weights.safetensors`` under ``path``; the directory appears (or is
    replaced, with ``overwrite``) only once both files are complete."""
    destination = Path(path).resolve()
    if destination.exists() and not overwrite:
        raise FileExistsError(f"checkpoint destination already exists: {destination}")
    destination.parent.mkdir(parents=True, exist_ok=True)
    tensors, layers = describe_layers(model.quantized)
    state = _StateCollector(model)
    for name, value in model.module.state_dict().items():
        if state.wanted(name):
            state.add(name, value)
    tensors.update(state.tensors)
    with tempfile.TemporaryDirectory(prefix="mlkit_checkpoint_", dir=destination.parent) as scratch:
        staged = Path(scratch) / "checkpoint"
        staged.mkdir()
        save_file(tensors, str(staged / WEIGHTS_FILE))
        (staged / MANIFEST_FILE).write_text(json.dumps(_manifest(model, layers, state.aliases, tensors), indent=2) + "\n")
        _publish(staged, destination)


def load_checkpoint(path: "str | Path", *, model: "nn.Module | Callable[[], nn.Module]", device: str = "cuda") -> QModel:
    """Rebuild a ``QModel`` from a checkpoint; ``model`` is the module (or a factory for it)
    whose state the checkpoint holds."""
    directory = Path(path)
    manifest = json.loads((directory / MANIFEST_FILE).read_text())
    if manifest.get("format_version") != FORMAT_VERSION:
        raise ValueError("unsupported mlkit checkpoint format version")
    dtype = getattr(torch, manifest["dtype"])
    module = model if isinstance(model, nn.Module) else model()
    module.to(dtype=dtype)
    tensors = load_file(str(directory / WEIGHTS_FILE), device=device)
    state = {name.removeprefix("state."): value for name, value in tensors.items() if name.startswith("state.")}
    for alias, first in manifest.get("state_aliases", {}).items():
        state[alias] = state[first]
    restored: dict[str, Q] = {}
    for name, entry in manifest["layers"].items():
        q = restore_layer(tensors, name, entry)
        with torch.no_grad():
            state[_weight_name(name)] = q.w.to(dtype)
        restored[name] = q.to("cpu", detach=True)
    tied = manifest.get("tied_weights", {})
    for parameter_name, layer_name in tied.items():
        state[parameter_name] = state[_weight_name(layer_name)]
    from mlkit_amd.conversion import install_transform, record_transform

    for descriptor in manifest.get("transforms", []):
        install_transform(module, descriptor)
        record_transform(module, descriptor)
    module.load_state_dict(state, strict=True)
    converted = QModel(module.eval(), None, name=manifest["name"])
    converted.quantized = restored
    converted.tied_weights = dict(tied)
    return converted
