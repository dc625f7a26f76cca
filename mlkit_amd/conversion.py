"""Online input rotations of linear layers: the part of the reference's ``rotate`` pass that
sits on the packed-inference path.

Mirrors /root/reference/src/mlkit/conversion/model_transforms.py:116-128 (the online branch of
``Rotate``: every ``o_proj`` / ``down_proj`` gets its weight columns rotated offline with a
per-layer seed and a forward pre-hook that rotates its inputs) and :179-209
(``record_transform``, ``install_transform``; descriptor ``{"kind": "rotation", "name", "seed"}``,
persisted in the checkpoint manifest and re-installed on load).  The residual-stream rotation
of the same pass needs the architecture adapters and norm fusion, which are outside this
package's path.
"""

from dataclasses import dataclass
from typing import Any

import torch
from torch import nn

from mlkit_amd.models import Model
from mlkit_amd.quantization.core import layer_seed
from mlkit_amd.quantization.transforms import OnlineRotation, rht

ROTATED_LAYER_NAMES = ("o_proj", "down_proj")


def record_transform(model: nn.Module, descriptor: dict[str, Any]) -> None:
    descriptors = getattr(model, "_mlkit_transforms", [])
    descriptors.append(descriptor)
    model.__dict__["_mlkit_transforms"] = descriptors


class RotateInputs:
    """The forward pre-hook of a rotated layer: its first positional input goes through the
    layer's online rotation (fp16 / bf16 inputs are transformed in fp32 inside the kernel and
    rounded once).  A class rather than a closure so that a packed layer can recognise the
    hook and run the rotation in the same library call as its matvec."""

    def __init__(self, rotation: OnlineRotation) -> None:
        self.rotation = rotation

    def __call__(self, layer: nn.Module, arguments: tuple) -> tuple:
        return (self.rotation(arguments[0]), *arguments[1:])


def install_transform(model: nn.Module, descriptor: dict[str, Any]) -> None:
    """Attach the online half of a recorded transform to the layer it names."""
    if descriptor["kind"] != "rotation":
        raise ValueError(f"unknown model transform {descriptor['kind']!r}")
    layer = model.get_submodule(descriptor["name"])
    hook = RotateInputs(OnlineRotation(descriptor["seed"], descriptor.get("block")))
    absorb = getattr(layer, "absorb_input_rotation", None)
    if absorb is not None and not layer._forward_pre_hooks:
        absorb(hook.rotation)  # a packed layer runs the rotation inside its own launch sequence
    else:
        layer.register_forward_pre_hook(hook)


@dataclass
class Rotate:
    """``Rotate(seed)(model)``: rotate the input side of every selected linear layer."""

    seed: int = 0
    names: tuple[str, ...] = ROTATED_LAYER_NAMES
    block: int | None = None   # rotate blocks of this many input features one by one (None: the whole row, as the reference)

    def __call__(self, model: "Model | nn.Module", calib: Any = None) -> None:
        module = model.module if isinstance(model, Model) else model
        with torch.no_grad():
            for name, layer in module.named_modules():
                if not isinstance(layer, nn.Linear) or name.split(".")[-1] not in self.names:
                    continue
                seed = layer_seed(name, self.seed)
                block = self.block if self.block and layer.in_features % self.block == 0 and layer.in_features > self.block else None
                layer.weight.copy_(rht(layer.weight.float(), seed=seed, block=block).to(layer.weight.dtype))
                descriptor = {"kind": "rotation", "name": name, "seed": seed}
                if block is not None:
                    descriptor["block"] = block
                install_transform(module, descriptor)
                record_transform(module, descriptor)


def rotate(seed: int = 0, names: tuple[str, ...] = ROTATED_LAYER_NAMES, block: int | None = None) -> Rotate:
    return Rotate(seed, tuple(names), block)
