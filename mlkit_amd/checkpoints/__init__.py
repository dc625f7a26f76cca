"""Tensor-only checkpoints: ``mlkit.json`` beside ``weights.safetensors``."""

from mlkit_amd.checkpoints.layout import FORMAT_VERSION, MANIFEST_FILE, WEIGHTS_FILE, load_checkpoint, save

__all__ = ["FORMAT_VERSION", "MANIFEST_FILE", "WEIGHTS_FILE", "load_checkpoint", "save"]
