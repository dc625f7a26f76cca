"""Named decoders: checkpoints and ``Q`` objects refer to a decoder by name.

Mirrors, in /root/reference/src/mlkit/quantization/codecs:
  registry.py:1-46        codec, decoder, registered, row_parameters
  scaled.py:19-101        decode_grouped, decode_scaled ("scaled"), decode_feedback ("feedback")
  scaled.py:104-128       decode_vector_scaled ("vector_scaled", "vector_feedback")
  composition.py:14-20    deterministic_signs
  composition.py:23-47    decode_basis ("basis")      composition.py:61-84   compose
  composition.py:87-116   concatenate_rows
Decoding uint8 codes with FP32 parameters on a HIP device runs ``mk_scalar_decode``; tensors
that track gradients, or live on the host, use the same expression in tensor operations.
"""

from collections.abc import Callable, Sequence
from typing import Any

import torch
from torch import Tensor

from mlkit_amd.quantization.core import Q

_DECODERS: dict[str, Callable[..., Tensor]] = {}
_ROW_PARAMETERS: dict[str, tuple[str, ...]] = {}


def codec(name: str, *, row_parameters: tuple[str, ...] | None = None) -> Callable[[Callable], Callable]:
    """Register ``function(codes, **params) -> Tensor`` under ``name``.

    ``row_parameters`` names the parameters holding one entry per weight row; declaring
    them lets row chunks of one matrix be joined (``concatenate_rows``).
    """
    def register(function: Callable[..., Tensor]) -> Callable[..., Tensor]:
        if not name or name in _DECODERS:
            raise ValueError(f"codec name {name!r} is empty or already registered")
        _DECODERS[name] = function
        if row_parameters is not None:
            _ROW_PARAMETERS[name] = tuple(row_parameters)
        return function

    return register


def decoder(name: str) -> Callable[..., Tensor]:
    try:
        return _DECODERS[name]
    except KeyError:
        raise ValueError(f"checkpoint requires registered codec {name!r}") from None


def registered(name: str | None) -> bool:
    return name in _DECODERS


def row_parameters(name: str | None) -> tuple[str, ...] | None:
    return None if name is None else _ROW_PARAMETERS.get(name)


def _tracked(*tensors: Tensor | None) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def _kernel_ready(codes: Tensor, scales: Tensor, values: Tensor, zero: Tensor | None) -> bool:
    return (codes.is_cuda and codes.dtype == torch.uint8 and codes.dim() == 2 and codes.is_contiguous()
            and scales.dtype == torch.float32 and values.dtype == torch.float32 and values.numel() <= 256
            and (zero is None or zero.dtype == torch.float32) and not _tracked(scales, values, zero))


def _expand(codes: Tensor, values: Tensor, scales: Tensor, zero: Tensor | None, index: Tensor) -> Tensor:
    out = values[codes.int()] * scales[:, index]
    return out if zero is None else out + zero[:, index]


def decode_grouped(codes: Tensor, scales: Tensor, values: Tensor, group: int, zero: Tensor | None) -> Tensor:
    """``values[codes] * scales[:, c // group] (+ zero[:, c // group])`` as FP32."""
    if _kernel_ready(codes, scales, values, zero):
        from mlkit_amd.kernels import scalar_decode

        return scalar_decode.decode(codes, scales.contiguous(), values.contiguous(),
                                    None if zero is None else zero.contiguous(), group)
    index = torch.arange(codes.shape[1], device=codes.device) // group
    return _expand(codes, values, scales, zero, index)


@codec("scaled", row_parameters=("scales", "zero"))
def decode_scaled(codes: Tensor, *, scales: Tensor, values: Tensor, group: int, offset: int = 0,
                  zero: Tensor | None = None) -> Tensor:
    if offset == 0:
        return decode_grouped(codes, scales, values, group, zero)
    index = torch.arange(offset, offset + codes.shape[1], device=codes.device) // group
    return _expand(codes, values, scales, zero, index)


@codec("feedback", row_parameters=("scales", "zero"))
def decode_feedback(codes: Tensor, *, scales: Tensor, values: Tensor, group: int, refit: int,
                    zero: Tensor | None = None, permutation: Tensor | None = None) -> Tensor:
    """Codes of an error-feedback sweep: scales are laid out region by region of ``refit``
    columns, ``ceil(refit / group)`` per region."""
    if refit % group == 0:
        out = decode_grouped(codes, scales, values, group, zero)
    elif _kernel_ready(codes, scales, values, zero):
        from mlkit_amd.kernels import scalar_decode

        out = scalar_decode.decode(codes, scales.contiguous(), values.contiguous(),
                                   None if zero is None else zero.contiguous(), group, refit=refit)
    else:
        columns = torch.arange(codes.shape[1], device=codes.device)
        index = (columns // refit) * (-(-refit // group)) + (columns % refit) // group
        out = _expand(codes, values, scales, zero, index)
    return out if permutation is None else out[:, permutation.argsort()]


@codec("vector_feedback", row_parameters=("scales", "zero"))
@codec("vector_scaled", row_parameters=("scales", "zero"))
def decode_vector_scaled(codes: Tensor, *, scales: Tensor, values: Tensor | None, group: int, dim: int,
                         offset: int = 0, zero: Tensor | None = None, refit: int | None = None,
                         permutation: Tensor | None = None) -> Tensor:
    """One code per block of ``dim`` columns: the codeword (a row of ``values``, or the E8P
    point of the code when ``values`` is None) laid out along the row, times the scale of each
    column's group; groups restart at every ``refit`` columns."""
    if values is None:
        from mlkit_amd.quantization.lattice import device_points

        values = device_points(codes.device)
    width = codes.shape[1] * dim
    columns = torch.arange(offset, offset + width, device=codes.device)
    index = columns // group if refit is None else (columns // refit) * (-(-refit // group)) + (columns % refit) // group
    out = values[codes.int()].reshape(codes.shape[0], width) * scales[:, index]
    if zero is not None:
        out = out + zero[:, index]
    return out if permutation is None else out[:, permutation.argsort()]


def deterministic_signs(width: int, seed: int, device: torch.device | str) -> Tensor:
    """Rademacher signs from an integer hash of ``index + seed``: identical on every device."""
    v = (torch.arange(width, device=device, dtype=torch.int64) + seed) & 0xFFFFFFFF
    for _ in range(2):
        v = ((v ^ (v >> 16)) * 0x45D9F3B) & 0xFFFFFFFF
    v = v ^ (v >> 16)
    return (v & 1).float() * 2 - 1


@codec("basis")
def decode_basis(codes: Tensor, *, inner_codec: str, shape: "tuple[int, int] | list[int]", left_seed: int | None,
                 right_seed: int | None, left_signs: Tensor | None, right_signs: Tensor | None,
                 **parameters: Any) -> Tensor:
    """Codes of a matrix quantized in a rotated basis: the inner decoder's reconstruction is
    rotated back, input side (columns) first, then output side (rows)."""
    from mlkit_amd.quantization.transforms import rotate

    inner = {key.removeprefix("inner_"): value for key, value in parameters.items()}
    restored = decoder(inner_codec)(codes, **inner)
    if right_seed is not None:
        signs = right_signs if right_signs is not None else deterministic_signs(shape[1], right_seed, codes.device)
        restored = rotate(restored, inverse=True, signs=signs)
    if left_seed is not None:
        signs = left_signs if left_signs is not None else deterministic_signs(shape[0], left_seed, codes.device)
        restored = rotate(restored.T.contiguous(), inverse=True, signs=signs).T
    return restored


def compose(quantized: Q, name: str, parameters: dict[str, Any]) -> Q:
    """Wrap a portable inner representation in the decoder ``name``; the inner codec's
    parameters travel with an ``inner_`` prefix."""
    if quantized.codes is None or quantized.codec is None or not registered(quantized.codec):
        raise ValueError("portable composition requires a registered inner codec")
    metadata = dict(quantized.metadata)
    metadata["trainable"] = [f"inner_{key}" for key in metadata.get("trainable", [])]
    formats = dict(metadata.get("parameter_formats", {}))
    if quantized.codec in {"scaled", "feedback", "vector_scaled", "vector_feedback"}:
        formats["scales"] = formats["zero"] = metadata.get("scale_fmt", "fp32")
    metadata["parameter_formats"] = {f"inner_{key}": value for key, value in formats.items()}
    metadata["parameter_bits"] = {f"inner_{key}": value for key, value in metadata.get("parameter_bits", {}).items()}
    inner = {f"inner_{key}": value for key, value in quantized.params.items()}
    return Q(codes=quantized.codes, params={**inner, "inner_codec": quantized.codec, **parameters},
             decode=decoder(name), codec=name, bits=quantized.bits, metadata=metadata)


def concatenate_rows(parts: Sequence[Q]) -> Q:
    """Join the representations of consecutive row chunks of one matrix."""
    head = parts[0]
    known = [part.bits for part in parts if part.bits is not None]
    bits = sum(known) if len(known) == len(parts) else None
    if any(part.codes is None for part in parts):
        return Q(torch.cat([part.w for part in parts]), bits=bits)
    per_row = row_parameters(head.codec)
    if per_row is None:
        raise ValueError(
            f"codec {head.codec!r} does not declare row parameters, so a row-separable "
            "quantizer cannot use it; register it with mk.codec(name, row_parameters=...)")
    params = dict(head.params)
    for key in per_row:
        if isinstance(head.params.get(key), Tensor):
            params[key] = torch.cat([part.params[key] for part in parts])
    return Q(codes=torch.cat([part.codes for part in parts]), params=params, decode=head.decode,
             codec=head.codec, bits=bits, metadata=head.metadata)
