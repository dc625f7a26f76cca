"""Integer codes as a little-endian bit stream, and back.

Code ``i`` of width ``b`` occupies stream bits ``[i*b, (i+1)*b)``; byte ``j`` holds stream
bits ``[8j, 8j+8)``, least significant first.  Layout, return types and errors are those of
the reference's ``pack`` / ``unpack`` (/root/reference/src/mlkit/quantization/operations/
bit_packing.py:13-135); the stream is what ``PackedLinear.packed`` and checkpoints hold.

Tensors on a HIP device go through ``mk_pack`` / ``mk_unpack`` (one thread per 32 codes, no
temporaries).  Host tensors are packed as bit planes: the stream *is* the codes' bits laid
end to end, so the codes are spread into one uint8 per bit, regrouped eight at a time and
weighted by powers of two.
"""

import math

import torch
from torch import Tensor

_KERNEL_CODE_BYTES = {torch.uint8: 1, torch.int16: 2, torch.int32: 4, torch.int64: 8}


def _bit_planes(values: Tensor, bits: int) -> Tensor:
    """``[n, bits]`` uint8: bit ``t`` of every value, least significant first."""
    shifts = torch.arange(bits, device=values.device, dtype=torch.int32)
    return ((values.to(torch.int32).unsqueeze(1) >> shifts) & 1).to(torch.uint8)


def pack(codes: Tensor, bits: int, *, overflow: Tensor | None = None) -> Tensor:
    """A flat uint8 tensor of ``ceil(codes.numel() * bits / 8)`` bytes.

    ``overflow`` (device tensors only): a one-element int32 tensor on the codes' device that the
    kernel sets to one when a code does not fit ``bits`` bits.  With it the call does not read
    the flag back (no synchronisation): a caller that packs many tensors hands the same flag to
    all of them and looks at it once (``check_overflow``)."""
    if not 1 <= bits <= 16:
        raise ValueError("packing supports one through sixteen bits")
    if codes.is_floating_point() or codes.is_complex():
        raise TypeError("codes must have an integer dtype")
    flat = codes.detach().reshape(-1)
    count = flat.numel()
    size = (count * bits + 7) // 8
    if flat.is_cuda:
        from mlkit_amd import native

        if flat.dtype not in _KERNEL_CODE_BYTES:
            flat = flat.to(torch.int32)
        flat = flat.contiguous()
        packed = torch.empty(size, dtype=torch.uint8, device=flat.device)
        deferred = overflow is not None
        if deferred:
            if overflow.dtype != torch.int32 or overflow.numel() != 1 or overflow.device != flat.device:
                raise ValueError("overflow must be a one-element int32 tensor on the codes' device")
        elif flat.dtype == torch.uint8 and bits >= 8:
            overflow = None    # every uint8 value fits: nothing to report, nothing to read back
        else:
            overflow = torch.zeros(1, dtype=torch.int32, device=flat.device)
        native.check(native.library().mk_pack(flat.data_ptr(), _KERNEL_CODE_BYTES[flat.dtype], count, bits,
                                              packed.data_ptr(), native.pointer(overflow),
                                              native.current_stream(flat.device)))
        if not deferred and overflow is not None:
            check_overflow(overflow, bits)
        return packed
    if count and (int(flat.min()) < 0 or int(flat.max()) >= 1 << bits):
        raise ValueError(f"codes exceed the unsigned capacity of {bits} bits")
    stream = _bit_planes(flat, bits).reshape(-1)
    if stream.numel() % 8:
        stream = torch.cat([stream, stream.new_zeros(8 - stream.numel() % 8)])
    weights = (1 << torch.arange(8, dtype=torch.int32)).to(torch.uint8)
    return (stream.view(-1, 8) * weights).sum(dim=1, dtype=torch.int32).to(torch.uint8)[:size]


def check_overflow(overflow: Tensor, bits: "int | None" = None) -> None:
    """Raises the error of ``pack`` when a deferred overflow flag is set (reads it back: one synchronisation)."""
    if int(overflow.item()):
        width = "the declared width" if bits is None else f"{bits} bits"
        raise ValueError(f"codes exceed the unsigned capacity of {width}")


def unpack(packed: Tensor, bits: int, shape: tuple[int, ...]) -> Tensor:
    """The codes of a stream as a tensor of ``shape``: uint8 for up to 8 bits, int32 above."""
    if not 1 <= bits <= 16 or packed.dtype != torch.uint8:
        raise ValueError("unpack requires uint8 storage and one through sixteen bits")
    shape = tuple(shape)
    if any(dimension < 0 for dimension in shape):
        raise ValueError("shape dimensions must be nonnegative")
    count = math.prod(shape)
    if packed.numel() != (count * bits + 7) // 8:
        raise ValueError(f"packed byte count {packed.numel()} does not match shape {shape} at {bits} bits")
    code_dtype = torch.uint8 if bits <= 8 else torch.int32
    if packed.is_cuda:
        from mlkit_amd import native

        stream = packed.reshape(-1).contiguous()
        codes = torch.empty(count, dtype=code_dtype, device=packed.device)
        native.check(native.library().mk_unpack(stream.data_ptr(), count, bits, codes.data_ptr(),
                                                native.current_stream(packed.device)))
        return codes.reshape(shape)
    planes = _bit_planes(packed.reshape(-1), 8).reshape(-1)[: count * bits].view(count, bits)
    weights = 1 << torch.arange(bits, dtype=torch.int32)
    return (planes.to(torch.int32) * weights).sum(dim=1, dtype=torch.int32).to(code_dtype).reshape(shape)
