"""ctypes binding of ``libmlkit_amd.so`` (the C ABI declared in ``include/mlkit_amd.h``).

The library is loaded on first use and a missing library is an error, never a silent
switch to another implementation: every fused path of this package runs a HIP kernel
or raises.  Build it with ``python -m mlkit_amd.build`` (hipcc, gfx950).
"""

import ctypes
import os
import pathlib
from typing import Any

import torch
from torch import Tensor

# MLKIT_AMD_LIBRARY selects another build of the same library (e.g. a profiling build).
LIBRARY_PATH = pathlib.Path(
    os.environ.get("MLKIT_AMD_LIBRARY") or pathlib.Path(__file__).resolve().parent / "libmlkit_amd.so"
)

MK_F32, MK_F16, MK_BF16 = 0, 1, 2
DTYPE_CODES = {torch.float32: MK_F32, torch.float16: MK_F16, torch.bfloat16: MK_BF16}

MK_ERR_INVALID, MK_ERR_UNSUPPORTED, MK_ERR_HIP = 1, 2, 3

_c_int, _c_float, _c_void_p, _c_longlong = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong

SCALE_FORMAT_CODES = {"fp32": 0, "fp16": 1, "bf16": 2, "fp8": 3, "e8m0": 4}

# name -> (restype, argtypes); mirrors include/mlkit_amd.h declaration by declaration.
SIGNATURES: dict[str, tuple[Any, list[Any]]] = {
    "mk_version": (ctypes.c_char_p, []),
    "mk_last_error": (ctypes.c_char_p, []),
    "mk_packed_layout_supported": (_c_int, [_c_int, _c_int, _c_int]),
    "mk_packed_matvec": (_c_int, [
        _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p,
        _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
        _c_float, _c_float, _c_void_p,
    ]),
    "mk_packed_matvec_group": (_c_int, [
        _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int,
        _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p,
    ]),
    "mk_rotated_packed_matvec": (_c_int, [
        _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_float,
        _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p,
    ]),
    "mk_rotated_packed_matvec_static": (_c_int, [
        _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_float,
        _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p,
    ]),
    "mk_packed_decode": (_c_int, [
        _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p,
    ]),
    "mk_packed_decode_rows": (_c_int, [
        _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p,
    ]),
    "mk_pack": (_c_int, [_c_void_p, _c_int, _c_longlong, _c_int, _c_void_p, _c_void_p, _c_void_p]),
    "mk_unpack": (_c_int, [_c_void_p, _c_longlong, _c_int, _c_void_p, _c_void_p]),
    "mk_scalar_encode": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int,
        _c_int, _c_int, _c_float, _c_float, _c_void_p,
    ]),
    "mk_scalar_decode": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
        _c_int, _c_int, _c_void_p,
    ]),
    "mk_search_scales": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_int,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p,
    ]),
    "mk_snap": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_longlong, _c_void_p]),
    "mk_fit_scales": (_c_int, [
        _c_void_p, _c_longlong, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_float,
        _c_float, _c_int, _c_int, _c_void_p,
    ]),
    "mk_reconstruct_activations": (_c_int, [
        _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
        _c_float, _c_float, _c_float, _c_void_p,
    ]),
    "mk_fwht": (_c_int, [
        _c_void_p, _c_int, _c_void_p, _c_int, _c_longlong, _c_int, _c_void_p, _c_void_p, _c_int,
        _c_float, _c_void_p,
    ]),
    "mk_cholesky_block": (_c_int, [_c_void_p, _c_longlong, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p]),
    "mk_rotate_blocks": (_c_int, [
        _c_void_p, _c_int, _c_void_p, _c_int, _c_longlong, _c_int, _c_int, _c_void_p, _c_int, _c_void_p,
        _c_void_p, _c_float, _c_void_p,
    ]),
    "mk_rotate_rows": (_c_int, [
        _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_float, _c_void_p,
    ]),
    "mk_basis_mix": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_longlong, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
    ]),
    "mk_feedback_round_tile": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
        _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
        _c_float, _c_void_p,
    ]),
    "mk_feedback_pending": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p,
    ]),
    "mk_feedback_block_update": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p,
    ]),
    "mk_feedback_sweep": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
        _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_int, _c_float,
        _c_float, _c_int, _c_int, _c_void_p,
    ]),
    "mk_feedback_block_update_staged": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p,
    ]),
    "mk_feedback_block_update_range": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
        _c_int, _c_void_p,
    ]),
    "mk_hessian_reversed": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p]),
    "mk_unit_upper_from_factor": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_void_p]),
    "mk_vector_nearest": (_c_int, [
        _c_void_p, _c_longlong, _c_int, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
    ]),
    "mk_feedback_round_vector_tile": (_c_int, [
        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p,
    ]),
}

_library: ctypes.CDLL | None = None


class NativeLibraryMissing(RuntimeError):
    """The HIP extension has not been built; there is no other implementation to fall back on."""


def available() -> bool:
    return LIBRARY_PATH.exists()


def library() -> ctypes.CDLL:
    """The loaded library with typed entry points; raises if it has not been built."""
    global _library
    if _library is None:
        if not LIBRARY_PATH.exists():
            raise NativeLibraryMissing(
                f"{LIBRARY_PATH} is missing: build the gfx950 kernels with "
                "`python -m mlkit_amd.build`; mlkit_amd has no fallback for its fused paths"
            )
        loaded = ctypes.CDLL(str(LIBRARY_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            function = getattr(loaded, name)
            function.restype = restype
            function.argtypes = argtypes
        _library = loaded
    return _library


def last_error() -> str:
    return library().mk_last_error().decode()


def check(status: int) -> None:
    """Map a nonzero status to the exception type the reference raises for that failure."""
    if status == 0:
        return
    message = last_error()
    if status == MK_ERR_HIP:
        raise RuntimeError(message)
    raise ValueError(message)


def pointer(tensor: Tensor | None) -> int | None:
    return None if tensor is None else tensor.data_ptr()


def dtype_code(tensor: Tensor) -> int:
    try:
        return DTYPE_CODES[tensor.dtype]
    except KeyError:
        raise ValueError(f"unsupported tensor dtype {tensor.dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device: torch.device) -> int:
    """The raw handle of the device's current stream (a plain C call where torch offers one:
    building a ``torch.cuda.Stream`` object costs several microseconds per launch)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def require_device(*tensors: Tensor | None) -> torch.device:
    """All given tensors must live on one CUDA (HIP) device; returns it."""
    device = None
    for tensor in tensors:
        if tensor is None:
            continue
        if not tensor.is_cuda:
            raise ValueError("fused kernels require CUDA tensors")
        if device is None:
            device = tensor.device
        elif tensor.device != device:
            raise ValueError("fused kernels require all tensors on one device")
    assert device is not None
    return device
