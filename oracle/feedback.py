"""Oracle (test infrastructure): LDL-form GPTQ / LDLQ error feedback on the CPU.

Follows, in the reference:
  algorithms/error_feedback.py:37-83     feedback_coefficients (step 1)       -> coefficients
  algorithms/error_feedback.py:266-371   ErrorFeedback.__call__               -> sweep
  algorithms/error_feedback.py:373-393   _pending_continuation                -> pending
  kernels/error_feedback.py:22-96        round_feedback_tile (arithmetic)     -> round_tile
  operations/losses.py:9-15              proxy_loss

Arithmetic form (kernels/error_feedback.py:60,88,94): ``target = weight + correction``;
the deviation ``weight - reconstruction`` is measured against the *original* weight and
is pushed to later columns of the tile by separate multiply and add.

Two places have no order fixed by the reference (its torch calls leave it to the BLAS):
the trailing block update (``addmm_``) and the triangular solve of the pending
continuation.  This oracle fixes them -- fmaf over ascending k from zero, then one add;
right-looking forward substitution -- and the HIP kernels follow the same orders.
Against the reference's own torch backend these two bit-level orders are *parity
unpinned* (the reference asserts its own backends against each other at rtol 1e-5).
Everything else of ``sweep`` -- including the region refits (pending continuation,
targets, scale fit) -- is pinned by the float64 textbook loops of
tests/test_oracle_feedback.py.

The sequential pieces run in C (``csrc/gptq_ref.c``); ``round_tile_numpy`` is the same
tile arithmetic in numpy and pins the C against a second implementation.
"""

import ctypes
import pathlib
import subprocess

import numpy as np

from . import scaling

F32 = np.float32
_HERE = pathlib.Path(__file__).resolve().parent
_LIB = None


def build(force: bool = False) -> pathlib.Path:
    """Compile ``libmk_oracle.so`` with gcc if it is missing (or ``force``)."""
    target = _HERE / "libmk_oracle.so"
    if force or not target.exists():
        subprocess.run(["make", "-C", str(_HERE), "-B" if force else "-s", "libmk_oracle.so"],
                       check=True, capture_output=True)
    return target


def _lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(str(build()))
    return _LIB


def _p(array, kind=ctypes.c_float):
    return None if array is None else array.ctypes.data_as(ctypes.POINTER(kind))


def coefficients(hessian: np.ndarray, damp: float = 0.01) -> tuple[np.ndarray, int]:
    """Unit upper-triangular ``A = R diag(R)^-1`` of the damped ``H = R R^T`` (step 1).

    Cholesky of the index-reversed damped Hessian, columns divided by the diagonal,
    reversed back.  Returns ``(A, status)``; a nonzero status reports an indefinite H.
    """
    reversed_h = np.array(hessian[::-1, ::-1], dtype=F32)
    diagonal = np.diagonal(reversed_h).copy()
    diagonal[diagonal == 0] = 1
    diagonal = diagonal + F32(damp) * np.maximum(diagonal.mean(dtype=F32), F32(1e-12))
    np.fill_diagonal(reversed_h, diagonal)
    try:
        lower = np.linalg.cholesky(reversed_h).astype(F32)
    except np.linalg.LinAlgError:
        return reversed_h, 1
    lower = lower / np.diagonal(lower)[None, :]
    return np.ascontiguousarray(lower[::-1, ::-1], dtype=F32), 0


def pending(feedback: np.ndarray, coeff: np.ndarray, start: int, stop: int) -> np.ndarray:
    rows, width = feedback.shape
    out = np.empty((rows, stop - start), dtype=F32)
    _lib().mk_ref_pending(_p(feedback), _p(coeff), _p(out), rows, width, start, stop)
    return out


def round_tile(original, feedback, coeff, scales, zeros, values, output, encoded, *,
               region_start, tile_start, tile_width, group, integer) -> None:
    rows, width = original.shape
    values = np.ascontiguousarray(values, dtype=F32)
    _lib().mk_ref_round_tile(
        _p(original), _p(feedback), _p(coeff), _p(scales), _p(zeros), _p(values),
        int(values.size), _p(output), _p(encoded, ctypes.c_uint8), rows, width,
        region_start, tile_start, tile_width, group, scales.shape[1], int(integer),
        ctypes.c_float(float(values.min())), ctypes.c_float(float(values.max())))


def round_tile_numpy(original, feedback, coeff, scales, zeros, values, output, encoded, *,
                     region_start, tile_start, tile_width, group, integer) -> None:
    values = np.asarray(values, dtype=F32)
    corrections = feedback[:, tile_start:tile_start + tile_width].copy()
    low, high = F32(values.min()), F32(values.max())
    for column in range(tile_width):
        position = tile_start + column
        weight = original[:, position]
        target = (weight + corrections[:, column]).astype(F32)
        slot = (position - region_start) // group
        scale = scales[:, slot]
        zero = np.zeros_like(scale) if zeros is None else zeros[:, slot]
        normalized = ((target - zero).astype(F32) / scale).astype(F32)
        if integer:
            code = np.clip(np.rint(normalized), low, high)
            index = code - low
            reconstruction = ((code * scale).astype(F32) + zero).astype(F32)
        else:
            index = np.abs(normalized[:, None] - values[None, :]).argmin(1)
            reconstruction = ((values[index] * scale).astype(F32) + zero).astype(F32)
        deviation = (weight - reconstruction).astype(F32)
        row = coeff[position, tile_start + column + 1: tile_start + tile_width]
        corrections[:, column + 1:] = (
            corrections[:, column + 1:] + (deviation[:, None] * row[None, :]).astype(F32)
        ).astype(F32)
        output[:, position] = reconstruction
        encoded[:, position] = index.astype(np.uint8)


def block_update(feedback, original, output, coeff, tile_start, tile_stop, mode: int = 0) -> None:
    rows, width = original.shape
    _lib().mk_ref_block_update(_p(feedback), _p(original), _p(output), _p(coeff), rows, width,
                               tile_start, tile_stop, mode)


def fit_scales(targets, values, group, asym):
    """fp16-stored scales (and offsets) of a region, C twin of scaling.initial_scales + store."""
    rows, span = targets.shape
    groups = (span + group - 1) // group
    values = np.asarray(values, dtype=F32)
    scales = np.empty((rows, groups), dtype=F32)
    zeros = np.empty((rows, groups), dtype=F32) if asym else None
    if asym:
        reciprocal = scaling.f32_reciprocal(float(values.max()) - float(values.min()))
    else:
        reciprocal = scaling.f32_reciprocal(float(np.abs(values).max()))
    targets = np.ascontiguousarray(targets, dtype=F32)
    _lib().mk_ref_fit_scales(_p(targets), _p(scales), _p(zeros), rows, span, group, int(asym),
                             ctypes.c_float(float(reciprocal)), ctypes.c_float(float(values.min())))
    return scales, zeros


def sweep(weight, coeff, values, *, group, integer, refit=128, block=128, asym=False,
          dead=None, update_mode: int = 0, tile_fn=round_tile) -> dict:
    """Natural-order LDL sweep with fp16 absmax/minmax region refits.

    ``weight`` [N, K], ``coeff`` = unit upper ``A`` [K, K] fp32.  Returns codes (uint8),
    scales/zero concatenated over regions, and the fp32 reconstruction.
    """
    original = np.array(weight, dtype=F32, order="C")   # the C routines index rows of `width` floats
    rows, width = original.shape
    if dead is not None:
        original[:, dead] = 0
    coeff = np.ascontiguousarray(coeff, dtype=F32)
    values = np.ascontiguousarray(values, dtype=F32)
    feedback = np.zeros_like(original)
    output = np.empty_like(original)
    encoded = np.empty(original.shape, dtype=np.uint8)
    refit_width = width if refit is None else refit
    all_scales, all_zeros = [], []
    for region_start in range(0, width, refit_width):
        region_stop = min(width, region_start + refit_width)
        targets = original[:, region_start:region_stop]
        if region_start:
            targets = (targets + pending(feedback, coeff, region_start, region_stop)).astype(F32)
        fitted_group = min(group, region_stop - region_start)
        scales, zeros = fit_scales(targets, values, fitted_group, asym)
        all_scales.append(scales)
        if zeros is not None:
            all_zeros.append(zeros)
        for tile_start in range(region_start, region_stop, block):
            tile_stop = min(region_stop, tile_start + block)
            tile_fn(original, feedback, coeff, scales, zeros, values, output, encoded,
                    region_start=region_start, tile_start=tile_start,
                    tile_width=tile_stop - tile_start, group=fitted_group, integer=integer)
            if tile_stop < width:
                block_update(feedback, original, output, coeff, tile_start, tile_stop, update_mode)
    return {
        "codes": encoded,
        "scales": np.concatenate(all_scales, 1),
        "zero": np.concatenate(all_zeros, 1) if all_zeros else None,
        "w": output,
        "group": group,
        "refit": refit_width,
        "feedback": feedback,
    }


def proxy_loss(weight, reconstruction, hessian) -> float:
    """``tr(E H E^T) / N`` with ``E = W - W_hat`` (operations/losses.py:9-15)."""
    error = np.asarray(weight, dtype=F32) - np.asarray(reconstruction, dtype=F32)
    weighted = error @ np.asarray(hessian, dtype=F32)
    return float(np.vdot(weighted.reshape(-1), error.reshape(-1)) / weight.shape[0])
