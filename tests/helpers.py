"""Shared builders for the parity tests: seeded synthetic layers quantised by the oracle."""

import concurrent.futures
import os

import numpy as np
import torch

from oracle import bitstream, scaling

F32 = np.float32


def normal_weight(rows, width, seed, scale=0.02, outlier_fraction=0.0, student_t=False):
    """fp16-rounded weights: N(0, scale^2), optional x20 outlier columns or Student-t(5)."""
    generator = torch.Generator().manual_seed(seed)
    weight = torch.randn(rows, width, generator=generator)
    if student_t:
        chi = torch.randn(5, rows, width, generator=generator).square().sum(0) / 5
        weight = weight / chi.sqrt()
    weight = weight * scale
    if outlier_fraction:
        count = max(1, round(outlier_fraction * width))
        columns = torch.randperm(width, generator=generator)[:count]
        weight[:, columns] *= 20
    return weight.half().float().numpy()


def activations(samples, width, seed, dtype=torch.float16):
    generator = torch.Generator().manual_seed(seed)
    return torch.randn(samples, width, generator=generator).to(dtype)


def _quantize_by_row_bands(weight, values, **options):
    """scaling.quantize, with large matrices cut into row bands that run on a thread pool (the
    codec is row-separable and numpy releases the interpreter lock inside its loops)."""
    rows = weight.shape[0]
    if weight.size < (1 << 22):
        return scaling.quantize(weight, values, **options)
    workers = min(16, os.cpu_count() or 1)
    bands = np.array_split(np.arange(rows), min(rows, 4 * workers))
    with concurrent.futures.ThreadPoolExecutor(workers) as pool:
        parts = list(pool.map(lambda band: scaling.quantize(weight[band[0]:band[-1] + 1], values, **options), bands))
    result = dict(parts[0])
    for key in ("codes", "scales", "zero"):
        result[key] = None if parts[0][key] is None else np.concatenate([part[key] for part in parts], 0)
    result["side_bits"] = sum(part["side_bits"] for part in parts)
    return result


def quantised_layer(weight, values, *, bits, group, integer, asym=False, scale="absmax", fmt="fp16"):
    """Oracle quantisation + packing.  Returns a dict of numpy arrays."""
    result = _quantize_by_row_bands(weight, values, group=group, integer=integer, asym=asym,
                                    scale=scale, fmt=fmt)
    result["packed"] = bitstream.pack(result["codes"], bits)
    result["bits"] = bits
    result["shape"] = weight.shape
    result["dense"] = scaling.decode_grouped(result["codes"], result["scales"], result["values"],
                                             result["group"], result["zero"])
    return result


def to_device(layer, scale_dtype=torch.float16, device="cuda"):
    """Device tensors of a quantised layer in the dtypes PackedLinear keeps them in."""
    out = {
        "packed": torch.from_numpy(layer["packed"]).to(device),
        "scales": torch.from_numpy(layer["scales"]).to(device=device, dtype=scale_dtype),
        "values": torch.from_numpy(np.asarray(layer["values"], dtype=F32)).to(device),
        "zeros": None,
    }
    if layer["zero"] is not None:
        out["zeros"] = torch.from_numpy(layer["zero"]).to(device=device, dtype=scale_dtype)
    return out


def uniform_grid(values):
    """(is_uniform, minimum, step) the way PackedLinear derives it (inference/packed_linear.py:90-97)."""
    values = torch.as_tensor(np.asarray(values, dtype=F32))
    steps = values.diff()
    uniform = bool(len(steps) and torch.allclose(steps, steps[0].expand_as(steps)))
    return uniform, float(values[0]), float(steps[0]) if len(steps) else 1.0


ROTATED_NEAR_TIE_FRACTION = 0.02


def check_rotated_layer(y, layer, device_rotated, oracle_rotated, dtype, bias=None):
    """A rotated layer's output against the oracle, in two parts that together say what a single looser
    output tolerance would blur:

    * the matvec: ``y`` against the float64 product of the dense reconstruction with the activations the
      DEVICE rotated (already rounded to ``dtype``), at the unrotated layers' tolerance: 1e-3 of the output
      range for fp16, 8e-3 for bf16;
    * the rotation: the device's rounded activations against the oracle's rotated activations rounded the same
      way.  They are the same sums (in another order for the row-rotation kernel): no value may differ by more
      than one unit in the last place of ``dtype`` (plus the fp32 summation noise, 1e-5 of the row's largest
      value, which matters for values near zero only), and at most ROTATED_NEAR_TIE_FRACTION of them may
      differ at all (values whose exact sum lies next to a rounding boundary).

    Returns ``(output error, fraction of differing activations)``."""
    from oracle import matvec as oracle_matvec

    device_rotated = device_rotated.detach().float().cpu()
    rounded_oracle = torch.as_tensor(np.asarray(oracle_rotated, dtype=F32)).to(dtype).float()
    reference = oracle_matvec.reconstruct_then_matmul_f64(
        device_rotated.numpy(), layer["dense"], None if bias is None else bias.float().cpu().numpy())
    error = np.abs(np.asarray(y, dtype=np.float64) - reference).max() / np.abs(reference).max()
    bound = 1e-3 if dtype == torch.float16 else 8e-3
    assert error <= bound, f"max error {error:.3e} of the output range"
    mantissa = 10 if dtype == torch.float16 else 7
    smallest = -14 if dtype == torch.float16 else -126
    magnitude = torch.maximum(device_rotated.abs(), rounded_oracle.abs()).clamp_min(2.0 ** smallest)
    unit = torch.exp2(torch.floor(torch.log2(magnitude)) - mantissa)
    difference = (device_rotated - rounded_oracle).abs()
    # before rounding the two fp32 sums agree to 1e-5 of the row's largest value, which for values near zero is more
    # than their own unit in the last place
    noise = 1e-5 * rounded_oracle.abs().amax(dim=-1, keepdim=True)
    assert bool((difference <= unit + noise).all()), "a rotated activation is more than one unit in the last place away"
    fraction = float((difference > 0).float().mean())
    assert fraction <= ROTATED_NEAR_TIE_FRACTION, f"{fraction:.4f} of the rotated activations differ"
    return error, fraction
