"""The E8P lattice codebook of QuIP# and its nearest-point search.

The point set: 256 magnitude patterns over {1/2, 3/2, 5/2}^8 -- the 227 of squared norm at
most 10 in lexicographic order, then 29 of squared norm 12 listed by bit mask -- each with
128 sign choices for its first seven coordinates and the eighth sign fixed by parity, in the
two cosets shifted by +1/4 and -1/4: 65,536 points.  ``code = pattern * 128 + sign bits``,
plus 32768 for the -1/4 coset.

Mirrors /root/reference/src/mlkit/quantization/grids/lattice.py (:15-39 the point set,
:42-52 per-device tables, :55-109 nearest_e8p).  On a HIP device the search is
``mk_vector_nearest``; host tensors, and ``backend="torch"``, take the same structured search
in tensor operations.
"""

import functools
import itertools

import torch
from torch import Tensor

NORM_TWELVE_MASKS = (
    241, 242, 244, 248, 55, 87, 103, 151, 167, 199, 59, 91, 107, 155, 171, 203, 61, 93, 109, 157, 173,
    206, 62, 94, 110, 158, 174, 236, 115,
)
COSETS = ((32768, -0.25), (0, 0.25))  # (code offset, shift), in the order ties are resolved


@functools.lru_cache(maxsize=1)
def absolute_points() -> Tensor:
    """[256, 8]: the magnitude patterns."""
    inside = [p for p in itertools.product((0.5, 1.5, 2.5), repeat=8) if sum(c * c for c in p) <= 10]
    edge = [[0.5 + ((mask >> axis) & 1) for axis in range(8)] for mask in NORM_TWELVE_MASKS]
    return torch.tensor(inside + edge, dtype=torch.float32)


@functools.lru_cache(maxsize=1)
def e8p_points() -> Tensor:
    """[65536, 8]: the point of every code."""
    patterns = absolute_points()
    choice = torch.arange(128)
    bits = (choice[:, None] >> torch.arange(7)) & 1                                    # [128, 7]
    eighth = (bits.sum(1)[None, :] + patterns.sum(1).long()[:, None]) & 1              # [256, 128]
    negative = torch.cat((bits.expand(256, 128, 7), eighth[..., None]), dim=2)
    signed = (patterns[:, None, :] * (1 - 2 * negative)).reshape(32768, 8)
    return torch.cat((signed + 0.25, signed - 0.25))


@functools.lru_cache(maxsize=8)
def device_points(device: torch.device, *, absolute: bool = False) -> Tensor:
    return (absolute_points() if absolute else e8p_points()).to(device)


@functools.lru_cache(maxsize=8)
def device_table(device: torch.device) -> Tensor:
    """The 65,536 points followed by the 256 magnitude patterns that generate them."""
    return torch.cat((e8p_points(), absolute_points())).to(device).contiguous()


def _structured_codes(samples: Tensor) -> Tensor:
    """Codes (int64) of the nearest points of ``samples[n, 8]`` in tensor operations: per coset,
    every pattern is scored against |v - shift|; a pattern whose parity disagrees with the
    number of negative coordinates pays for flipping its cheapest one."""
    patterns = device_points(samples.device, absolute=True)
    norms, parity = patterns.square().sum(1), patterns.sum(1).long() & 1
    weights = 1 << torch.arange(7, device=samples.device)
    count = samples.shape[0]
    best = torch.full((count,), float("inf"), device=samples.device)
    codes = torch.zeros(count, dtype=torch.long, device=samples.device)
    picked = torch.arange(count, device=samples.device)
    for offset, shift in COSETS:
        centered = samples - shift
        negative = centered < 0
        products = centered.abs()[:, None, :] * patterns                               # [n, 256, 8]
        flip_cost, flip_axis = products.min(2)
        odd = parity[None, :] != (negative.sum(1) & 1)[:, None]
        costs = centered.square().sum(1, keepdim=True) + norms - 2 * products.sum(2) + 4 * flip_cost * odd
        cost, pattern = costs.min(1)
        flipped = negative.clone()
        flipped[picked, flip_axis[picked, pattern]] ^= odd[picked, pattern]
        code = pattern * 128 + (flipped[:, :7] * weights).sum(1) + offset
        codes = torch.where(cost < best, code, codes)
        best = torch.minimum(best, cost)
    return codes


def nearest_e8p(value: Tensor, *, chunk: int = 512, return_indices: bool = False, backend: str = "auto") -> Tensor:
    """The nearest E8P point of every ``value[..., 8]`` (or its code)."""
    if value.shape[-1] != 8 or chunk < 1:
        raise ValueError("E8P quantization requires eight-dimensional vectors and positive chunk size")
    if backend not in {"auto", "torch", "hip", "triton"}:
        raise ValueError("E8P backend must be auto, torch or hip")
    if value.is_cuda and backend != "torch":
        from mlkit_amd.kernels import lattice_search

        codes = lattice_search.search(value, device_table(value.device))
        return codes if return_indices else device_points(value.device)[codes.long()].to(value.dtype)
    if backend in {"hip", "triton"}:
        raise ValueError("fused E8P requires a HIP device")
    parts = [_structured_codes(part) for part in value.reshape(-1, 8).float().split(chunk)]
    codes = torch.cat(parts) if parts else torch.empty(0, dtype=torch.long, device=value.device)
    if return_indices:
        return codes.reshape(value.shape[:-1])
    return device_points(value.device)[codes].reshape(value.shape).to(value.dtype)
