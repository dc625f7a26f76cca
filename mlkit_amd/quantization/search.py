"""Nearest-entry search over scalar and vector codebooks.

``snap`` (ascending scalar codebook, ties choose the lower entry) has the call surface of the
reference's /root/reference/src/mlkit/quantization/operations/search.py:9-27; FP32 HIP tensors
run ``mk_snap``.  Tensors that track gradients, other dtypes and host tensors use the
bisection in tensor operations, which is the same rule the kernel implements.

``nearest`` (operations/search.py:34-79) searches a codebook of vectors exhaustively: HIP
tensors with 2, 4, 8 or 16 coordinates run ``mk_vector_nearest``; anything else compares
squared distances in tensor operations, a bounded tile of them at a time.  One-coordinate
codebooks go to ``nearest_scalar`` (operations/search.py:82-98).
"""

import torch
from torch import Tensor


def nearest_indices(value: Tensor, table: Tensor) -> Tensor:
    """Index of the nearest entry of the ascending ``table``; equal distances pick the lower."""
    upper = torch.searchsorted(table, value.contiguous()).clamp_max(table.numel() - 1)
    lower = (upper - 1).clamp_min(0)
    take_lower = (value - table[lower]).abs() <= (value - table[upper]).abs()
    return torch.where(take_lower, lower, upper)


def snap(value: Tensor, codebook: Tensor) -> Tensor:
    table = codebook.to(device=value.device, dtype=value.dtype).flatten().sort().values
    if table.numel() == 0:
        raise ValueError("codebook cannot be empty")
    tracked = torch.is_grad_enabled() and (value.requires_grad or table.requires_grad)
    if value.is_cuda and value.dtype == torch.float32 and not tracked and value.numel() and table.numel() <= 256:
        from mlkit_amd.kernels import scalar_encode

        return scalar_encode.snap(value.contiguous(), table)
    return table[nearest_indices(value, table)]


DISTANCE_BUDGET = 1 << 23  # distances held at once by the tensor-operation search (32 MiB of FP32)


def nearest_scalar(value: Tensor, codebook: Tensor) -> Tensor:
    """Index into the (unsorted) scalar ``codebook`` of the entry nearest to each value; among
    equally near entries, and among duplicates, the lowest index."""
    ordered, origin = codebook.float().sort(stable=True)
    first = origin[torch.searchsorted(ordered, ordered)]  # duplicates answer with their first occurrence
    samples = value.float().contiguous()
    above = torch.searchsorted(ordered, samples).clamp_max(ordered.numel() - 1)
    below = (above - 1).clamp_min(0)
    gap_below, gap_above = (samples - ordered[below]).abs(), (samples - ordered[above]).abs()
    prefer_below = (gap_below < gap_above) | ((gap_below == gap_above) & (first[below] < first[above]))
    return torch.where(prefer_below, first[below], first[above])


def nearest(value: Tensor, codebook: Tensor, *, chunk: int | None = None, codebook_chunk: int = 4096,
            return_indices: bool = False) -> Tensor:
    """The codeword of ``codebook[entries, dim]`` nearest to each row of ``value[n, dim]`` (or
    its index, int64); the lowest index among equally near codewords."""
    if value.ndim != 2 or codebook.ndim != 2 or value.shape[1] != codebook.shape[1]:
        raise ValueError("value and codebook must be matrices with equal vector dimensions")
    if not codebook.shape[0] or codebook_chunk <= 0 or (chunk is not None and chunk <= 0):
        raise ValueError("codebook and chunk sizes must be nonempty and positive")
    codebook = codebook.to(value.device)
    dimension = codebook.shape[1]
    if dimension == 1:
        indices = nearest_scalar(value[:, 0], codebook[:, 0])
    elif value.is_cuda and dimension in (2, 4, 8, 16):
        from mlkit_amd.kernels import lattice_search

        indices = lattice_search.nearest(value, codebook).long()
    else:
        entries = codebook.float()
        rows = chunk or max(1, DISTANCE_BUDGET // min(codebook_chunk, entries.shape[0]))
        found = []
        for samples in value.float().split(rows):
            best = torch.full((samples.shape[0],), float("inf"), device=value.device)
            index = torch.zeros(samples.shape[0], dtype=torch.long, device=value.device)
            for start in range(0, entries.shape[0], codebook_chunk):
                distances = (entries[None, start:start + codebook_chunk] - samples[:, None]).square().sum(2)
                cost, local = distances.min(1)
                index = torch.where(cost < best, local + start, index)
                best = torch.minimum(best, cost)
            found.append(index)
        indices = torch.cat(found) if found else torch.empty(0, dtype=torch.long, device=value.device)
    return indices if return_indices else codebook[indices].to(value.dtype)
