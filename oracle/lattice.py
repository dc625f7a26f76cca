"""Oracle (test infrastructure): vector grids -- the E8P lattice codebook and nearest-codeword
search -- and the LDL error-feedback tile that rounds blocks of ``dimension`` columns.

Follows, in the reference:
  grids/lattice.py:15-39                 absolute_points, e8p_points (E8P as defined in QuIP#)
  grids/lattice.py:53-109, kernels/lattice_search.py:10-45
                                         nearest_e8p / nearest_lattice_code (structured search)
  kernels/error_feedback.py:146-238      round_vector_feedback_tile            -> round_vector_tile
  algorithms/error_feedback.py:296-371   ErrorFeedback.__call__ with a vector region -> vector_sweep
  codecs/scaled.py:106-128               decode_vector_scaled

The E8P point set: 256 magnitude patterns over {1/2, 3/2, 5/2}^8 (the 227 of squared norm
at most 10, in lexicographic order with the first coordinate slowest, then 29 patterns of
squared norm 12 listed by bit mask), each with 128 sign choices for its first seven
coordinates and the eighth sign fixed by parity, shifted by +1/4 and by -1/4: 65,536 points.
Code = pattern * 128 + sign bits (+ 32768 for the -1/4 coset).

Arithmetic the reference leaves to its reductions' order (sums over the 8 coordinates of a
cost, the sum over a block's deviations in the feedback update) is fixed here as: ascending
coordinate, each product rounded on its own.  The reference's own backends agree with each
other on 99 % of codes only (tests/kernels/test_error_feedback.py:104-122), so bit-level
agreement with it on near ties is *parity unpinned*; the search itself is pinned against a
brute force over all 65,536 points.
"""

import functools
import itertools

import numpy as np

F32 = np.float32

# Patterns of squared norm 12 (five coordinates 3/2, three 1/2), bit i set = coordinate i is 3/2.
NORM_TWELVE_MASKS = (
    241, 242, 244, 248, 55, 87, 103, 151, 167, 199, 59, 91, 107, 155, 171, 203, 61, 93, 109, 157, 173,
    206, 62, 94, 110, 158, 174, 236, 115,
)


@functools.lru_cache(maxsize=1)
def absolute_points() -> np.ndarray:
    """[256, 8] fp32 magnitude patterns."""
    interior = [point for point in itertools.product((0.5, 1.5, 2.5), repeat=8) if sum(c * c for c in point) <= 10]
    boundary = [[0.5 + ((mask >> axis) & 1) for axis in range(8)] for mask in NORM_TWELVE_MASKS]
    points = np.array(interior + boundary, dtype=F32)
    assert points.shape == (256, 8)
    return points


@functools.lru_cache(maxsize=1)
def e8p_points() -> np.ndarray:
    """[65536, 8] fp32: point ``code`` of the codebook."""
    magnitudes = absolute_points()
    first = (np.arange(128)[:, None] >> np.arange(7)) & 1                      # [128, 7] sign bits
    last = (first.sum(1)[None, :] + magnitudes.sum(1).astype(np.int64)[:, None]) % 2   # [256, 128]
    signs = np.concatenate([np.broadcast_to(first[None], (256, 128, 7)), last[..., None]], axis=2)
    lattice = (magnitudes[:, None, :] * (1 - 2 * signs)).reshape(-1, 8).astype(F32)
    return np.concatenate([lattice + F32(0.25), lattice - F32(0.25)]).astype(F32)


def nearest_e8p_codes(vectors: np.ndarray) -> np.ndarray:
    """Codes of the nearest E8P points, [n] int32, by the structured search: per coset, every
    magnitude pattern is scored against |v - shift|; a pattern whose sign parity disagrees with
    the input's pays for flipping its cheapest coordinate."""
    vectors = np.asarray(vectors, dtype=F32).reshape(-1, 8)
    patterns = absolute_points()
    norms = np.zeros(256, dtype=F32)
    for axis in range(8):
        norms = (norms + (patterns[:, axis] * patterns[:, axis]).astype(F32)).astype(F32)
    parities = patterns.sum(1).astype(np.int64) & 1
    best_cost = np.full(len(vectors), np.inf, dtype=F32)
    best_code = np.zeros(len(vectors), dtype=np.int64)
    for shift, coset in ((F32(-0.25), 32768), (F32(0.25), 0)):
        centered = (vectors - shift).astype(F32)
        negative = centered < 0
        absolute = np.abs(centered)
        products = (absolute[:, None, :] * patterns[None, :, :]).astype(F32)          # [n, 256, 8]
        correction_axis = products.argmin(2)                                          # first minimum
        correction_cost = products.min(2)
        mismatch = parities[None, :] != (negative.sum(1) & 1)[:, None]
        squares = np.zeros(len(vectors), dtype=F32)
        dots = np.zeros((len(vectors), 256), dtype=F32)
        for axis in range(8):
            squares = (squares + (centered[:, axis] * centered[:, axis]).astype(F32)).astype(F32)
            dots = (dots + products[:, :, axis]).astype(F32)
        costs = ((squares[:, None] + norms[None, :]).astype(F32) - (F32(2) * dots).astype(F32)).astype(F32)
        costs = (costs + (F32(4) * correction_cost * mismatch).astype(F32)).astype(F32)
        index = costs.argmin(1)
        rows = np.arange(len(vectors))
        cost = costs[rows, index]
        flipped = np.where(mismatch[rows, index], correction_axis[rows, index], 8)    # 8: nothing to flip
        sign_code = ((negative[:, :7].astype(np.int64) << np.arange(7)).sum(1)) ^ np.where(flipped < 7, 1 << np.minimum(flipped, 6), 0)
        code = index * 128 + sign_code + coset
        better = cost < best_cost
        best_code = np.where(better, code, best_code)
        best_cost = np.minimum(best_cost, cost)
    return best_code.astype(np.int32)


def nearest_codes(vectors: np.ndarray, codebook: np.ndarray) -> np.ndarray:
    """Index of the nearest codeword by squared distance (differences squared and summed over
    ascending coordinates in fp32), the lowest index on ties."""
    vectors = np.asarray(vectors, dtype=F32)
    codebook = np.asarray(codebook, dtype=F32)
    costs = np.zeros((len(vectors), len(codebook)), dtype=F32)
    for axis in range(codebook.shape[1]):
        difference = (codebook[None, :, axis] - vectors[:, None, axis]).astype(F32)
        costs = (costs + (difference * difference).astype(F32)).astype(F32)
    return costs.argmin(1).astype(np.int32)


def decode_vector_scaled(codes, scales, codebook, group, dimension, refit=None) -> np.ndarray:
    """``codebook[codes]`` laid out along the row, times the column's scale."""
    width = codes.shape[1] * dimension
    columns = np.arange(width)
    slots = columns // group if refit is None else (columns // refit) * (-(-refit // group)) + (columns % refit) // group
    return (np.asarray(codebook, dtype=F32)[codes.astype(np.int64)].reshape(codes.shape[0], width) * scales[:, slots]).astype(F32)


def round_vector_tile(original, feedback, coeff, scales, codebook, output, encoded, *, region_start, tile_start,
                      tile_width, group, dimension, lattice) -> None:
    """Columns [tile_start, tile_start + tile_width) of every row, in blocks of `dimension`:
    target = weight + correction, code of the nearest codeword to target / scale (true division),
    reconstruction = codeword * scale, and the block's deviations times their coefficient rows
    (products rounded one by one, summed over ascending coordinate, then one add) pushed to the
    later columns of the tile."""
    codebook = np.asarray(codebook, dtype=F32)
    corrections = feedback[:, tile_start:tile_start + tile_width].copy()
    for local in range(0, tile_width, dimension):
        position = tile_start + local
        weight = original[:, position:position + dimension]
        target = (weight + corrections[:, local:local + dimension]).astype(F32)
        scale = scales[:, (position - region_start) // group]
        normalized = (target / scale[:, None]).astype(F32)
        codes = nearest_e8p_codes(normalized) if lattice else nearest_codes(normalized, codebook)
        reconstruction = (codebook[codes] * scale[:, None]).astype(F32)
        deviation = (weight - reconstruction).astype(F32)
        later = slice(local + dimension, tile_width)
        pushed = np.zeros((original.shape[0], tile_width - local - dimension), dtype=F32)
        for axis in range(dimension):
            row = coeff[position + axis, tile_start + local + dimension:tile_start + tile_width]
            product = (deviation[:, axis:axis + 1] * row[None, :]).astype(F32)
            pushed = product if axis == 0 else (pushed + product).astype(F32)
        corrections[:, later] = (corrections[:, later] + pushed).astype(F32)
        output[:, position:position + dimension] = reconstruction
        encoded[:, position // dimension] = codes


def vector_sweep(weight, coeff, codebook, *, group, dimension, lattice, refit=None, block=128, fmt="fp16") -> dict:
    """The LDLQ sweep of feedback.sweep for a vector grid (step = dimension): absmax scales
    per group (magnitude = the codebook's largest absolute entry), refitted per region."""
    from . import feedback as scalar_feedback, scaling

    original = np.array(weight, dtype=F32, order="C")
    rows, width = original.shape
    codebook = np.ascontiguousarray(codebook, dtype=F32)
    coeff = np.ascontiguousarray(coeff, dtype=F32)
    pushed = np.zeros_like(original)
    output = np.empty_like(original)
    encoded = np.empty((rows, width // dimension), dtype=np.int32)
    region_width = width if refit is None else refit
    reciprocal = scaling.f32_reciprocal(float(np.abs(codebook).max()))
    all_scales = []
    for region_start in range(0, width, region_width):
        region_stop = min(width, region_start + region_width)
        targets = original[:, region_start:region_stop]
        if region_start:
            targets = (targets + scalar_feedback.pending(pushed, coeff, region_start, region_stop)).astype(F32)
        fitted_group = min(group or width, region_stop - region_start)
        low, high = scaling.group_extrema(targets, fitted_group)
        scales, _ = scaling.store_scale((np.maximum(np.maximum(high, -low), F32(1e-12)) * reciprocal).astype(F32), fmt)
        all_scales.append(scales)
        for tile_start in range(region_start, region_stop, block):
            tile_stop = min(region_stop, tile_start + block)
            round_vector_tile(original, pushed, coeff, scales, codebook, output, encoded, region_start=region_start,
                              tile_start=tile_start, tile_width=tile_stop - tile_start, group=fitted_group,
                              dimension=dimension, lattice=lattice)
            if tile_stop < width:
                scalar_feedback.block_update(pushed, original, output, coeff, tile_start, tile_stop, 0)
    return {"codes": encoded, "scales": np.concatenate(all_scales, 1), "w": output, "refit": region_width}
