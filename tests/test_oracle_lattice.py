"""Pins of the oracle's vector grids: the E8P point set by its defining properties, the
structured search against a brute force over all 65,536 points, the generic nearest-codeword
search, and the vector feedback sweep against the textbook block-LDL loop in float64."""

import numpy as np
import pytest

from oracle import feedback, lattice

import helpers
from test_oracle_feedback import hessian

F32 = np.float32


def test_e8p_point_set_properties():
    patterns = lattice.absolute_points()
    points = lattice.e8p_points()
    assert patterns.shape == (256, 8) and points.shape == (65536, 8)
    norms = (patterns.astype(np.float64) ** 2).sum(1)
    assert (norms[:227] <= 10).all() and (norms[227:] == 12).all() and len(np.unique(patterns, axis=0)) == 256
    assert set(np.unique(patterns)) == {0.5, 1.5, 2.5}
    assert len(np.unique(points, axis=0)) == 65536                       # all codes are distinct points
    # every point is a point of D8-hat = {x in (Z + 1/2)^8 : sum(x) even} shifted by +-1/4
    for half, shift in ((points[:32768], 0.25), (points[32768:], -0.25)):
        base = half.astype(np.float64) - shift
        assert np.array_equal(base * 2 % 2, np.ones_like(base))          # half-integers
        assert (base.sum(1) % 2 == 0).all()
    # code numbering: pattern * 128 + sign bits of the first seven coordinates
    code = 37 * 128 + 0b1010011
    expected = patterns[37].copy()
    expected[[0, 1, 4, 6]] *= -1
    if int(patterns[37].sum() + 4) % 2:
        expected[7] *= -1
    np.testing.assert_array_equal(points[code], expected + 0.25)
    np.testing.assert_array_equal(points[code + 32768], expected - 0.25)


@pytest.mark.parametrize("spread", [0.3, 1.0, 2.5])
def test_structured_search_finds_the_nearest_point(spread):
    rng = np.random.default_rng(int(spread * 10))
    vectors = (rng.standard_normal((400, 8)) * spread).astype(F32)
    codes = lattice.nearest_e8p_codes(vectors)
    points = lattice.e8p_points().astype(np.float64)
    distances = ((vectors[:, None, :].astype(np.float64) - points[None]) ** 2).sum(2)
    chosen = distances[np.arange(len(vectors)), codes]
    np.testing.assert_allclose(chosen, distances.min(1), rtol=1e-5, atol=1e-6)
    assert (codes == distances.argmin(1)).mean() > 0.98          # the rest are exact or near ties
    # an exact lattice point is returned as itself
    exact = lattice.e8p_points()[[5, 4000, 40000, 65535]]
    np.testing.assert_array_equal(lattice.nearest_e8p_codes(exact), [5, 4000, 40000, 65535])


def test_nearest_codeword_is_a_brute_force_argmin_with_ties_to_the_lower_index():
    rng = np.random.default_rng(2)
    codebook = rng.standard_normal((600, 4)).astype(F32)
    codebook[17] = codebook[3]                                           # a duplicate: index 3 must win
    vectors = rng.standard_normal((300, 4)).astype(F32)
    vectors[0] = codebook[17]
    codes = lattice.nearest_codes(vectors, codebook)
    distances = ((vectors[:, None, :].astype(np.float64) - codebook[None].astype(np.float64)) ** 2).sum(2)
    assert (codes == distances.argmin(1)).mean() > 0.99 and codes[0] == 3
    np.testing.assert_allclose(distances[np.arange(300), codes], distances.min(1), rtol=1e-5)


def classic_block_ldl(weight, hessian_matrix, quantize_block, dimension, damp=0.01):
    """Textbook LDLQ with blocks: H + damp = L D L^T by blocks; block k is rounded after adding
    the feedback of the earlier blocks' errors; float64 throughout (the inverse-Cholesky form
    of the same recursion, one block of columns at a time)."""
    h = hessian_matrix.astype(np.float64).copy()
    h[np.diag_indices_from(h)] += damp * np.mean(np.diag(h))
    upper = np.linalg.cholesky(np.linalg.inv(h)).T
    w = weight.astype(np.float64).copy()
    out = np.zeros_like(w)
    for start in range(0, w.shape[1], dimension):
        stop = start + dimension
        out[:, start:stop] = quantize_block(w[:, start:stop], start)
        error = (w[:, start:stop] - out[:, start:stop]) @ np.linalg.inv(upper[start:stop, start:stop])
        w[:, stop:] -= error @ upper[start:stop, stop:]
    return out


@pytest.mark.parametrize("name", ["lattice", "quadruples"])
def test_vector_sweep_follows_the_textbook_block_loop(name):
    """One scale per row fitted once: the oracle's additive-correction sweep with block
    coefficients A = R blockdiag(R)^-1 is the block-LDL recursion; the same codes but for
    near ties, the same reconstruction where codes agree."""
    rows, width = 16, 64
    rng = np.random.default_rng(5)
    weight = helpers.normal_weight(rows, width, seed=51, scale=1.0)
    h = hessian(width, seed=52)
    if name == "lattice":
        codebook, dimension, is_lattice = lattice.e8p_points(), 8, True
        search = lattice.nearest_e8p_codes
    else:
        codebook, dimension, is_lattice = rng.standard_normal((600, 4)).astype(F32), 4, False
        search = lambda v: lattice.nearest_codes(v, codebook)  # noqa: E731
    coeff = block_coefficients(h, dimension)
    result = lattice.vector_sweep(weight, coeff, codebook, group=None, dimension=dimension, lattice=is_lattice,
                                  refit=None, block=32)
    scale = result["scales"][:, 0].astype(np.float64)

    def quantize_block(block, start):
        codes = search((block / scale[:, None]).astype(F32))
        return codebook[codes].astype(np.float64) * scale[:, None]

    expected = classic_block_ldl(weight, h, quantize_block, dimension)
    agree = np.isclose(result["w"], expected, rtol=1e-5, atol=1e-6).reshape(rows, -1, dimension).all(2)
    assert agree.mean() > 0.97, agree.mean()
    restored = lattice.decode_vector_scaled(result["codes"], result["scales"], codebook, width, dimension)
    np.testing.assert_array_equal(restored, result["w"])
    # feedback helps: the Hessian-weighted error is below that of direct rounding
    direct = quantize_block(weight.astype(np.float64), 0) if False else np.concatenate(
        [quantize_block(weight[:, s:s + dimension].astype(np.float64), s) for s in range(0, width, dimension)], 1)
    assert feedback.proxy_loss(weight, result["w"], h) < feedback.proxy_loss(weight, direct.astype(F32), h)


def block_coefficients(hessian_matrix, step, damp=0.01):
    """A = R blockdiag(R)^-1 for the damped H = R R^T (upper R), float64 -> fp32."""
    h = hessian_matrix.astype(np.float64).copy()
    h[np.diag_indices_from(h)] += damp * np.mean(np.diag(h))
    lower = np.linalg.cholesky(h[::-1, ::-1])
    upper = lower[::-1, ::-1]
    out = np.zeros_like(upper)
    for start in range(0, len(h), step):
        stop = start + step
        out[:, start:stop] = upper[:, start:stop] @ np.linalg.inv(upper[start:stop, start:stop])
    return np.ascontiguousarray(out, dtype=F32)
