"""Pins of the oracle's transforms: the Sylvester matrix product in float64, involution,
orthogonality of the Paley and DCT bases, the factor table (tests/quantization/test_operations.py:8-25,91-100
in /root/reference), and known answers for the conventions a property cannot see: the literal sign
patterns of the Paley matrices (operations/orthogonal_transforms.py:38-67), the DCT-II fallback against
scipy's, the integer hash of the deterministic signs and the sha256 layer seed, all worked out outside the
oracle (tests/golden/make_transform_known_answers.py: Python integers and hashlib only)."""

import hashlib
import json
import pathlib

import numpy as np
import pytest
import scipy.fft
import torch

from mlkit_amd.quantization import codecs as host_codecs
from mlkit_amd.quantization import core as host_core
from mlkit_amd.quantization import transforms as host_transforms
from oracle import transforms

F32 = np.float32
KNOWN = json.loads((pathlib.Path(__file__).resolve().parent / "golden" / "transform_known_answers.json").read_text())

# Derived by hand.  Nonzero squares modulo 11: {1, 3, 4, 5, 9}; modulo 13: {1, 3, 4, 9, 10, 12}.
# Paley I, order 12: row 1 is [-1, then chi(0 - j) + [j == 0] for j = 0..10] = [-1, 1, chi(10), chi(9), ...,
# chi(1)].  Paley II, order 28: row 1 of the conference matrix is [1, 0, chi(12), chi(11), ..., chi(1)];
# the matrix's row 1 is that plus the identity, then that minus the identity; row 14 is row 0 of C - I
# followed by row 0 of -C - I.
PALEY_12_ROW_1 = [-1, 1, -1, 1, -1, -1, -1, 1, 1, 1, -1, 1]
CONFERENCE_14_ROW_1 = [1, 0, 1, -1, 1, 1, -1, -1, -1, -1, 1, 1, -1, 1]
PALEY_28_ROW_1 = ([1, 1] + CONFERENCE_14_ROW_1[2:]) + ([1, -1] + CONFERENCE_14_ROW_1[2:])
PALEY_28_ROW_14 = [-1] + [1] * 13 + [-1] * 14


def sign_pattern(matrix, order):
    scaled = np.asarray(matrix, dtype=np.float64) * np.sqrt(order)
    np.testing.assert_allclose(np.abs(scaled), 1.0, rtol=1e-6)
    return np.rint(scaled).astype(int).tolist()


@pytest.mark.parametrize("width", [1, 2, 4, 8, 16, 32, 64, 128, 2048])
@pytest.mark.parametrize("normalize", [True, False])
def test_fwht_equals_the_sylvester_product(width, normalize, rng):
    value = rng.standard_normal((3, width)).astype(F32)
    exact = value.astype(np.float64) @ transforms.sylvester(width)
    if normalize:
        exact /= np.sqrt(width)
    np.testing.assert_allclose(transforms.fwht(value, normalize), exact, rtol=1e-4, atol=1e-4)


def test_fwht_small_cases_by_hand():
    np.testing.assert_array_equal(transforms.fwht(np.array([[1, 2, 3, 4]], dtype=F32), False), [[10, -2, -4, 0]])
    np.testing.assert_array_equal(transforms.fwht(np.array([[5.0]], dtype=F32)), [[5.0]])
    np.testing.assert_array_equal(transforms.fwht(np.array([[1, 0, 0, 0]], dtype=F32)), [[0.5, 0.5, 0.5, 0.5]])
    assert transforms.normaliser(4096) == F32(1 / 64)
    with pytest.raises(ValueError, match="power-of-two"):
        transforms.fwht(np.zeros((2, 12), dtype=F32))


def test_fwht_is_an_involution_and_keeps_norms(rng):
    value = rng.standard_normal((5, 512)).astype(F32)
    once = transforms.fwht(value)
    np.testing.assert_allclose(transforms.fwht(once), value, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(np.linalg.norm(once, axis=1), np.linalg.norm(value, axis=1), rtol=1e-5)


@pytest.mark.parametrize("order", [4, 8, 12, 20, 24, 28, 44, 76])
def test_paley_matrices_are_orthonormal_sign_matrices(order):
    matrix = transforms.paley(order)
    np.testing.assert_allclose(np.abs(matrix) * np.sqrt(order), np.ones((order, order)), rtol=1e-6)
    np.testing.assert_allclose(matrix.astype(np.float64) @ matrix.T.astype(np.float64), np.eye(order), atol=1e-6)


@pytest.mark.parametrize("source", ["oracle", "host"])
def test_paley_sign_patterns_are_the_known_ones(source):
    """A transposed character matrix, a flipped first column or row, or other block orders of the
    Paley II matrix are still Hadamard matrices; they fail here."""
    build = transforms.paley if source == "oracle" else (lambda order: host_transforms.paley_matrix(order).numpy())
    twelve, twenty_eight = sign_pattern(build(12), 12), sign_pattern(build(28), 28)
    assert twelve[0] == [1] * 12 and [row[0] for row in twelve] == [1] + [-1] * 11
    assert twelve[1] == PALEY_12_ROW_1
    assert twelve[2][1] == 1 and twelve[1][2] == -1          # chi(1) = +1 below the diagonal, chi(-1) = -1 above it
    assert twenty_eight[0] == [1] * 14 + [-1] + [1] * 13
    assert twenty_eight[1] == PALEY_28_ROW_1
    assert twenty_eight[14] == PALEY_28_ROW_14
    assert [row[0] for row in twenty_eight] == [1] * 14 + [-1] + [1] * 13
    for order, expected in KNOWN["paley"].items():
        assert sign_pattern(build(int(order)), int(order)) == expected, order
    assert KNOWN["paley"]["12"][1] == PALEY_12_ROW_1 and KNOWN["paley"]["28"][1] == PALEY_28_ROW_1


@pytest.mark.parametrize("source", ["oracle", "host"])
@pytest.mark.parametrize("width, order", [(7, 7), (43, 43), (86, 43), (11008, 43)])
def test_the_fallback_basis_is_scipy_s_orthonormal_dct_two(source, width, order):
    """Widths whose odd factor reaches no Paley order with a multiplier of 1 to 16 (7; 43, the odd factor of
    11008) keep an orthonormal DCT-II of that factor, y = D x in scipy's convention: a transposed matrix
    (a DCT-III) or an unscaled first row fails here."""
    factor = transforms.transform_factor(width) if source == "oracle" else host_transforms.transform_factor(width)
    assert factor[:2] == (order, width // order)
    basis = np.asarray(factor[2], dtype=np.float64)
    np.testing.assert_allclose(basis, scipy.fft.dct(np.eye(order), type=2, norm="ortho", axis=0), atol=2e-7)
    probe = np.arange(1.0, order + 1.0)
    np.testing.assert_allclose(basis @ probe, scipy.fft.dct(probe, type=2, norm="ortho"), atol=1e-5)
    assert abs(basis[0, 0] - 1 / np.sqrt(order)) < 1e-7 and basis[1, 0] > 0 > basis[1, -1]


def test_structured_transform_applies_the_basis_to_the_outer_axis():
    """``out[f', p] = sum_f basis[f', f] H(x)[f, p]``: the unit vector e_f of a width with power 1 comes out as
    column f of the basis, and with power 2 as (column f) x (1, +-1) / sqrt 2."""
    eye = np.eye(12, dtype=F32)
    np.testing.assert_allclose(transforms.structured(eye), transforms.paley(12).T, atol=1e-7)
    np.testing.assert_allclose(transforms.structured(eye, inverse=True), transforms.paley(12), atol=1e-7)
    host = host_transforms.structured_transform(torch.eye(12)).numpy()
    np.testing.assert_allclose(host, transforms.paley(12).T, atol=1e-6)
    wide = transforms.structured(np.eye(24, dtype=F32))           # 24 = 12 x 2
    pattern = np.array(KNOWN["paley"]["12"], dtype=np.float64) / np.sqrt(12)
    expected = np.kron(pattern, np.array([[1, 1], [1, -1]]) / np.sqrt(2)).T
    np.testing.assert_allclose(wide, expected, atol=1e-6)


def test_transform_factor_table():
    expected = {4096: (1, 4096), 14336: (28, 512), 896: (28, 32), 4864: (76, 64), 11008: (43, 256),
                12: (12, 1), 20: (20, 1), 28: (28, 1), 96: (12, 8), 7: (7, 1)}
    for width, (order, power) in expected.items():
        got = transforms.transform_factor(width)
        assert got[:2] == (order, power), width
        if got[2] is not None:
            np.testing.assert_allclose(got[2].astype(np.float64) @ got[2].T.astype(np.float64), np.eye(order), atol=1e-5)
    with pytest.raises(ValueError):
        transforms.transform_factor(0)


@pytest.mark.parametrize("width", [12, 20, 28, 96, 896, 4864, 7])
def test_structured_round_trip_and_norm(width, rng):
    value = rng.standard_normal((3, width)).astype(F32)
    signs = transforms.deterministic_signs(width, 11)
    rotated = transforms.randomized(value, signs)
    np.testing.assert_allclose(np.linalg.norm(rotated, axis=1), np.linalg.norm(value, axis=1), rtol=1e-5)
    np.testing.assert_allclose(transforms.randomized(rotated, signs, inverse=True), value, rtol=1e-5, atol=1e-5)
    order, power, basis = transforms.transform_factor(width)
    dense = np.kron(np.eye(1) if basis is None else basis.astype(np.float64),
                    transforms.sylvester(power) / np.sqrt(power))
    np.testing.assert_allclose(rotated, (value * signs).astype(np.float64) @ dense.T, rtol=1e-4, atol=1e-5)


def test_deterministic_signs_known_answers():
    for case in KNOWN["signs"]:
        assert transforms.deterministic_signs(16, case["seed"]).tolist() == case["first"], case["seed"]
        assert host_codecs.deterministic_signs(16, case["seed"], "cpu").tolist() == case["first"], case["seed"]
    # the hash itself: 0 stays 0 (sign -1), and the listed values of index + seed
    for value, hashed in KNOWN["hash"].items():
        sign = 1.0 if hashed & 1 else -1.0
        assert transforms.deterministic_signs(1, int(value))[0] == sign
        assert host_codecs.deterministic_signs(1, int(value), "cpu")[0] == sign
    assert KNOWN["hash"]["0"] == 0 and KNOWN["hash"]["1"] == 824515495
    # index + seed wraps modulo 2^32: seed 2^32 - 8 reaches 0 at index 8
    assert transforms.deterministic_signs(16, (1 << 32) - 8)[8:].tolist() == transforms.deterministic_signs(8, 0).tolist()
    assert abs(transforms.deterministic_signs(4096, 7).mean()) < 0.06


def test_layer_seed_known_answers():
    # sha256(b"1:x") begins 55 3f 12 1d 1e ce f2 a1: little-endian 0xa1f2ce1e1d123f55 = 11669616213202452309,
    # and modulo 2^63 - 1 that is 2446244176347676502
    assert hashlib.sha256(b"1:x").hexdigest()[:16] == "553f121d1ecef2a1"
    assert 0xA1F2CE1E1D123F55 % (2**63 - 1) == 2446244176347676502
    for case in KNOWN["layer_seed"]:
        assert transforms.layer_seed(case["name"], case["seed"]) == case["value"], case
        assert host_core.layer_seed(case["name"], case["seed"]) == case["value"], case
    assert transforms.layer_seed("x", 1) == 2446244176347676502
    assert transforms.layer_seed("a") != transforms.layer_seed("b")
