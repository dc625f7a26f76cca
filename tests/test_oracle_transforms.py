"""Pins of the oracle's transforms: the Sylvester matrix product in float64, involution,
orthogonality of the Paley and DCT bases, the factor table, and the integer hash and sha256
seed computed by hand (tests/quantization/test_operations.py:8-25,91-100 in /root/reference)."""

import hashlib

import numpy as np
import pytest

from oracle import transforms

F32 = np.float32


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


def test_deterministic_signs_by_hand():
    def one(index, seed):
        v = (index + seed) & 0xFFFFFFFF
        v = ((v ^ (v >> 16)) * 0x45D9F3B) & 0xFFFFFFFF
        v = ((v ^ (v >> 16)) * 0x45D9F3B) & 0xFFFFFFFF
        v ^= v >> 16
        return 1.0 if v & 1 else -1.0

    signs = transforms.deterministic_signs(16, 123456789)
    assert signs.tolist() == [one(i, 123456789) for i in range(16)]
    # 0 hashes to 0: the first sign of seed 0 is -1; a sample is roughly balanced
    assert transforms.deterministic_signs(1, 0)[0] == -1.0
    assert abs(transforms.deterministic_signs(4096, 7).mean()) < 0.06


def test_layer_seed_is_the_low_eight_bytes_of_sha256():
    digest = hashlib.sha256(b"3:model.layers.0.mlp.down_proj").digest()
    assert transforms.layer_seed("model.layers.0.mlp.down_proj", 3) == int.from_bytes(digest[:8], "little") % (2**63 - 1)
    assert transforms.layer_seed("a") != transforms.layer_seed("b")
