"""Pins of the oracle's LDL error feedback: the inverse-Cholesky identity in float64, the
textbook GPTQ loop, a second implementation of the tile arithmetic, the triangular-solve
definition, and the invariants the reference asserts (tests/quantization/test_algorithms.py:
12-46,142-202, tests/kernels/test_error_feedback.py:31-42 in /root/reference)."""

import numpy as np
import pytest

from oracle import feedback, scaling

import helpers

F32 = np.float32
INT4 = scaling.int_values(4)


def hessian(width, seed, samples=None, dead=()):
    rng = np.random.default_rng(seed)
    samples = samples or 3 * width
    inputs = rng.standard_normal((samples, width)).astype(F32)
    inputs[:, ::5] *= 3
    inputs += 0.4 * np.roll(inputs, 1, axis=1)
    inputs[:, list(dead)] = 0
    return (inputs.T @ inputs / samples).astype(F32)


def classic_gptq(weight, hessian_matrix, quantize_column, damp=0.01):
    """The textbook loop: Hinv = chol_upper(inverse(H + damp)), column j rounded, later columns
    receive -err * Hinv[j, j+1:] with err = (w_j - q_j) / Hinv[j, j]; all in float64."""
    h = hessian_matrix.astype(np.float64).copy()
    dead = np.diag(h) == 0
    h[dead, dead] = 1
    h[np.diag_indices_from(h)] += damp * np.mean(np.diag(h))
    upper = np.linalg.cholesky(np.linalg.inv(h)).T
    w = weight.astype(np.float64).copy()
    w[:, dead] = 0
    out = np.zeros_like(w)
    for j in range(w.shape[1]):
        out[:, j] = quantize_column(w[:, j], j)
        error = (w[:, j] - out[:, j]) / upper[j, j]
        w[:, j + 1:] -= error[:, None] * upper[j, j + 1:][None, :]
    return out


def test_coefficients_equal_the_inverse_cholesky_form():
    h = hessian(96, seed=1)
    coeff, status = feedback.coefficients(h, 0.01)
    assert status == 0
    damped = h.astype(np.float64).copy()
    damped[np.diag_indices_from(damped)] += 0.01 * np.mean(np.diag(damped))
    t = np.linalg.cholesky(np.linalg.inv(damped)).T            # Hinv = T^T T, T upper
    expected = np.linalg.inv(t) @ np.diag(np.diag(t))           # unit upper: A = T^-1 diag(T)
    np.testing.assert_allclose(np.triu(coeff), np.triu(expected), rtol=1e-3, atol=1e-5)
    np.testing.assert_array_equal(np.diag(coeff), np.ones(96, dtype=F32))
    assert np.abs(np.tril(coeff, -1)).max() == 0


def test_indefinite_hessian_is_reported():
    h = hessian(16, seed=2)
    h[3, 3] = -5
    assert feedback.coefficients(h, 0.0)[1] != 0


@pytest.mark.parametrize("refit,block", [(None, 32), (None, 128)])
def test_sweep_follows_the_textbook_loop(refit, block):
    """With one fixed scale per row (fitted once on the original weights) the LDL sweep and the
    inverse-Cholesky loop are the same recursion."""
    rows, width = 24, 96
    weight = helpers.normal_weight(rows, width, seed=5)
    h = hessian(width, seed=6)
    coeff, _ = feedback.coefficients(h, 0.01)
    result = feedback.sweep(weight, coeff, INT4, group=width, integer=True, refit=refit, block=block)
    scale = result["scales"][:, 0].astype(np.float64)

    def quantize_column(column, j):
        return np.clip(np.rint(column / scale), -8, 7) * scale

    expected = classic_gptq(weight, h, quantize_column)
    mismatched = (np.abs(result["w"] - expected) > 1e-6 + 1e-5 * np.abs(expected)).mean()
    assert mismatched < 0.002, mismatched  # a rounding tie may flip between fp32 and float64
    loss = feedback.proxy_loss(weight, result["w"], h)
    rtn = scaling.decode_grouped(scaling.encode(weight, result["scales"], None, INT4, width, True),
                                 result["scales"], INT4, width)
    assert loss < feedback.proxy_loss(weight, rtn, h)


def test_c_tile_equals_numpy_tile_and_update_modes_agree():
    rows, width = 37, 192
    weight = helpers.normal_weight(rows, width, seed=7)
    coeff, _ = feedback.coefficients(hessian(width, seed=8), 0.01)
    for values, integer, asym in ((INT4, True, False), (INT4, True, True), (scaling.NF4_VALUES, False, False)):
        fast = feedback.sweep(weight, coeff, values, group=64, integer=integer, refit=64, block=64, asym=asym)
        slow = feedback.sweep(weight, coeff, values, group=64, integer=integer, refit=64, block=64, asym=asym,
                              tile_fn=feedback.round_tile_numpy)
        np.testing.assert_array_equal(fast["codes"], slow["codes"])
        np.testing.assert_array_equal(fast["w"], slow["w"])
        np.testing.assert_array_equal(fast["scales"], slow["scales"])
        separate = feedback.sweep(weight, coeff, values, group=64, integer=integer, refit=64, block=64, asym=asym,
                                  update_mode=1)
        assert (separate["codes"] == fast["codes"]).mean() > 0.995   # fma vs mul+add: only ties move
        restored = scaling.decode_feedback(fast["codes"], fast["scales"], values, 64, 64, fast["zero"])
        np.testing.assert_array_equal(restored, fast["w"])


def test_pending_is_a_triangular_solve():
    rows, width = 16, 160
    coeff, _ = feedback.coefficients(hessian(width, seed=9), 0.01)
    pushed = (np.random.default_rng(1).standard_normal((rows, width)) * 0.01).astype(F32)
    solved = feedback.pending(pushed, coeff, 32, 160)
    block = np.triu(coeff[32:160, 32:160]).astype(np.float64)
    np.testing.assert_allclose(solved @ block, pushed[:, 32:], rtol=1e-4, atol=1e-7)


def test_block_update_is_a_matrix_product():
    rows, width = 20, 96
    weight = helpers.normal_weight(rows, width, seed=10)
    coeff, _ = feedback.coefficients(hessian(width, seed=11), 0.01)
    output = (weight + np.random.default_rng(2).standard_normal(weight.shape).astype(F32) * 0.002).astype(F32)
    for mode in (0, 1):
        pushed = np.zeros_like(weight)
        feedback.block_update(pushed, weight, output, coeff, 16, 48, mode)
        exact = (weight - output)[:, 16:48].astype(np.float64) @ coeff[16:48, 48:].astype(np.float64)
        np.testing.assert_allclose(pushed[:, 48:], exact, rtol=1e-4, atol=1e-8)
        assert np.abs(pushed[:, :48]).max() == 0


def test_dead_channels_round_to_zero_and_bits_add_up():
    rows, width = 12, 128
    weight = helpers.normal_weight(rows, width, seed=12)
    h = hessian(width, seed=13, dead=(5, 77))
    coeff, status = feedback.coefficients(h, 0.01)
    assert status == 0
    result = feedback.sweep(weight, coeff, INT4, group=32, integer=True, refit=64, block=32,
                            dead=np.diag(h) == 0)
    assert np.isfinite(result["w"]).all()
    assert np.abs(result["w"][:, [5, 77]]).max() == 0
    assert result["scales"].shape == (rows, width // 32)
    bits = 4 * rows * width + 16 * result["scales"].size
    assert bits / (rows * width) == 4.5


def test_fit_scales_c_equals_numpy():
    targets = helpers.normal_weight(9, 200, seed=14, student_t=True)
    for asym in (False, True):
        scales, zeros = feedback.fit_scales(targets, INT4, 64, asym)
        expected, zero = scaling.initial_scales(targets, INT4, 64, asym)
        np.testing.assert_array_equal(scales, scaling.store_scale(expected, "fp16")[0])
        if asym:
            np.testing.assert_array_equal(zeros, scaling.stored_offset(zero, "fp16"))


def classic_gptq_with_region_refits(weight, hessian_matrix, refit, group, asym, damp=0.01):
    """The inverse-Cholesky loop in float64 where, at the first column of every region of
    `refit` columns, the region's fp16 scales (and offsets) are fitted to the running weights
    of that region -- the values its columns would take if nothing more were rounded
    (algorithms/error_feedback.py:296-303,373-393 in /root/reference).  Scale fitting goes
    through scaling.initial_scales / store_scale, not through the sweep's own C fit."""
    h = hessian_matrix.astype(np.float64).copy()
    h[np.diag_indices_from(h)] += damp * np.mean(np.diag(h))
    upper = np.linalg.cholesky(np.linalg.inv(h)).T
    w = weight.astype(np.float64).copy()
    rows, width = w.shape
    out = np.zeros_like(w)
    all_scales, all_zeros = [], []
    for j in range(width):
        if j % refit == 0:
            stop = min(width, j + refit)
            fitted_group = min(group, stop - j)
            scales, zero = scaling.initial_scales(w[:, j:stop].astype(F32), INT4, fitted_group, asym)
            scales, _ = scaling.store_scale(scales, "fp16")
            if zero is not None:
                zero = scaling.stored_offset(zero, "fp16")
                all_zeros.append(zero)
            all_scales.append(scales)
        slot = (j % refit) // fitted_group
        scale = scales[:, slot].astype(np.float64)
        offset = 0.0 if zero is None else zero[:, slot].astype(np.float64)
        out[:, j] = np.clip(np.rint((w[:, j] - offset) / scale), -8, 7) * scale + offset
        error = (w[:, j] - out[:, j]) / upper[j, j]
        w[:, j + 1:] -= error[:, None] * upper[j, j + 1:][None, :]
    return out, np.concatenate(all_scales, 1), np.concatenate(all_zeros, 1) if all_zeros else None


@pytest.mark.parametrize("refit,group,block,asym", [
    (32, 32, 32, False), (32, 32, 32, True), (64, 64, 64, False), (64, 64, 64, True),
    (64, 16, 32, False), (64, 32, 64, True), (32, 8, 16, True), (64, 64, 16, False),
    (48, 16, 48, False),                      # ragged: the last region holds 32 of 48 columns
])
def test_sweep_with_region_refits_follows_the_textbook_loop(refit, group, block, asym):
    """Region refits (pending continuation -> targets -> scale fit -> tiles) against the float64
    textbook loop: identical stored scales, reconstruction within 1e-6 + 1e-5 |w|."""
    rows, width = 24, 128
    weight = helpers.normal_weight(rows, width, seed=21 + refit + group)
    h = hessian(width, seed=22 + block)
    coeff, status = feedback.coefficients(h, 0.01)
    assert status == 0
    result = feedback.sweep(weight, coeff, INT4, group=group, integer=True, refit=refit, block=block, asym=asym)
    expected, scales, zeros = classic_gptq_with_region_refits(weight, h, refit, group, asym)
    np.testing.assert_array_equal(result["scales"], scales)
    if asym:
        np.testing.assert_array_equal(result["zero"], zeros)
    assert (np.abs(result["w"] - expected) <= 1e-6 + 1e-5 * np.abs(expected)).all()
    # Dropping the pending continuation (fitting to the original weights) must fail this pin.
    naive = scaling.store_scale(scaling.initial_scales(weight[:, refit:2 * refit], INT4,
                                                       min(group, refit), asym)[0], "fp16")[0]
    per_region = -(-refit // min(group, refit))
    assert not np.array_equal(naive, scales[:, per_region:2 * per_region])


def test_sweep_accepts_column_permuted_views():
    """Fancy-indexed columns come back from numpy in column-major order; the sweep must read
    them as rows all the same (activation order hands it `weight[:, permutation]`)."""
    rows, width = 16, 96
    weight = helpers.normal_weight(rows, width, seed=40)
    coeff, _ = feedback.coefficients(hessian(width, seed=41), 0.01)
    permutation = np.random.default_rng(3).permutation(width)
    view = weight[:, permutation]
    direct = feedback.sweep(view, coeff, INT4, group=32, integer=True, refit=32, block=32)
    copied = feedback.sweep(np.ascontiguousarray(view), coeff, INT4, group=32, integer=True, refit=32, block=32)
    np.testing.assert_array_equal(direct["codes"], copied["codes"])
    first = np.clip(np.rint(view[:, 0] / direct["scales"][:, 0]), -8, 7) + 8
    np.testing.assert_array_equal(direct["codes"][:, 0], first.astype(np.uint8))
