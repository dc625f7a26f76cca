"""Pins of the oracle's grouped-scaling functions: closed forms, IEEE conversions through an
independent library (torch casts), brute force, and the reference's own tolerances
(tests/quantization/test_formats.py:12-16,54-60, tests/kernels/test_scalar_encode.py:44-85,
tests/kernels/test_scalar_decode.py:8-17,61-73 in /root/reference)."""

import numpy as np
import pytest
import torch

from oracle import scaling

import helpers

F32 = np.float32
INT4 = scaling.int_values(4)
SEVEN = np.array([-1, -0.5, -0.25, 0, 0.25, 0.5, 1], dtype=F32)


@pytest.mark.parametrize("fmt,cast", [("fp16", torch.float16), ("bf16", torch.bfloat16)])
def test_store_scale_equals_ieee_casts(fmt, cast, rng):
    value = np.exp(rng.uniform(-20, 12, 20000)).astype(F32)
    stored, bits = scaling.store_scale(value, fmt)
    clamped = torch.from_numpy(value).clamp(2.0**-24, 65504) if fmt == "fp16" else torch.from_numpy(value)
    np.testing.assert_array_equal(stored, clamped.to(cast).float().numpy())
    assert bits == 16


def test_store_scale_fp8_equals_direct_cast_including_ties(rng):
    value = np.exp(rng.uniform(-8, 6.1, 50000)).astype(F32)
    # exact ties between neighbouring e4m3 values (normal and subnormal range)
    grid = torch.arange(0, 127, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    ties = ((grid[1:] + grid[:-1]) / 2).astype(F32)
    value = np.concatenate([value, ties[ties >= 2.0**-9], grid[1:]])
    stored, bits = scaling.store_scale(value, "fp8")
    direct = torch.from_numpy(value).clamp(2.0**-9, 448).to(torch.float8_e4m3fn).float().numpy()
    np.testing.assert_array_equal(stored, direct)
    assert bits == 8


def test_store_scale_e8m0_is_the_nearest_power_of_two_in_log_space(rng):
    value = np.exp(rng.uniform(-30, 30, 20000)).astype(F32)
    stored, _ = scaling.store_scale(value, "e8m0")
    exponent = np.log2(stored.astype(np.float64))
    np.testing.assert_array_equal(exponent, np.rint(exponent))
    assert (np.abs(np.log2(value.astype(np.float64)) - exponent) <= 0.5).all()
    np.testing.assert_array_equal(scaling.store_scale(np.array([1.0, 2.0, 3.0, 2.9, 2.8], dtype=F32), "e8m0")[0],
                                  np.array([1, 2, 4, 4, 2], dtype=F32))  # 2^1.5 = 2.828...


@pytest.mark.parametrize("asym", [False, True])
@pytest.mark.parametrize("shape,group", [((16, 256), 64), ((8, 250), 50), ((5, 70), 128)])
def test_rtn_closed_forms(shape, group, asym):
    weight = helpers.normal_weight(*shape, seed=3, student_t=True)
    result = scaling.quantize(weight, INT4, group=group, integer=True, asym=asym)
    group = result["group"]
    groups = -(-shape[1] // group)
    assert result["scales"].shape == (shape[0], groups)
    assert result["side_bits"] == 16 * shape[0] * groups * (2 if asym else 1)
    assert result["codes"].dtype == np.uint8 and result["codes"].max() <= 15
    columns = np.arange(shape[1]) // group
    scale = result["scales"][:, columns]
    restored = scaling.decode_grouped(result["codes"], result["scales"], INT4, group, result["zero"])
    # inside the clamp range rounding is to the nearest step (scales are fp16-rounded, so the
    # largest magnitude of a group may clip by a fraction of a step)
    zero = 0 if result["zero"] is None else result["zero"][:, columns]
    normalized = (weight - zero) / scale
    inside = (normalized >= -8) & (normalized <= 7)
    assert (np.abs(weight - restored)[inside] <= scale[inside] * 0.5000001).all()
    assert inside.mean() > 0.98
    if not asym:
        blocks_max = np.abs(np.pad(weight, ((0, 0), (0, groups * group - shape[1]))).reshape(shape[0], groups, group)).max(-1)
        expected = np.maximum(blocks_max, F32(1e-12)) * F32(0.125)
        np.testing.assert_array_equal(result["scales"], scaling.store_scale(expected.astype(F32), "fp16")[0])


def test_asymmetric_offsets_follow_the_group_minimum():
    weight = helpers.normal_weight(8, 256, seed=4) + F32(0.05)
    scales, zero = scaling.initial_scales(weight, INT4, 64, True)
    low = weight.reshape(8, 4, 64).min(-1)
    high = weight.reshape(8, 4, 64).max(-1)
    np.testing.assert_array_equal(scales, (np.maximum(high - low, F32(1e-12)) * (F32(1) / F32(15))).astype(F32))
    np.testing.assert_array_equal(zero, (low - F32(-8) * scales).astype(F32))
    stored = scaling.stored_offset(zero, "fp16")
    np.testing.assert_array_equal(np.sign(stored), np.sign(zero))
    np.testing.assert_array_equal(np.abs(stored), np.abs(zero).astype(np.float16).astype(F32))


def test_nearest_codes_equals_brute_force_with_lower_index_on_ties(rng):
    for table in (SEVEN, scaling.NF4_VALUES, np.sort(rng.standard_normal(200).astype(F32))):
        value = (rng.standard_normal(5000) * 0.8).astype(np.float16).astype(F32)  # fp16 values tie often
        midpoints = ((table[1:].astype(np.float64) + table[:-1]) / 2).astype(F32)
        value = np.concatenate([value, midpoints, table, [-7.0, 7.0]]).astype(F32)
        distances = np.abs(value[:, None] - table[None, :])  # fp32, as the reference computes them
        brute = distances.argmin(1)  # first minimum = lowest index
        np.testing.assert_array_equal(scaling.nearest_codes(value, table), brute)


def test_integer_codes_round_half_to_even_and_saturate():
    value = np.array([[-9.0, -8.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 6.5, 7.5, 8.0, 0.49999997]], dtype=F32)
    codes = scaling.encode(value, np.ones((1, 1), dtype=F32), None, INT4, 16, True)
    assert codes[0].tolist() == [0, 0, 6, 6, 8, 8, 10, 10, 14, 15, 15, 8]


def test_division_is_true_division_not_reciprocal_multiplication(rng):
    value = rng.standard_normal((64, 64)).astype(F32)
    scales = (rng.random((64, 1)) + 0.01).astype(F32)
    exact = (value.astype(np.float64) / scales.astype(np.float64)).astype(F32)  # correctly rounded quotient
    np.testing.assert_array_equal(scaling.normalize(value, scales, None, 64), exact)
    assert (exact != (value * (F32(1) / scales)).astype(F32)).any()


@pytest.mark.parametrize("values,integer", [(INT4, True), (SEVEN, False)])
def test_scale_search_against_float64_brute_force(values, integer):
    weight = helpers.normal_weight(48, 512, seed=7, student_t=True)
    group = 64
    scales, _ = scaling.store_scale(scaling.initial_scales(weight, values, group, False)[0], "fp16")
    fractions = np.linspace(0.5, 1.0, 20).astype(F32)
    chosen = scaling.search_scales(weight, scales, None, values, fractions, group, "fp16", integer)

    def error64(candidate):
        blocks = weight.reshape(48, -1, group)
        normalized = (blocks / candidate[..., None]).astype(F32)
        if integer:
            rounded = np.clip(np.rint(normalized), -8, 7)
        else:
            rounded = values[np.abs(normalized[..., None] - values).argmin(-1)]
        return ((rounded.astype(np.float64) * candidate[..., None] - blocks) ** 2).sum(-1)

    best, best_error = scales.copy(), error64(scales)
    for fraction in fractions:
        candidate, _ = scaling.store_scale((scales * fraction).astype(F32), "fp16")
        error = error64(candidate)
        better = error < best_error
        best, best_error = np.where(better, candidate, best), np.minimum(best_error, error)
    assert (chosen == best).mean() >= 0.97          # the reference's own agreement bound
    np.testing.assert_allclose(error64(chosen), best_error, rtol=1e-3)
    assert (error64(chosen) <= error64(scales) * (1 + 1e-6)).all()   # never worse than absmax
    assert (chosen != scales).mean() > 0.3


@pytest.mark.parametrize("values,integer,asym,fmt", [
    (INT4, True, False, "fp16"), (INT4, True, True, "fp16"), (SEVEN, False, False, "fp16"),
    (scaling.NF4_VALUES, False, False, "bf16"), (scaling.int_values(3), True, False, "fp16"),
])
def test_scale_search_selects_the_float64_winner_wherever_it_is_clear(values, integer, asym, fmt):
    """Every group whose float64 least error beats every differently-stored candidate by more
    than 1e-4 relative must get exactly that candidate: a wrong candidate order, a wrong
    storage rounding of a candidate or a wrong comparison cannot hide inside a percentage."""
    rows, width, group = 64, 640, 64
    weight = helpers.normal_weight(rows, width, seed=31, student_t=True)
    base, zero = scaling.initial_scales(weight, values, group, asym)
    base, _ = scaling.store_scale(base, fmt)
    fractions = np.linspace(0.5, 1.0, 20).astype(F32)
    chosen = scaling.search_scales(weight, base, zero, values, fractions, group, fmt, integer)

    blocks = weight.reshape(rows, -1, group)
    centered = blocks if zero is None else (blocks - zero[..., None]).astype(F32)

    def error64(candidate):
        normalized = (centered / candidate[..., None]).astype(F32)
        if integer:
            rounded = np.clip(np.rint(normalized), values.min(), values.max())
        else:
            rounded = values[np.abs(normalized[..., None] - values).argmin(-1)]
        return ((rounded.astype(np.float64) * candidate[..., None] - centered) ** 2).sum(-1)

    candidates = [base] + [scaling.store_scale((base * f).astype(F32), fmt)[0] for f in fractions]
    errors = np.stack([error64(c) for c in candidates])            # [21, rows, groups]
    stack = np.stack(candidates)
    winner = errors.argmin(0)                                       # first index of the least error
    least = np.take_along_axis(errors, winner[None], 0)[0]
    best_scale = np.take_along_axis(stack, winner[None], 0)[0]
    rivals = np.where(stack != best_scale[None], errors, np.inf).min(0)
    clear = rivals > least * (1 + 1e-4)
    assert clear.mean() > 0.9, clear.mean()                         # the criterion must not be vacuous
    np.testing.assert_array_equal(chosen[clear], best_scale[clear])
    assert (chosen[clear] != base[clear]).mean() > 0.3              # and most winners are shrunken scales


def test_scale_search_keeps_the_base_scale_on_an_exact_tie():
    """A group of zeros has error exactly 0 under every candidate: the base scale stays
    (grouped_scaling.py:343-350, `error < best_error`).  The fractions end below 1 so that
    "the last candidate wins ties" would pick a different stored value; fp32 storage keeps the
    candidates distinct."""
    weight = helpers.normal_weight(4, 128, seed=32)
    weight[1, 64:] = 0
    weight[3, :64] = 0
    fractions = np.array([0.5, 0.75], dtype=F32)
    for values, integer in ((INT4, True), (SEVEN, False)):
        base, _ = scaling.store_scale(scaling.initial_scales(weight, values, 64, False)[0], "fp32")
        chosen = scaling.search_scales(weight, base, None, values, fractions, 64, "fp32", integer)
        assert chosen[1, 1] == base[1, 1] and chosen[3, 0] == base[3, 0]
        assert base[1, 1] != F32(base[1, 1] * F32(0.75))


def test_ordered_group_error_is_a_sum_of_squares(rng):
    weight = helpers.normal_weight(8, 384, seed=8)
    scales = scaling.initial_scales(weight, INT4, 128, False)[0]
    ordered = scaling.group_error_ordered(weight, scales, None, INT4, 128, True)
    blocks = weight.reshape(8, 3, 128)
    restored = np.clip(np.rint(blocks / scales[..., None]), -8, 7) * scales[..., None]
    np.testing.assert_allclose(ordered, ((restored - blocks).astype(np.float64) ** 2).sum(-1), rtol=1e-5)


def test_decode_index_maps():
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 16, (4, 20), dtype=np.uint8)
    scales = (rng.random((4, 4)) + 0.5).astype(F32)
    zero = rng.standard_normal((4, 4)).astype(F32)
    dense = scaling.decode_grouped(codes, scales, INT4, 6, zero)
    for r in range(4):
        for c in range(20):
            assert dense[r, c] == F32(F32(INT4[codes[r, c]] * scales[r, c // 6]) + zero[r, c // 6])
    # feedback codec: regions of 10 columns with ceil(10 / 4) = 3 scale slots each
    scales = (rng.random((4, 6)) + 0.5).astype(F32)
    index = scaling.feedback_scale_index(20, 4, 10)
    assert index.tolist() == [0, 0, 0, 0, 1, 1, 1, 1, 2, 2, 3, 3, 3, 3, 4, 4, 4, 4, 5, 5]
    dense = scaling.decode_feedback(codes, scales, INT4, 4, 10)
    assert dense[2, 13] == F32(INT4[codes[2, 13]] * scales[2, 3])
    # no fused multiply-add: multiply rounds before the add
    one = scaling.decode_grouped(np.array([[15]], dtype=np.uint8), np.array([[F32(0.1)]]), INT4, 1,
                                 np.array([[F32(1e-8)]]))
    assert one[0, 0] == F32(F32(7 * F32(0.1)) + F32(1e-8))
