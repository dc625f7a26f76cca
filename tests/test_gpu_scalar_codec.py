"""GPU parity (through the C ABI) of the scalar codec kernels against the oracle: every
comparison here is bit for bit (codes, scales, decoded values)."""

import numpy as np
import pytest
import torch

from oracle import scaling

import helpers

pytestmark = pytest.mark.gpu

F32 = np.float32
INT4 = scaling.int_values(4)
INT3 = scaling.int_values(3)
SEVEN = np.array([-1, -0.5, -0.25, 0, 0.25, 0.5, 1], dtype=F32)
TABLE256 = np.sort(np.random.default_rng(3).standard_normal(256).astype(F32))
FRACTIONS = np.linspace(0.5, 1.0, 20).astype(F32)


def dev(array):
    return None if array is None else torch.from_numpy(np.ascontiguousarray(array)).cuda()


def host(tensor):
    torch.cuda.synchronize()
    return tensor.cpu().numpy()


CASES = [
    # rows, width, group, values, integer, asym
    (64, 256, 128, INT4, True, False),
    (64, 256, 128, INT4, True, True),
    (33, 250, 50, INT3, True, True),      # groups that are not a power of two, ragged width
    (17, 203, 64, INT4, True, False),     # odd width: scalar path, partial last group
    (64, 512, 64, scaling.NF4_VALUES, False, False),
    (64, 512, 64, SEVEN, False, False),
    (16, 384, 128, TABLE256, False, True),
    (8, 96, 96, INT4, True, False),       # one group per row
]


@pytest.mark.parametrize("rows,width,group,values,integer,asym", CASES)
def test_fit_encode_decode_match_oracle(rows, width, group, values, integer, asym):
    from mlkit_amd.kernels import scalar_decode, scalar_encode

    weight = helpers.normal_weight(rows, width, seed=rows + width, student_t=True)
    expected_scales, expected_zero = scaling.initial_scales(weight, values, group, asym)
    expected_scales, _ = scaling.store_scale(expected_scales, "fp16")
    reciprocal = scaling.f32_reciprocal(float(values.max() - values.min()) if asym else float(np.abs(values).max()))
    scales, zeros = scalar_encode.fit_scales(dev(weight), group, asym=asym, reciprocal=float(reciprocal),
                                             value_minimum=float(values.min()), scale_format="fp16",
                                             store_zero=False)
    np.testing.assert_array_equal(host(scales), expected_scales)
    if asym:
        np.testing.assert_array_equal(host(zeros), expected_zero)
        stored = scalar_encode.fit_scales(dev(weight), group, asym=True, reciprocal=float(reciprocal),
                                          value_minimum=float(values.min()), scale_format="fp16",
                                          store_zero=True)[1]
        expected_zero = scaling.stored_offset(expected_zero, "fp16")
        np.testing.assert_array_equal(host(stored), expected_zero)
        zeros = stored
    expected_codes = scaling.encode(weight, expected_scales, expected_zero, values, group, integer)
    codes = scalar_encode.encode(dev(weight), scales, zeros, dev(values), group, None, integer=integer,
                                 minimum=float(values.min()), maximum=float(values.max()))
    np.testing.assert_array_equal(host(codes), expected_codes)
    expected = scaling.decode_grouped(expected_codes, expected_scales, values, group, expected_zero)
    decoded = scalar_decode.decode(codes, scales, dev(values), zeros, group)
    np.testing.assert_array_equal(host(decoded), expected)


def test_exact_ties_follow_half_even_and_lower_entry():
    from mlkit_amd.kernels import scalar_encode

    # scale 1, values on exact half steps: rint ties to even; codebook ties to the lower entry
    value = np.array([[-2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.5, 9.0, -9.0, 0.0, 0.75, -0.75, 0.375, -0.375, 0.125, 3.0]],
                     dtype=F32)
    scales = np.ones((1, 1), dtype=F32)
    integer = scalar_encode.encode(dev(value), dev(scales), None, dev(INT4), 16, None, integer=True,
                                   minimum=-8.0, maximum=7.0)
    np.testing.assert_array_equal(host(integer), scaling.encode(value, scales, None, INT4, 16, True))
    assert host(integer)[0, :7].tolist() == [6, 6, 8, 8, 10, 10, 12]
    table = scalar_encode.encode(dev(value), dev(scales), None, dev(SEVEN), 16, None, integer=False,
                                 minimum=-1.0, maximum=1.0)
    np.testing.assert_array_equal(host(table), scaling.encode(value, scales, None, SEVEN, 16, False))
    brute = np.abs(value[0, :, None].astype(np.float64) - SEVEN[None, :].astype(np.float64)).argmin(1)
    np.testing.assert_array_equal(host(table)[0], brute)


@pytest.mark.parametrize("fmt", ["fp32", "fp16", "bf16", "fp8", "e8m0"])
def test_fit_scales_storage_formats(fmt):
    from mlkit_amd.kernels import scalar_encode

    weight = helpers.normal_weight(48, 512, seed=9, scale=0.3, student_t=True)
    expected, zero = scaling.initial_scales(weight, INT4, 64, True)
    expected, _ = scaling.store_scale(expected, fmt)
    scales, zeros = scalar_encode.fit_scales(dev(weight), 64, asym=True, reciprocal=float(scaling.f32_reciprocal(15.0)),
                                             value_minimum=-8.0, scale_format=fmt, store_zero=True)
    np.testing.assert_array_equal(host(scales), expected)
    np.testing.assert_array_equal(host(zeros), scaling.stored_offset(zero, fmt))


def test_fit_scales_on_a_column_slice_and_non_finite_input():
    from mlkit_amd.kernels import scalar_encode

    weight = helpers.normal_weight(32, 640, seed=4)
    region = dev(weight)[:, 128:384]
    scales, _ = scalar_encode.fit_scales(region, 128, asym=False, reciprocal=0.125, value_minimum=-8.0,
                                         scale_format="fp16", store_zero=False)
    expected, _ = scaling.store_scale(scaling.initial_scales(weight[:, 128:384], INT4, 128, False)[0], "fp16")
    np.testing.assert_array_equal(host(scales), expected)
    broken = weight.copy()
    broken[3, 70] = np.inf
    broken[5, 200] = np.nan
    scales, _ = scalar_encode.fit_scales(dev(broken), 64, asym=False, reciprocal=0.125, value_minimum=-8.0,
                                         scale_format="fp16", store_zero=False)
    scales = host(scales)
    assert np.isnan(scales[3, 1]) and np.isnan(scales[5, 3])
    assert np.isfinite(np.delete(scales.reshape(-1), [3 * 10 + 1, 5 * 10 + 3])).all()


@pytest.mark.parametrize("rows,width,group,values,integer,asym,fmt", [
    (64, 512, 64, SEVEN, False, False, "fp16"),
    (64, 512, 128, INT4, True, False, "fp16"),
    (32, 480, 32, INT3, True, True, "bf16"),
    (16, 200, 48, scaling.NF4_VALUES, False, False, "fp8"),
    (8, 1024, 1024, INT4, True, False, "fp32"),
    (16, 200, 50, INT4, True, False, "fp16"),
])
def test_search_scales_matches_oracle(rows, width, group, values, integer, asym, fmt):
    from mlkit_amd.kernels import scalar_encode

    weight = helpers.normal_weight(rows, width, seed=width + group, student_t=True)
    scales, zero = scaling.initial_scales(weight, values, group, asym)
    scales, _ = scaling.store_scale(scales, fmt)
    expected = scaling.search_scales(weight, scales, zero, values, FRACTIONS, group, fmt, integer)
    selected = scalar_encode.search_scales(dev(weight), dev(scales), dev(zero), dev(values), dev(FRACTIONS),
                                           group, None, fmt, integer=integer, minimum=float(values.min()),
                                           maximum=float(values.max()))
    np.testing.assert_array_equal(host(selected), expected)
    assert (expected != scales).mean() > 0.2  # the search does move scales


def test_feedback_codec_scale_indexing():
    from mlkit_amd.kernels import scalar_decode

    rng = np.random.default_rng(5)
    rows, width, group, refit = 24, 448, 64, 192   # last region narrower (64 columns)
    per_region = -(-refit // group)
    groups = (width // refit) * per_region + 1
    codes = rng.integers(0, 16, (rows, width), dtype=np.uint8)
    scales = rng.random((rows, groups), dtype=F32) + F32(0.5)
    zeros = rng.standard_normal((rows, groups)).astype(F32)
    expected = scaling.decode_feedback(codes, scales, INT4, group, refit, zeros)
    decoded = scalar_decode.decode(dev(codes), dev(scales), dev(INT4), dev(zeros), group, refit=refit)
    np.testing.assert_array_equal(host(decoded), expected)


def test_snap_matches_nearest_entry():
    from mlkit_amd.kernels import scalar_encode

    rng = np.random.default_rng(6)
    value = (rng.standard_normal((37, 129)) * 0.7).astype(F32)
    value[0, :7] = [0.75, -0.75, 0.375, 0.125, -0.125, 5.0, -5.0]
    snapped = scalar_encode.snap(dev(value), dev(SEVEN))
    expected = SEVEN[scaling.nearest_codes(value, SEVEN)]
    np.testing.assert_array_equal(host(snapped), expected)


def test_large_layer_round_trip_properties():
    """Full-size 4096x14336 INT4-g128: codes in range, half-step error bound, and decode
    of encode is idempotent (re-encoding the reconstruction returns the same codes)."""
    from mlkit_amd.kernels import scalar_decode, scalar_encode

    generator = torch.Generator(device="cuda").manual_seed(11)
    weight = (torch.randn((4096, 14336), device="cuda", generator=generator) * 0.02).half().float()
    values = dev(INT4)
    scales, _ = scalar_encode.fit_scales(weight, 128, asym=False, reciprocal=0.125, value_minimum=-8.0,
                                         scale_format="fp16", store_zero=False)
    codes = scalar_encode.encode(weight, scales, None, values, 128, None, integer=True, minimum=-8.0, maximum=7.0)
    decoded = scalar_decode.decode(codes, scales, values, None, 128)
    assert int(codes.max()) <= 15
    bound = scales.repeat_interleave(128, dim=1) * 0.5
    inside = weight.abs() <= scales.repeat_interleave(128, dim=1) * 7.0
    assert bool(((weight - decoded).abs() <= bound * 1.0001)[inside].all())
    again = scalar_encode.encode(decoded, scales, None, values, 128, None, integer=True, minimum=-8.0, maximum=7.0)
    assert torch.equal(again, codes)


def _activation_formats():
    import mlkit_amd as mk

    return {
        "int3-g32": mk.int(3, group=32),
        "int4-row": mk.int(4, group=None),
        "int4-fp32": mk.int(4, group=32, scale_fmt="fp32"),
        "nf4-g64": mk.nf4(group=64),
        "mxfp4": mk.mxfp4(),
        "int4-asymmetric": mk.int(4, group=32, asym=True),
        "int4-asymmetric-fp32": mk.int(4, group=32, asym=True, scale_fmt="fp32"),
        "int4-bf16": mk.int(4, group=32, scale_fmt="bf16"),
        "int4-fp8": mk.int(4, group=32, scale_fmt="fp8"),
        "e2m1-fp16": mk.scaled(mk.grid.fp("e2m1"), group=32),
    }


@pytest.mark.parametrize("name", ["int3-g32", "int4-row", "int4-fp32", "nf4-g64", "mxfp4", "int4-asymmetric",
                                  "int4-asymmetric-fp32", "int4-bf16", "int4-fp8", "e2m1-fp16"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_fused_activation_reconstruction_is_exact_on_rounding_ties(name, dtype):
    """The reference's own test (tests/kernels/test_activation_reconstruction.py:20-40): half
    precision inputs land on exact rounding ties; the fused kernel must equal the fitted
    format (itself checked against the oracle above) on every element."""
    fmt = _activation_formats()[name]
    generator = torch.Generator(device="cuda").manual_seed(97)
    inputs = torch.randn(512, 2050, dtype=dtype, device="cuda", generator=generator)
    inputs *= torch.rand(512, 1, device="cuda", generator=generator) * 20 + 0.01
    expected = fmt(inputs.float()).w.to(dtype)
    result = fmt.reconstruct_activations(inputs)
    assert result.dtype == dtype
    mismatched = int((result != expected).sum())
    assert mismatched == 0, f"{mismatched} of {result.numel()} elements differ"
    small = torch.randn(7, 130, dtype=dtype, device="cuda", generator=generator)
    torch.testing.assert_close(fmt.reconstruct_activations(small), fmt(small.float()).w.to(dtype), rtol=0, atol=0)


def test_activation_reconstruction_matches_oracle_directly():
    import mlkit_amd as mk

    value = helpers.normal_weight(33, 512, seed=40, scale=1.0)
    expected = scaling.quantize(value, INT4, group=64, integer=True, asym=True)
    dense = scaling.decode_grouped(expected["codes"], expected["scales"], INT4, 64, expected["zero"])
    result = mk.int(4, group=64, asym=True).reconstruct_activations(dev(value))
    np.testing.assert_array_equal(host(result), dense)
