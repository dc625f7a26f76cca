"""GPU parity (through the C ABI) of the error-feedback kernels against the C oracle:
reconstructions, codes, solved continuations and the trailing update bit for bit."""

import numpy as np
import pytest
import torch

from oracle import feedback as oracle_feedback, scaling

import helpers

pytestmark = pytest.mark.gpu

F32 = np.float32
INT4 = scaling.int_values(4)
SEVEN = np.array([-1, -0.5, -0.25, 0, 0.25, 0.5, 1], dtype=F32)


def dev(array):
    return None if array is None else torch.from_numpy(np.ascontiguousarray(array)).cuda()


def host(tensor):
    torch.cuda.synchronize()
    return tensor.cpu().numpy()


def problem(rows, width, seed, samples=None):
    """Weights and the unit upper coefficient matrix of a correlated synthetic Hessian."""
    rng = np.random.default_rng(seed)
    weight = helpers.normal_weight(rows, width, seed=seed)
    samples = samples or 2 * width
    inputs = rng.standard_normal((samples, width)).astype(F32)
    inputs[:, ::7] *= 4
    inputs += 0.5 * np.roll(inputs, 1, axis=1)
    hessian = (inputs.T @ inputs / samples).astype(F32)
    coeff, status = oracle_feedback.coefficients(hessian, 0.01)
    assert status == 0
    return weight, coeff, hessian


@pytest.mark.parametrize("rows,width,tile_start,tile_width,group,values,integer,asym", [
    (71, 96, 0, 96, 32, INT4, True, False),          # the reference's own tile test shape
    (64, 256, 128, 128, 128, INT4, True, False),
    (64, 256, 0, 128, 64, INT4, True, True),
    (35, 512, 128, 200, 128, INT4, True, False),     # four-slot kernel
    (19, 640, 64, 300, 50, INT4, True, True),        # sixteen-slot kernel, ragged groups
    (64, 256, 128, 128, 64, scaling.NF4_VALUES, False, False),
    (33, 128, 0, 100, 128, SEVEN, False, True),
    # tables of 17 to 256 values: the sixteen lanes of a row search the table together
    (64, 256, 128, 128, 64, np.sinh(np.linspace(-3, 3, 256)).astype(F32), False, False),
    (37, 256, 0, 128, 32, np.sinh(np.linspace(-3, 3, 256)).astype(F32), False, True),
    (50, 384, 128, 100, 128, (np.linspace(-1, 1, 40) ** 3).astype(F32), False, False),   # ragged tile, 40 values
    (16, 128, 0, 128, 128, np.linspace(-1, 1, 17).astype(F32), False, True),              # 17 values: ties to the lower entry
])
def test_round_tile_matches_oracle(rows, width, tile_start, tile_width, group, values, integer, asym):
    from mlkit_amd.kernels import error_feedback

    weight, coeff, _ = problem(rows, width, seed=rows + tile_width)
    rng = np.random.default_rng(1)
    feedback = (rng.standard_normal((rows, width)) * 0.004).astype(F32)
    region_start = tile_start - (group if tile_start >= group and tile_start % group == 0 else 0)
    region = weight[:, region_start:tile_start + tile_width]
    scales, zeros = oracle_feedback.fit_scales(region, values, group, asym)
    expected_out = np.zeros_like(weight)
    expected_codes = np.zeros(weight.shape, dtype=np.uint8)
    oracle_feedback.round_tile(weight, feedback, coeff, scales, zeros, values, expected_out, expected_codes,
                               region_start=region_start, tile_start=tile_start, tile_width=tile_width,
                               group=group, integer=integer)
    output = torch.zeros((rows, width), device="cuda")
    encoded = torch.zeros((rows, width), device="cuda", dtype=torch.uint8)
    bits = 4 if integer else int(np.ceil(np.log2(len(values))))
    error_feedback.round_tile(dev(weight), dev(feedback), dev(coeff), dev(scales), dev(zeros), output, encoded,
                              region_start=region_start, tile_start=tile_start, tile_width=tile_width,
                              group=group, bits=bits, values=dev(values), integer_grid=integer)
    np.testing.assert_array_equal(host(encoded), expected_codes)
    np.testing.assert_array_equal(host(output), expected_out)


@pytest.mark.parametrize("asym", [False, True])
@pytest.mark.parametrize("tile_width", [128, 96])
def test_round_tile_on_quotients_next_to_half_integers(asym, tile_width):
    """Every target of the tile divides by its scale to k + 1/2 exactly, or to the fp32 numbers right next to
    it on either side: the cases in which the correctly rounded quotient, and not a product with the scale's
    reciprocal, decides the code (a sweep that multiplied by reciprocals would miss a few per cent of these
    codes, as the last assertion shows).  No feedback and no coefficients, so that every column is such a
    case; codes and reconstructions equal the oracle's (true division, round half to even)."""
    from mlkit_amd.kernels import error_feedback

    rows, width, group = 192, 256, 64
    rng = np.random.default_rng(31 + tile_width)
    scales = (rng.random((rows, width // group)) * 0.05 + 0.002).astype(np.float16).astype(F32)
    scales[::3] = (2.0 ** rng.integers(-9, -3, (len(scales[::3]), width // group))).astype(F32)     # exact ties
    zeros = (rng.standard_normal((rows, width // group)) * 0.01).astype(np.float16).astype(F32) if asym else None
    halves = rng.integers(-9, 9, (rows, width)).astype(F32) + F32(0.5)
    wide = np.repeat(scales, group, axis=1)
    weight = (halves * wide).astype(F32)
    if asym:
        weight = (weight + np.repeat(zeros, group, axis=1)).astype(F32)
    nudge = rng.integers(-2, 3, (rows, width))
    weight = np.where(nudge < 0, np.nextafter(weight, F32(-np.inf)), np.where(nudge > 0, np.nextafter(weight, F32(np.inf)), weight)).astype(F32)
    weight[5, 7] = np.nan                                             # a value that is not a number takes the division, too
    feedback = np.zeros_like(weight)
    coeff = np.eye(width, dtype=F32)
    expected_out = np.zeros_like(weight)
    expected_codes = np.zeros(weight.shape, dtype=np.uint8)
    oracle_feedback.round_tile(weight, feedback, coeff, scales, zeros, INT4, expected_out, expected_codes,
                               region_start=0, tile_start=64, tile_width=tile_width, group=group, integer=True)
    output = torch.zeros((rows, width), device="cuda")
    encoded = torch.zeros((rows, width), device="cuda", dtype=torch.uint8)
    error_feedback.round_tile(dev(weight), dev(feedback), dev(coeff), dev(scales), None if zeros is None else dev(zeros), output,
                              encoded, region_start=0, tile_start=64, tile_width=tile_width, group=group, bits=4,
                              values=dev(INT4), integer_grid=True)
    keep = np.ones(weight.shape, dtype=bool)
    keep[5, 7] = False
    np.testing.assert_array_equal(host(encoded)[keep], expected_codes[keep])
    np.testing.assert_array_equal(host(output)[keep], expected_out[keep])
    # the crafted cases really sit at the boundaries: a product with the reciprocal alone would miss some codes
    inside = slice(64, 64 + tile_width)
    centered = weight[:, inside] - (np.repeat(zeros, group, axis=1)[:, inside] if asym else 0)
    by_reciprocal = np.clip(np.rint((centered.astype(F32) * (F32(1) / wide[:, inside])).astype(F32)), -8, 7) + 8
    assert (by_reciprocal[keep[:, inside]] != expected_codes[:, inside][keep[:, inside]]).sum() > 0


@pytest.mark.parametrize("rows,width,start,stop", [(64, 384, 128, 256), (37, 512, 192, 492), (16, 1024, 0, 1024)])
def test_pending_continuation_matches_oracle(rows, width, start, stop):
    from mlkit_amd.kernels import error_feedback

    weight, coeff, _ = problem(rows, width, seed=width + start)
    rng = np.random.default_rng(2)
    feedback = (rng.standard_normal((rows, width)) * 0.01).astype(F32)
    expected = oracle_feedback.pending(feedback, coeff, start, stop)
    solved = error_feedback.pending_continuation(dev(feedback), dev(coeff), start, stop)
    np.testing.assert_array_equal(host(solved), expected)
    targets = error_feedback.pending_continuation(dev(feedback), dev(coeff), start, stop, original=dev(weight))
    np.testing.assert_array_equal(host(targets), (weight[:, start:stop] + expected).astype(F32))
    # the textbook definition: x U = feedback[:, region]
    block = coeff[start:stop, start:stop].astype(np.float64)
    np.testing.assert_allclose(expected @ block, feedback[:, start:stop], rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("rows,width,start,stop", [(128, 512, 0, 128), (200, 700, 128, 256), (71, 333, 64, 101),
                                                   (64, 256, 0, 255)])
def test_block_update_matches_fma_chain(rows, width, start, stop):
    from mlkit_amd.kernels import error_feedback

    weight, coeff, _ = problem(rows, width, seed=width + stop)
    rng = np.random.default_rng(3)
    output = (weight + rng.standard_normal(weight.shape).astype(F32) * 0.003).astype(F32)
    feedback = (rng.standard_normal(weight.shape) * 0.01).astype(F32)
    expected = feedback.copy()
    oracle_feedback.block_update(expected, weight, output, coeff, start, stop, mode=0)
    updated = dev(feedback)
    error_feedback.block_update(updated, dev(weight), dev(output), dev(coeff), start, stop)
    np.testing.assert_array_equal(host(updated), expected)
    exact = feedback[:, stop:].astype(np.float64) + (weight - output)[:, start:stop].astype(np.float64) @ coeff[start:stop, stop:].astype(np.float64)
    np.testing.assert_allclose(host(updated)[:, stop:], exact, rtol=1e-4, atol=1e-6)
    np.testing.assert_array_equal(host(updated)[:, :stop], feedback[:, :stop])


@pytest.mark.parametrize("rows,width,first,chain,chains,begin,end", [
    (130, 1024, 0, 128, 4, 512, 1024),     # a deferred super-block reaching the far columns
    (64, 700, 64, 96, 3, 352, 700),        # ragged widths, unaligned end
    (64, 640, 128, 128, 1, 256, 384),      # the narrow update inside a super-block
    (33, 333, 10, 50, 2, 111, 333),        # nothing aligned: scalar loads
])
def test_chained_block_update_equals_tile_after_tile(rows, width, first, chain, chains, begin, end):
    from mlkit_amd.kernels import error_feedback

    weight, coeff, _ = problem(rows, width, seed=width + chains)
    rng = np.random.default_rng(4)
    output = (weight + rng.standard_normal(weight.shape).astype(F32) * 0.003).astype(F32)
    feedback = (rng.standard_normal(weight.shape) * 0.01).astype(F32)
    expected = feedback.copy()
    for index in range(chains):   # the oracle applies one tile at a time to every later column
        start = first + index * chain
        scratch = expected.copy()
        oracle_feedback.block_update(scratch, weight, output, coeff, start, start + chain, mode=0)
        expected[:, begin:end] = scratch[:, begin:end]
    updated = dev(feedback)
    error_feedback.block_update_range(updated, dev(weight), dev(output), dev(coeff), first, chain, chains, begin, end)
    np.testing.assert_array_equal(host(updated), expected)


@pytest.mark.parametrize("rows,width,first,chain,chains,begin,end", [
    (2048, 5120, 0, 128, 4, 512, 5120),     # 576 tiles: a whole round of 512 on large tiles, 64 as quarter tiles
    (1024, 9216, 128, 128, 2, 384, 9216),   # 552 tiles, two chains
    (2048, 5120, 0, 256, 2, 512, 5120),     # chains of 256 columns: large tiles throughout
    (256, 1024, 0, 128, 4, 512, 1024),      # fewer tiles than slots
    (256, 640, 128, 128, 1, 256, 512),      # one chain over a few tiles: quarter tiles only
])
def test_update_from_kept_deviations_equals_the_recomputing_update(rows, width, first, chain, chains, begin, end):
    """mk_feedback_block_update_staged (deviations handed over column-major; whole rounds on
    128 x 128 tiles, a short last round as 64 x 64 tiles) against mk_feedback_block_update_range,
    which the test above pins to the oracle: the same sums, bit for bit."""
    from mlkit_amd import native
    from mlkit_amd.kernels import error_feedback

    generator = torch.Generator(device="cuda").manual_seed(rows + width)
    weight = torch.randn((rows, width), device="cuda", generator=generator) * 0.02
    output = weight + torch.randn((rows, width), device="cuda", generator=generator) * 0.003
    coeff = torch.randn((width, width), device="cuda", generator=generator).triu(1) * 0.05
    feedback = torch.randn((rows, width), device="cuda", generator=generator) * 0.01
    expected = feedback.clone()
    error_feedback.block_update_range(expected, weight, output, coeff, first, chain, chains, begin, end)
    deviations = (weight - output).T.contiguous()
    updated = feedback.clone()
    native.check(native.library().mk_feedback_block_update_staged(
        updated.data_ptr(), deviations.data_ptr(), coeff.data_ptr(), rows, width, first, chain, chains, begin, end,
        native.current_stream(updated.device)))
    assert torch.equal(updated, expected)
    assert torch.equal(updated[:, :begin], feedback[:, :begin])


@pytest.mark.parametrize("width,step", [(1024, 1), (1100, 1), (1536, 8), (2304, 1)])
def test_blocked_factorisation_matches_the_float64_coefficients(width, step):
    """`feedback_coefficients` on the device factors matrices of 1024 columns and more block by
    block (`mk_cholesky_block` plus matrix products).  Against the float64 definition at the
    reference's tolerance (tests/quantization/test_algorithms.py:142-166, rtol 1e-3 on the
    upper triangle), and against the library factorisation of the same matrix."""
    import mlkit_amd as mk

    rng = np.random.default_rng(width)
    inputs = rng.standard_normal((2 * width, width)).astype(np.float32)
    inputs[:, ::13] *= 6
    inputs[:, 5] = 0   # a dead channel
    hessian = (inputs.T @ inputs / inputs.shape[0]).astype(np.float32)
    result, status = mk.feedback_coefficients(dev(hessian).clone(), step)
    assert status == 0
    expected, expected_status = oracle_feedback.coefficients(hessian) if step == 1 else (None, 0)
    assert expected_status == 0
    if step == 1:
        upper = np.triu(np.ones((width, width), dtype=bool), 1)
        np.testing.assert_allclose(host(result)[upper], expected[upper], rtol=1e-3, atol=2e-6)
    library, library_status = mk.feedback_coefficients(torch.from_numpy(hessian).clone(), step)   # CPU: LAPACK
    assert library_status == 0
    blocks = np.kron(np.eye(width // step, dtype=bool), np.ones((step, step), dtype=bool))
    outside = np.triu(np.ones((width, width), dtype=bool), 1) & ~blocks
    np.testing.assert_allclose(host(result)[outside], library.numpy()[outside], rtol=1e-3, atol=2e-6)


@pytest.mark.parametrize("width", [1664, 2304])
def test_look_ahead_factorisation_equals_the_one_stream_order(width, monkeypatch):
    """From `LOOK_AHEAD_WIDTH` columns on, the far part of every trailing update runs on a second
    stream; events keep the order in which updates reach an entry, so the coefficients (the
    entries above the diagonal; below it both leave leftovers) are the same bit for bit.
    Twice, because a race would not show every time."""
    import mlkit_amd as mk
    from mlkit_amd.quantization import feedback

    rng = np.random.default_rng(width + 1)
    inputs = rng.standard_normal((2 * width, width)).astype(np.float32)
    inputs[:, ::7] *= 4
    hessian = dev((inputs.T @ inputs / inputs.shape[0]).astype(np.float32))
    monkeypatch.setattr(feedback, "FACTOR_GRAPHS", False)       # launch by launch, with the constants set here
    monkeypatch.setattr(feedback, "FACTORIZATION_PANEL", 256)   # several panels at these widths
    monkeypatch.setattr(feedback, "LOOK_AHEAD_WIDTH", 1 << 30)
    expected, status = mk.feedback_coefficients(hessian.clone(), 1)
    assert status == 0
    monkeypatch.setattr(feedback, "LOOK_AHEAD_WIDTH", 1024)
    for _ in range(2):
        result, status = mk.feedback_coefficients(hessian.clone(), 1)
        assert status == 0
        np.testing.assert_array_equal(np.triu(host(result), 1), np.triu(host(expected), 1))


@pytest.mark.parametrize("look_ahead", [False, True])
def test_captured_factorisation_equals_the_launch_by_launch_one(look_ahead, monkeypatch):
    """From the second matrix of a width on, the factorisation replays a captured graph.  Five
    different matrices of one width, with eager work and synchronisations between the replays and
    another width in between: every result equals the one computed launch by launch, bit for bit
    above the diagonal; an indefinite matrix reports its column through the graph as well."""
    import mlkit_amd as mk
    from mlkit_amd.quantization import feedback

    feedback.clear_factor_graphs()
    monkeypatch.setattr(feedback, "FACTORIZATION_PANEL", 512)
    monkeypatch.setattr(feedback, "LOOK_AHEAD_WIDTH", 1024 if look_ahead else 1 << 30)
    width = 1664
    generator = torch.Generator(device="cuda").manual_seed(11)

    def hessian_of(scale):
        inputs = torch.randn((2 * width, width), device="cuda", generator=generator) * scale
        inputs[:, ::9] *= 3
        return inputs.T @ inputs / inputs.shape[0]

    try:
        matrices = [hessian_of(1.0 + 0.5 * index) for index in range(5)]
        monkeypatch.setattr(feedback, "FACTOR_GRAPHS", False)
        expected = [mk.feedback_coefficients(matrix.clone(), 1)[0] for matrix in matrices]
        monkeypatch.setattr(feedback, "FACTOR_GRAPHS", True)
        other = hessian_of(2.0)[:1280, :1280].contiguous()
        for index, matrix in enumerate(matrices):
            result, status = mk.feedback_coefficients(matrix.clone(), 1)
            assert status == 0
            assert torch.equal(result.triu(1), expected[index].triu(1)), index
            busy = (matrix @ matrix).sum()            # eager work and a synchronisation between replays
            torch.cuda.synchronize()
            assert torch.isfinite(busy)
            if index == 2:
                mk.feedback_coefficients(other.clone(), 1)   # another width in between
        assert feedback._factor_graphs[(0, width)] is not None
        broken = matrices[0].clone()
        broken[900, 900] = -1e6
        assert mk.feedback_coefficients(broken, 1, damp=0.0)[1] != 0
        assert mk.feedback_coefficients(matrices[1].clone(), 1)[1] == 0   # the status starts from zero again
    finally:
        feedback.clear_factor_graphs()


def test_blocked_factorisation_reports_an_indefinite_matrix():
    import mlkit_amd as mk

    width = 1280
    rng = np.random.default_rng(3)
    inputs = rng.standard_normal((width // 2, width)).astype(np.float32)   # rank deficient
    hessian = (inputs.T @ inputs).astype(np.float32)
    hessian[700, 700] = -5000.0
    _, status = mk.feedback_coefficients(dev(hessian).clone(), 1, damp=0.0)
    assert status != 0
    quantizer = mk.gptq(mk.int(4, group=128))
    with pytest.raises(ValueError, match="positive definite"):
        quantizer(dev(np.zeros((8, width), dtype=np.float32)), mk.Ctx("layer", H=dev(hessian)))
