"""GPU parity of the vector grids: nearest-codeword search (E8P structured search and
exhaustive codebooks) and the LDL feedback tile that rounds blocks of columns, against the
oracle, bit for bit; then the public API (`mk.scaled` over `mk.grid.vector` / `mk.grid.e8p`,
`mk.ldlq(step=dimension)`) against the oracle's sweep and in the shape of the reference's
own tests (/root/reference/tests/kernels/test_error_feedback.py:67-130,
tests/quantization/test_lattice.py)."""

import numpy as np
import pytest
import torch

import mlkit_amd as mk
from mlkit_amd.quantization.core import Ctx
from oracle import lattice as oracle_lattice

import helpers

pytestmark = pytest.mark.gpu

F32 = np.float32


def dev(array):
    return None if array is None else torch.from_numpy(np.ascontiguousarray(array)).cuda()


def host(tensor):
    torch.cuda.synchronize()
    return tensor.cpu().numpy()


def codebook_of(entries, dimension, seed):
    return np.random.default_rng(seed).standard_normal((entries, dimension)).astype(F32)


def calibrated(rows, width, seed, step):
    rng = np.random.default_rng(seed)
    weight = helpers.normal_weight(rows, width, seed=seed)
    inputs = rng.standard_normal((3 * width, width)).astype(F32)
    inputs[:, ::7] *= 4
    inputs += 0.5 * np.roll(inputs, 1, axis=1)
    hessian = (inputs.T @ inputs / len(inputs)).astype(F32)
    return weight, hessian


# ---- search ---------------------------------------------------------------------------


def test_lattice_search_matches_oracle_codes():
    from mlkit_amd.kernels import lattice_search
    from mlkit_amd.quantization.lattice import device_table

    rng = np.random.default_rng(5)
    points = oracle_lattice.e8p_points()
    samples = np.concatenate([
        rng.standard_normal((20000, 8)).astype(F32) * F32(1.2),
        rng.standard_normal((2000, 8)).astype(F32) * F32(4.0),            # beyond the outer shell
        np.zeros((3, 8), dtype=F32),                                      # equidistant from many points
        points[rng.integers(0, 65536, 500)],                              # lattice points themselves
        ((points[rng.integers(0, 65536, 500)] + points[rng.integers(0, 65536, 500)]) * F32(0.5)).astype(F32),
        np.round(rng.standard_normal((500, 8)) * 2).astype(F32) * F32(0.5),   # half-integers: many exact ties
    ])
    expected = oracle_lattice.nearest_e8p_codes(samples)
    codes = host(lattice_search.search(dev(samples), device_table(torch.device("cuda", 0))))
    np.testing.assert_array_equal(codes, expected)


def test_lattice_table_on_device_is_the_oracle_point_set():
    from mlkit_amd.quantization.lattice import device_table

    table = host(device_table(torch.device("cuda", 0)))
    np.testing.assert_array_equal(table[:65536], oracle_lattice.e8p_points())
    np.testing.assert_array_equal(table[65536:], oracle_lattice.absolute_points())


@pytest.mark.parametrize("entries,dimension,count", [(256, 8, 5000), (600, 4, 5000), (37, 2, 3000), (1000, 16, 2000),
                                                      (65536, 8, 96), (1, 4, 40)])
def test_codebook_search_matches_oracle_codes(entries, dimension, count):
    from mlkit_amd.kernels import lattice_search

    codebook = codebook_of(entries, dimension, seed=entries + dimension)
    if entries >= 37:
        codebook[30] = codebook[4]       # duplicates: the lower index must win
        codebook[-1] = codebook[11]
    rng = np.random.default_rng(count)
    samples = rng.standard_normal((count, dimension)).astype(F32)
    samples[:20] = codebook[rng.integers(0, entries, 20)]
    if entries >= 37:
        samples[20], samples[21] = codebook[4], codebook[11]
    expected = oracle_lattice.nearest_codes(samples, codebook)
    codes = host(lattice_search.nearest(dev(samples), dev(codebook)))
    np.testing.assert_array_equal(codes, expected)
    if entries >= 37:
        assert codes[20] == 4 and codes[21] == 11


def test_nearest_returns_codewords_or_indices_and_handles_other_dimensions():
    codebook = torch.randn(50, 8, device="cuda")
    samples = torch.randn(200, 8, device="cuda")
    indices = mk.nearest(samples, codebook, return_indices=True)
    assert indices.dtype == torch.int64
    torch.testing.assert_close(mk.nearest(samples, codebook), codebook[indices], rtol=0, atol=0)
    odd = torch.randn(40, 3, device="cuda")      # three coordinates: tensor operations on the device
    found = mk.nearest(samples[:, :3].contiguous(), odd, return_indices=True)
    expected = oracle_lattice.nearest_codes(host(samples[:, :3]), host(odd))
    assert (host(found) == expected).mean() > 0.99
    scalar = torch.tensor([[0.5], [-1.0], [0.5], [2.0]], device="cuda")
    picked = mk.nearest(torch.tensor([[0.4], [10.0], [-0.25]], device="cuda"), scalar, return_indices=True)
    assert picked.tolist() == [0, 3, 0]          # -0.25 is equally far from -1.0 and 0.5: the lower index
    with pytest.raises(ValueError, match="equal vector dimensions"):
        mk.nearest(samples, odd)


def test_e8p_grid_rounds_to_the_optimal_point():
    # the reference's tests/quantization/test_lattice.py:7-23
    from mlkit_amd.quantization.lattice import absolute_points, e8p_points, nearest_e8p

    assert absolute_points().shape == (256, 8)
    points = e8p_points()
    assert points.shape == (65536, 8) and len(points.unique(dim=0)) == 65536
    samples = torch.randn(17, 8, device="cuda", generator=torch.Generator(device="cuda").manual_seed(61))
    result = mk.grid.e8p()(samples)
    indices = nearest_e8p(samples, return_indices=True)
    torch.testing.assert_close(points.cuda()[indices.long()], result, rtol=0, atol=0)
    brute = mk.nearest(samples, points.cuda())
    torch.testing.assert_close((samples - result).square().sum(1), (samples - brute).square().sum(1),
                               rtol=1e-5, atol=1e-6)
    # the device kernel and the tensor-operation search reach the same cost (test_lattice.py:26-35)
    more = torch.randn(1024, 8)
    torch.testing.assert_close((more - nearest_e8p(more.cuda()).cpu()).square().sum(1),
                               (more - nearest_e8p(more, backend="torch")).square().sum(1), rtol=1e-5, atol=1e-5)
    with pytest.raises(ValueError, match="HIP device"):
        nearest_e8p(more, backend="hip")


# ---- the feedback tile ----------------------------------------------------------------


@pytest.mark.parametrize("name,rows,width,tile_start,tile_width,group,dimension,entries", [
    ("lattice", 37, 256, 0, 128, 256, 8, 65536),
    ("lattice", 64, 512, 256, 256, 32, 8, 65536),       # the widest tile, grouped scales
    ("lattice", 5, 96, 32, 40, 32, 8, 65536),           # a ragged last tile
    ("octets", 48, 256, 128, 128, 128, 8, 256),
    ("quadruples", 33, 128, 0, 100, 16, 4, 600),
    ("pairs", 20, 192, 64, 128, 64, 2, 50),
    ("sixteens", 9, 256, 0, 256, 64, 16, 300),
])
def test_round_vector_tile_matches_oracle(name, rows, width, tile_start, tile_width, group, dimension, entries):
    from mlkit_amd.kernels import error_feedback
    from mlkit_amd.quantization.lattice import device_table

    lattice = name == "lattice"
    weight, hessian = calibrated(rows, width, seed=rows + tile_width, step=dimension)
    coefficients, status = mk.feedback_coefficients(dev(hessian).clone(), dimension)   # an input of both sides
    assert int(status) == 0
    coeff = host(coefficients)
    rng = np.random.default_rng(2)
    feedback = (rng.standard_normal((rows, width)) * 0.004).astype(F32)
    codebook = oracle_lattice.e8p_points() if lattice else codebook_of(entries, dimension, seed=entries)
    region_start = max(0, (tile_start // group - 1) * group)
    magnitude = np.abs(codebook).max()
    groups = -(-(width - region_start) // group)
    padded = np.zeros((rows, groups * group), dtype=F32)
    padded[:, :width - region_start] = weight[:, region_start:]
    scales = (np.abs(padded.reshape(rows, groups, group)).max(2) / magnitude).astype(F32)
    expected_out = np.zeros_like(weight)
    expected_codes = np.zeros((rows, width // dimension), dtype=np.int32)
    oracle_lattice.round_vector_tile(weight, feedback, coeff, scales, codebook, expected_out, expected_codes,
                                     region_start=region_start, tile_start=tile_start, tile_width=tile_width,
                                     group=group, dimension=dimension, lattice=lattice)
    output = torch.zeros((rows, width), device="cuda")
    encoded = torch.zeros((rows, width // dimension), device="cuda", dtype=torch.int32)
    table = device_table(torch.device("cuda", 0)) if lattice else dev(codebook)
    error_feedback.round_vector_tile(dev(weight), dev(feedback), dev(coeff), dev(scales), table, output, encoded,
                                     region_start=region_start, tile_start=tile_start, tile_width=tile_width,
                                     group=group, dimension=dimension, codebook_size=entries, lattice=lattice)
    np.testing.assert_array_equal(host(encoded), expected_codes)
    np.testing.assert_array_equal(host(output), expected_out)


def test_round_vector_tile_answers_code_zero_for_values_that_are_not_numbers():
    """No distance of a NaN vector compares below infinity: the code is 0 and the reconstruction is code 0's
    table point times the scale (the reference reconstructs ``table[0]`` there), in the first block of a row
    and, through the corrections, in every later block of that row; other rows are untouched."""
    from mlkit_amd.kernels import error_feedback
    from mlkit_amd.quantization.lattice import device_table

    rows, width = 6, 64
    weight, hessian = calibrated(rows, width, seed=77, step=8)
    weight[2, 3] = np.nan
    coefficients, status = mk.feedback_coefficients(dev(hessian).clone(), 8)
    assert int(status) == 0
    scales = np.full((rows, 1), 0.01, dtype=F32)
    points = oracle_lattice.e8p_points()
    for lattice, table, entries in ((True, device_table(torch.device("cuda", 0)), 65536),
                                    (False, dev(codebook_of(256, 8, seed=1)), 256)):
        output = torch.full((rows, width), 7.0, device="cuda")
        encoded = torch.full((rows, width // 8), 9, device="cuda", dtype=torch.int32)
        error_feedback.round_vector_tile(dev(weight), torch.zeros((rows, width), device="cuda"), coefficients, dev(scales),
                                         table, output, encoded, region_start=0, tile_start=0, tile_width=width, group=width,
                                         dimension=8, codebook_size=entries, lattice=lattice)
        first = points[0] if lattice else codebook_of(256, 8, seed=1)[0]
        assert host(encoded)[2].tolist() == [0] * (width // 8)
        np.testing.assert_array_equal(host(output)[2].reshape(-1, 8), np.tile(first * F32(0.01), (width // 8, 1)))
        assert np.isfinite(host(output)).all() and (host(encoded)[[0, 1, 3, 4, 5]] != 9).all()


def test_round_vector_tile_refuses_what_the_kernel_does_not_cover():
    from mlkit_amd.kernels import error_feedback

    rows, width = 4, 512
    tensors = [torch.zeros((rows, width), device="cuda") for _ in range(2)]
    coeff = torch.eye(width, device="cuda")
    scales = torch.ones((rows, 1), device="cuda")
    output = torch.zeros((rows, width), device="cuda")

    def call(dimension, tile_width, entries=16, tile_start=0):
        codebook = torch.zeros((entries, dimension), device="cuda")
        encoded = torch.zeros((rows, width // dimension), device="cuda", dtype=torch.int32)
        error_feedback.round_vector_tile(tensors[0], tensors[1], coeff, scales, codebook, output, encoded,
                                         region_start=0, tile_start=tile_start, tile_width=tile_width, group=width,
                                         dimension=dimension, codebook_size=entries, lattice=False)

    with pytest.raises(ValueError, match="at most 256 columns"):
        call(8, 512)
    with pytest.raises(ValueError, match="2, 4, 8 or 16"):
        call(32, 128)
    with pytest.raises(ValueError, match="whole codewords"):
        call(8, 100)
    with pytest.raises(ValueError, match="outside a row"):
        call(8, 128, tile_start=448)


# ---- the public API -------------------------------------------------------------------


FORMATS = {
    "lattice": (None, 8, None),
    "grouped-lattice": (None, 8, 32),
    "octets": ((256, 8), 8, None),
    "quadruples": ((600, 4), 4, 16),
}


def format_of(name):
    shape, dimension, group = FORMATS[name]
    if shape is None:
        return mk.scaled(mk.grid.e8p(), group=group), dimension, None
    codebook = codebook_of(*shape, seed=83)
    return mk.scaled(mk.grid.vector(torch.from_numpy(codebook)), group=group), dimension, codebook


@pytest.mark.parametrize("name", list(FORMATS))
@pytest.mark.parametrize("refit", [32, None])
def test_vector_ldlq_on_device_matches_oracle_sweep(name, refit):
    fmt, dimension, codebook = format_of(name)
    rows, width = 48, 256
    weight, hessian = calibrated(rows, width, seed=7, step=dimension)
    context = Ctx("layer", H=dev(hessian))
    result = mk.ldlq(fmt, step=dimension, refit=refit, backend="hip")(dev(weight), context)
    assert result.codec == "vector_feedback" and result.codes.dtype == torch.int32
    # the coefficient matrix is an input of the sweep: hand the oracle the very same one
    coeff = host(mk.feedback_coefficients(dev(hessian).clone(), dimension)[0])
    lattice = codebook is None
    expected = oracle_lattice.vector_sweep(weight, coeff, oracle_lattice.e8p_points() if lattice else codebook,
                                           group=fmt.group or width, dimension=dimension, lattice=lattice,
                                           refit=refit, block=128)
    np.testing.assert_array_equal(host(result.params["scales"]), expected["scales"])
    np.testing.assert_array_equal(host(result.codes), expected["codes"])
    np.testing.assert_array_equal(host(result.w), expected["w"])
    # the codec's decoder reproduces the reconstruction from codes and parameters alone
    from mlkit_amd.quantization.codecs import decoder

    np.testing.assert_array_equal(host(decoder("vector_feedback")(result.codes, **result.params)), expected["w"])
    side = 16 * expected["scales"].size
    assert result.bits == pytest.approx(fmt.grid.bits * rows * width / dimension + side)


@pytest.mark.parametrize("name", list(FORMATS))
@pytest.mark.parametrize("refit", [32, None])
def test_fused_vector_feedback_matches_block_by_block_rounding(name, refit):
    # /root/reference/tests/kernels/test_error_feedback.py:79-100
    fmt, dimension, _ = format_of(name)
    weight, hessian = calibrated(64, 256, seed=11, step=dimension)
    weights = dev(weight)
    expected = mk.ldlq(fmt, step=dimension, refit=refit, backend="torch")(weights, Ctx("layer", H=dev(hessian)))
    actual = mk.ldlq(fmt, step=dimension, refit=refit, backend="hip")(weights, Ctx("layer", H=dev(hessian)))
    assert actual.codec == expected.codec == "vector_feedback"
    assert actual.codes.dtype == expected.codes.dtype
    assert actual.bits == pytest.approx(expected.bits)
    assert actual.metadata == expected.metadata
    # feedback sums are ordered differently, so a rare near tie may select another codeword
    assert (actual.codes == expected.codes).float().mean() > 0.99
    torch.testing.assert_close(mk.proxy_loss(weights, actual.w, dev(hessian)),
                               mk.proxy_loss(weights, expected.w, dev(hessian)), rtol=1e-2, atol=0)


def test_fused_vector_feedback_requires_a_step_of_the_grid_dimension():
    # /root/reference/tests/kernels/test_error_feedback.py:103-110
    fmt, _, _ = format_of("lattice")
    weight, hessian = calibrated(32, 128, seed=3, step=16)
    with pytest.raises(ValueError, match="step equal to its dimension"):
        mk.ldlq(fmt, step=16, refit=None, backend="hip")(dev(weight), Ctx("layer", H=dev(hessian)))
    result = mk.ldlq(fmt, step=16, refit=None)(dev(weight), Ctx("layer", H=dev(hessian)))
    assert result.codec == "vector_feedback"


def test_fused_vector_feedback_reduces_the_loss_of_direct_rounding():
    # /root/reference/tests/kernels/test_error_feedback.py:113-121
    fmt, dimension, _ = format_of("lattice")
    weight, hessian = calibrated(64, 256, seed=13, step=dimension)
    weights = dev(weight)
    direct = fmt(weights, Ctx("layer", H=dev(hessian)))
    assert direct.codec == "vector_scaled"
    result = mk.ldlq(fmt, step=dimension, refit=None)(weights, Ctx("layer", H=dev(hessian)))
    assert mk.proxy_loss(weights, result.w, dev(hessian)) < mk.proxy_loss(weights, direct.w, dev(hessian))


def test_scaled_vector_grid_on_device_matches_oracle_round_to_nearest():
    rows, width, group = 40, 256, 64
    weight = helpers.normal_weight(rows, width, seed=21)
    for lattice in (True, False):
        codebook = oracle_lattice.e8p_points() if lattice else codebook_of(300, 8, seed=9)
        grid = mk.grid.e8p() if lattice else mk.grid.vector(torch.from_numpy(codebook))
        context = Ctx("layer")
        result = mk.scaled(grid, group=group)(dev(weight), context)
        scales = host(result.params["scales"])
        normalized = (weight.reshape(rows, -1, group) / scales[:, :, None]).astype(F32).reshape(-1, 8)
        expected = (oracle_lattice.nearest_e8p_codes(normalized) if lattice
                    else oracle_lattice.nearest_codes(normalized, codebook))
        np.testing.assert_array_equal(host(result.codes).reshape(-1), expected)
        np.testing.assert_array_equal(
            host(result.w), oracle_lattice.decode_vector_scaled(expected.reshape(rows, -1), scales, codebook, group, 8))
        assert result.params["values"] is None if lattice else result.params["values"].shape == (300, 8)
        assert context.additional_bits == (0 if lattice else 300 * 8 * 32)


def test_vector_codecs_survive_a_checkpoint_and_stay_dense_under_optimize(tmp_path):
    from torch import nn

    torch.manual_seed(44)

    def build():
        return nn.Sequential(nn.Linear(64, 48), nn.ReLU(), nn.Linear(48, 16, bias=False))

    codebook = torch.randn(64, 4)
    for fmt, values_kept in ((mk.scaled(mk.grid.e8p(), group=32), False), (mk.scaled(mk.grid.vector(codebook), group=16), True)):
        converted = mk.quantize(build(), fmt, calib=None)
        assert converted.quantized["0"].codec == "vector_scaled"
        inputs = torch.randn(4, 64)
        expected = converted(inputs)
        target = tmp_path / ("codebook" if values_kept else "lattice")
        mk.save(converted, target)
        restored = mk.load_checkpoint(target, model=build)
        torch.testing.assert_close(restored(inputs), expected, rtol=0, atol=0)
        entry = restored.quantized["0"]
        # codes come back in the narrowest integer type that holds `code_bits`
        assert entry.codec == "vector_scaled" and not entry.codes.is_floating_point() and entry.params["dim"] in (4, 8)
        assert (entry.params["values"] is not None) == values_kept
        assert entry.bits == converted.quantized["0"].bits
        # vector codes have no packed kernel: the optimizer keeps such layers dense
        packed = mk.optimize(restored)
        assert packed.execution_backend == "packed:0"
        with torch.inference_mode():
            torch.testing.assert_close(packed(inputs), expected, rtol=1e-4, atol=1e-5)
    # calibrated LDLQ over the lattice through the same driver
    calibrated_model = mk.quantize(build(), mk.ldlq(mk.scaled(mk.grid.e8p(), group=None), step=8),
                                   calib=[torch.randn(32, 64) for _ in range(4)])
    assert calibrated_model.quantized["0"].codec == "vector_feedback"
