"""GPU parity (through the C ABI) of the Walsh-Hadamard kernels against the oracle:
bit for bit against the stage-by-stage fp32 restatement, to 1e-4 against the Sylvester
matrix product in float64 (the reference's own bound, tests/quantization/test_operations.py:99-100)."""

import numpy as np
import pytest
import torch

from oracle import transforms

pytestmark = pytest.mark.gpu

F32 = np.float32


def dev(array):
    return torch.from_numpy(np.ascontiguousarray(array)).cuda()


def host(tensor):
    torch.cuda.synchronize()
    return tensor.float().cpu().numpy()


@pytest.mark.parametrize("width", [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384, 32768])
@pytest.mark.parametrize("normalize", [True, False])
def test_transform_is_bit_exact(width, normalize):
    from mlkit_amd.kernels import hadamard

    rng = np.random.default_rng(width)
    rows = 5 if width >= 4096 else 37
    value = rng.standard_normal((rows, width)).astype(F32)
    out = host(hadamard.transform(dev(value), normalize=normalize))
    np.testing.assert_array_equal(out, transforms.fwht(value, normalize))
    if width <= 2048:
        exact = value.astype(np.float64) @ transforms.sylvester(width)
        if normalize:
            exact = exact / np.sqrt(width)
        np.testing.assert_allclose(out, exact, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("width", [256, 512, 1024, 2048, 4096])
def test_register_transform_of_many_rows_is_bit_exact(width):
    """4096 fp32 rows and more take `fwht_rows_kernel` (a row in the registers of one wavefront, no
    LDS): the stagewise oracle on sampled rows, and the workgroup kernel (fewer rows per call) on
    all of them, bit for bit; with signs in front and behind whose period spans three rows."""
    from mlkit_amd.kernels import hadamard

    rows = 4098   # not a multiple of the four rows a workgroup takes
    generator = torch.Generator(device="cuda").manual_seed(width)
    value = torch.randn((rows, width), device="cuda", generator=generator)
    out = hadamard.transform(value)
    picked = [0, 1, 2, 3, 1000, 4095, 4096, 4097]
    np.testing.assert_array_equal(host(out[picked]), transforms.fwht(host(value[picked])))
    pieces = torch.cat([hadamard.transform(value[:2049].contiguous()), hadamard.transform(value[2049:].contiguous())])
    assert torch.equal(out, pieces)
    assert torch.equal(hadamard.transform(value, normalize=False)[:7], hadamard.transform(value[:7].contiguous(), normalize=False))
    signs = dev(transforms.deterministic_signs(3 * width, seed=2))
    blocks = value[: 4098 - 4098 % 3].view(-1, 3, width)
    signed = hadamard.transform(blocks, signs_before=signs, signs_after=signs)
    expected = torch.cat([hadamard.transform(blocks[:600].contiguous(), signs_before=signs, signs_after=signs),
                          hadamard.transform(blocks[600:].contiguous(), signs_before=signs, signs_after=signs)])
    assert torch.equal(signed, expected)
    in_place = value.clone()
    hadamard.transform(in_place, out=in_place)
    assert torch.equal(in_place, out)


def test_leading_dimensions_and_involution():
    from mlkit_amd.kernels import hadamard

    rng = np.random.default_rng(1)
    value = rng.standard_normal((3, 7, 256)).astype(F32)
    once = hadamard.transform(dev(value))
    np.testing.assert_array_equal(host(once), transforms.fwht(value))
    np.testing.assert_allclose(host(hadamard.transform(once)), value, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(np.linalg.norm(host(once)), np.linalg.norm(value), rtol=1e-5)


def test_rejects_other_widths():
    from mlkit_amd.kernels import hadamard

    with pytest.raises(ValueError, match="power-of-two"):
        hadamard.transform(torch.zeros((4, 12), device="cuda"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_half_precision_rows_compute_in_fp32(dtype):
    from mlkit_amd.kernels import hadamard

    generator = torch.Generator().manual_seed(2)
    value = torch.randn((8, 4096), generator=generator).to(dtype)
    out = hadamard.transform(value.cuda())
    assert out.dtype == dtype
    expected = torch.from_numpy(transforms.fwht(value.float().numpy())).to(dtype)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), expected)


def test_fused_signs_match_separate_multiplication():
    from mlkit_amd.kernels import hadamard

    rng = np.random.default_rng(3)
    value = rng.standard_normal((9, 1024)).astype(F32)
    signs = transforms.deterministic_signs(1024, seed=77)
    forward = hadamard.transform(dev(value), signs_before=dev(signs))
    np.testing.assert_array_equal(host(forward), transforms.fwht((value * signs).astype(F32)))
    inverse = hadamard.transform(forward, signs_after=dev(signs))
    np.testing.assert_allclose(host(inverse), value, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("width", [12, 20, 28, 96, 896, 4864, 7, 14336])
def test_blocked_transform_matches_oracle(width):
    from mlkit_amd.kernels import hadamard

    order, power, basis = transforms.transform_factor(width)
    rng = np.random.default_rng(width)
    rows = 6
    value = rng.standard_normal((rows, width)).astype(F32)
    signs = transforms.deterministic_signs(width, seed=5)
    blocks = hadamard.transform(dev(value).view(rows, order, power), signs_before=dev(signs))
    np.testing.assert_array_equal(host(blocks).reshape(rows, width),
                                  transforms.fwht((value * signs).astype(F32).reshape(rows, order, power)).reshape(rows, width))
    mixed = hadamard.mix_blocks(blocks, dev(basis), transpose=False).view(rows, width)
    expected = transforms.randomized(value, signs)
    np.testing.assert_allclose(host(mixed), expected, rtol=1e-5, atol=1e-5)
    # inverse: H blocks, transposed basis, signs afterwards
    back = hadamard.transform(mixed.view(rows, order, power))
    back = hadamard.mix_blocks(back, dev(basis), transpose=True, signs_after=dev(signs)).view(rows, width)
    np.testing.assert_allclose(host(back), value, rtol=1e-5, atol=2e-5)
    np.testing.assert_allclose(host(back), transforms.randomized(expected, signs, inverse=True), rtol=1e-5, atol=2e-5)


@pytest.mark.parametrize("width", [896, 4864, 11008, 14336])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_one_launch_blocked_transform_equals_the_two_calls(width, dtype):
    """`mk_rotate_blocks` against `mk_fwht` + `mk_basis_mix` (+ the cast), bit for bit, forward
    with the signs in front and inverse with the signs behind; 5 rows and 1 row."""
    from mlkit_amd.kernels import hadamard

    order, power, basis = transforms.transform_factor(width)
    assert hadamard.fits_one_launch(order, power)
    generator = torch.Generator(device="cuda").manual_seed(width)
    signs = dev(transforms.deterministic_signs(width, seed=9))
    for rows in (5, 1):
        value = torch.randn((rows, order, power), device="cuda", generator=generator).to(dtype)
        for inverse in (False, True):
            before, after = (None, signs) if inverse else (signs, None)
            staged = torch.empty(value.shape, device="cuda", dtype=torch.float32)
            hadamard.transform(value, signs_before=before, out=staged)
            expected = hadamard.mix_blocks(staged, dev(basis), transpose=inverse, signs_after=after).to(dtype)
            result = hadamard.rotate_blocks(value, dev(basis), transpose=inverse, signs_before=before, signs_after=after)
            assert result.dtype == dtype
            assert torch.equal(result, expected)


@pytest.mark.parametrize("width", [14336, 7168, 5120, 6144])
def test_one_pass_rotation_of_many_rows_equals_the_two_calls(width):
    """More than 256 outer rows of fp32 take `rotate_matrix_kernel` (transform between registers
    and lanes, one LDS exchange, basis product on the matrix cores): bit for bit what `mk_fwht` +
    `mk_basis_mix` give, forward with the signs in front and inverse with the signs behind; and
    `mk.rht` on a weight-sized tensor goes that way."""
    from mlkit_amd.kernels import hadamard

    order, power, basis = transforms.transform_factor(width)
    rows = 301
    generator = torch.Generator(device="cuda").manual_seed(width)
    value = torch.randn((rows, order, power), device="cuda", generator=generator)
    assert hadamard.streams_in_one_pass(value, order, power)
    signs = dev(transforms.deterministic_signs(width, seed=9))
    for inverse in (False, True):
        before, after = (None, signs) if inverse else (signs, None)
        staged = hadamard.transform(value, signs_before=before)
        expected = hadamard.mix_blocks(staged, dev(basis), transpose=inverse, signs_after=after)
        result = hadamard.rotate_blocks(value, dev(basis), transpose=inverse, signs_before=before, signs_after=after)
        assert torch.equal(result, expected)
        assert torch.equal(hadamard.rotate_blocks(value, dev(basis), transpose=inverse), 
                           hadamard.mix_blocks(hadamard.transform(value), dev(basis), transpose=inverse))
    import mlkit_amd as mk

    flat = value.view(rows, width)
    rotated = mk.rht(flat, seed=3)
    torch.testing.assert_close(rotated.norm(dim=1), flat.norm(dim=1), rtol=1e-5, atol=0)
    torch.testing.assert_close(mk.rht(rotated, seed=3, inverse=True), flat, rtol=1e-5, atol=2e-5)
    np.testing.assert_allclose(host(mk.structured_transform(flat[:4].contiguous())),
                               host(mk.structured_transform(flat))[:4], rtol=1e-5, atol=1e-5)  # few rows: the LDS kernel


def test_one_launch_blocked_transform_declines_what_does_not_fit():
    from mlkit_amd.kernels import hadamard

    assert not hadamard.fits_one_launch(7, 16)       # blocks narrower than an MFMA tile
    assert not hadamard.fits_one_launch(97, 64)      # basis beyond three MFMA row tiles
    assert not hadamard.fits_one_launch(3, 32768)    # more than 160 KB of LDS
    value = torch.zeros((2, 7, 16), device="cuda")
    with pytest.raises(Exception, match="do not fit one workgroup"):
        hadamard.rotate_blocks(value, torch.eye(7, device="cuda"), transpose=False)


def test_weight_sized_rotation_keeps_norms():
    """4096 x 14336 fp32 along K as 7 x 2048 blocks (the literal blocked FWHT) and along
    4096: row norms are preserved and the transform is its own inverse."""
    from mlkit_amd.kernels import hadamard

    generator = torch.Generator(device="cuda").manual_seed(4)
    weight = torch.randn((4096, 14336), device="cuda", generator=generator) * 0.02
    blocks = hadamard.transform(weight.view(4096, 7, 2048))
    torch.testing.assert_close(blocks.view(4096, -1).norm(dim=1), weight.norm(dim=1), rtol=1e-5, atol=0)
    torch.testing.assert_close(hadamard.transform(blocks).view_as(weight), weight, rtol=1e-5, atol=1e-6)
    sample = weight[:3].cpu().numpy().reshape(3, 7, 2048)
    np.testing.assert_array_equal(host(blocks[:3]), transforms.fwht(sample))


@pytest.mark.parametrize("width", [32, 64, 512, 896, 4096, 4864, 11008, 14336, 32768])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_row_rotation_kernel_matches_oracle(width, dtype):
    """mk_rotate_rows (mix, then one Walsh-Hadamard transform per output block; the online
    rotation of activations) against the oracle's transform-then-mix: the same linear map in
    another summation order, so fp32 results agree to rounding (the reference's own bound for
    the basis product, rtol 1e-5 of the row norm scale), and rows are independent."""
    from mlkit_amd.quantization.transforms import OnlineRotation, random_signs

    rotation = OnlineRotation(seed=width + 1)
    signs = host(random_signs(width, width + 1, "cuda"))
    for rows in (1, 8, 33):
        generator = torch.Generator().manual_seed(width + rows)
        value = torch.randn((rows, width), generator=generator).to(dtype)
        rotated = rotation(value.cuda())
        assert rotated.dtype == dtype and rotated.shape == value.shape
        expected = transforms.randomized(value.float().numpy(), signs)
        if dtype == torch.float32:
            np.testing.assert_allclose(host(rotated), expected, rtol=1e-5, atol=2e-5)
            np.testing.assert_allclose(np.linalg.norm(host(rotated), axis=1), np.linalg.norm(value.numpy(), axis=1), rtol=1e-5)
        else:
            rounded = torch.from_numpy(expected).to(dtype).float().numpy()
            step = 2.0 ** (-10 if dtype == torch.float16 else -7)
            assert np.abs(host(rotated.float()) - rounded).max() <= step * np.abs(expected).max()
            assert (host(rotated.float()) == rounded).mean() > 0.99          # one rounding: only near-ties move
    first = rotation(value[:1].cuda())
    assert torch.equal(first, rotated[:1])


def test_known_answers_of_the_bases_on_the_device():
    """The device path applies the known Paley sign patterns and scipy's DCT-II to the outer axis
    (tests/golden/transform_known_answers.json, worked out with Python integers): a unit vector e_f comes out
    as column f of the basis, and with a power-of-two factor as that column times the Sylvester block."""
    import json
    import pathlib

    import scipy.fft

    from mlkit_amd.quantization import codecs, transforms as device_transforms

    known = json.loads((pathlib.Path(__file__).resolve().parent / "golden" / "transform_known_answers.json").read_text())
    for order in (12, 20, 28, 44):
        pattern = np.array(known["paley"][str(order)], dtype=np.float64) / np.sqrt(order)
        out = host(device_transforms.structured_transform(torch.eye(order, device="cuda")))
        np.testing.assert_allclose(out, pattern.T, atol=1e-6)
        back = host(device_transforms.structured_transform(torch.eye(order, device="cuda"), inverse=True))
        np.testing.assert_allclose(back, pattern, atol=1e-6)
    pattern = np.array(known["paley"]["28"], dtype=np.float64) / np.sqrt(28)
    for power in (2, 32, 512):                                        # 56, 896, 14336 = 28 x power
        width = 28 * power
        rows = torch.zeros(3, width, device="cuda")
        picks = [(0, 0), (1, power + 1), (2, 14 * power + power - 1)]  # e_(f, p) at rows 0, 1, 2
        for row, index in picks:
            rows[row, index] = 1.0
        out = host(device_transforms.structured_transform(rows)).reshape(3, 28, power)
        sylvester = transforms.sylvester(power) / np.sqrt(power)
        for row, index in picks:
            f, p = divmod(index, power)
            np.testing.assert_allclose(out[row], np.outer(pattern[:, f], sylvester[:, p]), atol=1e-6)
    for width, order in ((7, 7), (43, 43), (86, 43), (11008, 43)):
        power = width // order
        dct = scipy.fft.dct(np.eye(order), type=2, norm="ortho", axis=0)
        rows = torch.zeros(order, width, device="cuda")
        rows[torch.arange(order), torch.arange(order) * power] = 1.0   # e_(f, 0)
        out = host(device_transforms.structured_transform(rows)).reshape(order, order, power)
        np.testing.assert_allclose(out[:, :, 0], dct.T / np.sqrt(power), atol=1e-6)
    for case in known["signs"]:
        assert codecs.deterministic_signs(16, case["seed"], "cuda").tolist() == case["first"]
