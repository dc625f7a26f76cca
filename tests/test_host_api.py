"""Host-side logic of the package on the CPU: the C ABI's symbol table, the API surface
(names, arguments, error messages of the reference), and the tensor-operation paths against
the oracle.  No kernel is launched here."""

import ctypes
import pathlib
import re

import numpy as np
import pytest
import torch
from torch import nn

import mlkit_amd as mk
from mlkit_amd import native
from mlkit_amd.inference.packed_linear import packed_compatible
from mlkit_amd.kernels import packed_linear as packed_kernels
from mlkit_amd.quantization import codecs, transforms as host_transforms
from mlkit_amd.quantization.core import Ctx
from oracle import bitstream as oracle_bits, feedback as oracle_feedback, scaling, transforms as oracle_transforms

import helpers

ROOT = pathlib.Path(__file__).resolve().parent.parent
F32 = np.float32


def test_library_exports_every_declared_entry_point():
    header = (ROOT / "include" / "mlkit_amd.h").read_text()
    declared = set(re.findall(r"^(?:const char \*|int )\s*(mk_\w+)\(", header, flags=re.M))
    assert declared == set(native.SIGNATURES), declared ^ set(native.SIGNATURES)
    assert len(declared) >= 15
    if not native.available():
        pytest.skip("libmlkit_amd.so has not been built in this tree")
    library = ctypes.CDLL(str(native.LIBRARY_PATH))
    for name in declared:
        assert hasattr(library, name), f"{name} is declared but not exported"
    library.mk_version.restype = ctypes.c_char_p
    assert re.fullmatch(rb"\d+\.\d+\.\d+", library.mk_version())


def test_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    monkeypatch.setattr(native, "_library", None)
    monkeypatch.setattr(native, "LIBRARY_PATH", tmp_path / "absent.so")
    with pytest.raises(native.NativeLibraryMissing, match="no fallback"):
        native.library()


def test_nothing_in_the_package_imports_the_oracle():
    for source in (ROOT / "mlkit_amd").rglob("*.py"):
        text = source.read_text()
        assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), source


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8, 11, 16])
def test_pack_and_unpack_follow_the_bit_stream(bits, rng):
    codes = rng.integers(0, 1 << bits, (13, 37))
    packed = mk.pack(torch.from_numpy(codes), bits)
    assert packed.dtype == torch.uint8 and packed.numel() == -(-codes.size * bits // 8)
    np.testing.assert_array_equal(packed.numpy(), oracle_bits.pack(codes, bits))
    restored = mk.unpack(packed, bits, (13, 37))
    assert restored.dtype == (torch.uint8 if bits <= 8 else torch.int32)
    np.testing.assert_array_equal(restored.numpy(), codes)


def test_pack_validation_messages():
    with pytest.raises(ValueError, match="capacity"):
        mk.pack(torch.tensor([0, 16]), 4)
    with pytest.raises(TypeError):
        mk.pack(torch.tensor([0.5]), 4)
    with pytest.raises(ValueError, match="byte count"):
        mk.unpack(torch.zeros(3, dtype=torch.uint8), 4, (7,))
    assert mk.unpack(torch.zeros(0, dtype=torch.uint8), 3, (0, 5)).shape == (0, 5)


def test_grids():
    assert mk.grid.int(4).values.tolist() == list(range(-8, 8)) and mk.grid.int(4).integer
    with pytest.raises(ValueError):
        mk.grid.int(1)
    seven = mk.grid.values([1, -1, 0.5, -0.5, 0.25, -0.25, 0], bits=3)
    assert seven.bits == 3 and seven.values.tolist() == [-1, -0.5, -0.25, 0, 0.25, 0.5, 1]
    with pytest.raises(ValueError, match="capacity"):
        mk.grid.values(torch.arange(9.0), bits=3)
    e2m1 = mk.grid.fp("e2m1")
    assert e2m1.bits == 4 and e2m1.values.numel() == 15 and e2m1.values.max() == 6
    e4m3 = mk.grid.fp("e4m3")
    assert e4m3.bits == 8 and float(e4m3.values.max()) == 240.0 and e4m3.values.numel() == 2 * 119 + 1
    np.testing.assert_array_equal(mk.NF4_VALUES.numpy(), scaling.NF4_VALUES)
    assert repr(mk.int(4, group=128)) == "scaled(Grid(int4, bits=4, dim=1), group=128, scale='absmax')"
    assert repr(mk.int(4, asym=True, scale_fmt="bf16")).endswith("scale_fmt='bf16', asym=True)")


@pytest.mark.parametrize("fmt", ["fp32", "fp16", "bf16", "fp8", "e8m0"])
def test_store_scale_matches_oracle(fmt, rng):
    value = np.exp(rng.uniform(-12, 8, 5000)).astype(F32)
    stored, bits = mk.store_scale(torch.from_numpy(value), fmt)
    expected, expected_bits = scaling.store_scale(value, fmt)
    np.testing.assert_array_equal(stored.numpy(), expected)
    assert bits == expected_bits


@pytest.mark.parametrize("asym", [False, True])
@pytest.mark.parametrize("shape,group", [((16, 256), 64), ((8, 250), 50), ((5, 70), None)])
def test_scaled_tensor_path_matches_oracle(shape, group, asym):
    weight = helpers.normal_weight(*shape, seed=21, student_t=True)
    result = mk.int(4, group=group, asym=asym)(torch.from_numpy(weight))
    expected = scaling.quantize(weight, scaling.int_values(4), group=group, integer=True, asym=asym)
    np.testing.assert_array_equal(result.codes.numpy(), expected["codes"])
    np.testing.assert_array_equal(result.params["scales"].numpy(), expected["scales"])
    if asym:
        np.testing.assert_array_equal(result.params["zero"].numpy(), expected["zero"])
    assert result.bits == 4 * weight.size + expected["side_bits"]
    assert result.codec == "scaled" and result.metadata["code_bits"] == 4 and result.metadata["scale_fmt"] == "fp16"
    dense = scaling.decode_grouped(expected["codes"], expected["scales"], expected["values"], expected["group"], expected["zero"])
    np.testing.assert_array_equal(result.w.numpy(), dense)
    assert mk.int(4, group=group, asym=asym).logical_bits(shape) == result.bits


def test_codebook_mse_tensor_path_matches_oracle_at_the_reference_tolerance():
    values = np.array([-1, -0.5, -0.25, 0, 0.25, 0.5, 1], dtype=F32)
    weight = helpers.normal_weight(32, 512, seed=22, student_t=True)
    result = mk.scaled(mk.grid.values(values, bits=3), group=64, scale="mse")(torch.from_numpy(weight))
    expected = scaling.quantize(weight, values, group=64, integer=False, scale="mse")
    assert (result.params["scales"].numpy() == expected["scales"]).mean() >= 0.97
    same = (result.params["scales"].numpy() == expected["scales"]).repeat(64, axis=1)
    np.testing.assert_array_equal(result.codes.numpy()[same], expected["codes"][same])


def test_scaled_rejects_bad_input():
    with pytest.raises(ValueError, match="finite"):
        mk.int(4)(torch.tensor([[1.0, float("inf")] * 8]))
    with pytest.raises(ValueError, match="finite"):
        mk.int(4)(torch.ones(4, 4, dtype=torch.int32))
    with pytest.raises(ValueError):
        mk.scaled(mk.grid.int(4), group=0)
    with pytest.raises(ValueError, match="asymmetric"):
        mk.scaled(mk.grid.int(4), asym=True, scale_fmt="e8m0")
    rounder = mk.int(4, group=8).fit(torch.randn(4, 32), Ctx())
    with pytest.raises(ValueError, match="contiguous slice"):
        rounder(torch.randn(4, 8), slice(0, 16))


def test_codec_registry_and_row_concatenation():
    with pytest.raises(ValueError, match="already registered"):
        mk.codec("scaled")(lambda codes: codes)
    with pytest.raises(ValueError, match="registered codec"):
        codecs.decoder("nonexistent")
    weight = torch.from_numpy(helpers.normal_weight(12, 128, seed=23))
    whole = mk.int(4, group=32)(weight)
    parts = [mk.int(4, group=32)(weight[:5]), mk.int(4, group=32)(weight[5:])]
    joined = mk.concatenate_rows(parts)
    assert torch.equal(joined.codes, whole.codes) and torch.equal(joined.params["scales"], whole.params["scales"])
    assert joined.bits == whole.bits and torch.equal(joined.w, whole.w)

    @mk.codec("test_unjoinable")
    def decode_plain(codes, *, table):
        return table[codes.int()]

    orphan = mk.Q(codes=torch.zeros(2, 2, dtype=torch.uint8), params={"table": torch.ones(1)}, decode=decode_plain,
                  codec="test_unjoinable")
    with pytest.raises(ValueError, match="row parameters"):
        mk.concatenate_rows([orphan, orphan])


def test_feedback_decoder_index_map_and_permutation(rng):
    codes = rng.integers(0, 16, (4, 20), dtype=np.uint8)
    scales = (rng.random((4, 6)) + 0.5).astype(F32)
    values = scaling.int_values(4)
    out = codecs.decode_feedback(torch.from_numpy(codes), scales=torch.from_numpy(scales), values=torch.from_numpy(values),
                                 group=4, refit=10)
    np.testing.assert_array_equal(out.numpy(), scaling.decode_feedback(codes, scales, values, 4, 10))
    permutation = torch.from_numpy(rng.permutation(20))
    permuted = codecs.decode_feedback(torch.from_numpy(codes), scales=torch.from_numpy(scales),
                                      values=torch.from_numpy(values), group=4, refit=10, permutation=permutation)
    assert torch.equal(permuted[:, permutation], out)


def test_deterministic_signs_and_layer_seed_match_oracle():
    np.testing.assert_array_equal(mk.deterministic_signs(300, 99, "cpu").numpy(), oracle_transforms.deterministic_signs(300, 99))
    assert mk.layer_seed("model.layers.3.mlp.down_proj", 5) == oracle_transforms.layer_seed("model.layers.3.mlp.down_proj", 5)


@pytest.mark.parametrize("width", [12, 28, 96, 896, 7, 64])
def test_host_transforms_match_oracle(width, rng):
    value = rng.standard_normal((4, width)).astype(F32)
    order, power, basis = mk.transform_factor(width)
    expected = oracle_transforms.transform_factor(width)
    assert (order, power) == expected[:2]
    if basis is not None:
        np.testing.assert_allclose(basis.numpy(), expected[2], atol=1e-7)
    out = mk.structured_transform(torch.from_numpy(value))
    np.testing.assert_allclose(out.numpy(), oracle_transforms.structured(value), rtol=1e-5, atol=1e-6)
    back = mk.rht(mk.rht(torch.from_numpy(value), seed=3), seed=3, inverse=True)
    np.testing.assert_allclose(back.numpy(), value, rtol=1e-5, atol=1e-5)
    with pytest.raises(ValueError, match="power-of-two"):
        mk.hadamard(torch.zeros(2, 12))


def test_gptq_tensor_path_matches_oracle_sweep(rng):
    weight = helpers.normal_weight(24, 256, seed=24)
    inputs = rng.standard_normal((768, 256)).astype(F32)
    inputs[:, 9] = 0  # a dead channel
    hessian = (inputs.T @ inputs / 768).astype(F32)
    result = mk.gptq(mk.int(4, group=64), refit=64, block_size=64)(torch.from_numpy(weight), Ctx(H=torch.from_numpy(hessian)))
    coeff, status = oracle_feedback.coefficients(hessian, 0.01)
    assert status == 0
    np.testing.assert_allclose(mk.feedback_coefficients(torch.from_numpy(hessian).clone(), 1)[0].numpy(), coeff,
                               rtol=2e-4, atol=1e-6)
    expected = oracle_feedback.sweep(weight, coeff, scaling.int_values(4), group=64, integer=True, refit=64, block=64,
                                     dead=np.diag(hessian) == 0, update_mode=1)
    assert result.codec == "feedback" and result.params["refit"] == 64 and result.params["permutation"] is None
    assert (result.codes.numpy() == expected["codes"]).mean() > 0.995   # BLAS order differs from the oracle's chain
    assert result.bits == 4 * weight.size + 16 * 24 * 4
    assert float(result.w[:, 9].abs().max()) == 0
    loss = float(mk.proxy_loss(torch.from_numpy(weight), result.w, torch.from_numpy(hessian)))
    rtn = mk.int(4, group=64)(torch.from_numpy(weight)).w
    assert loss < float(mk.proxy_loss(torch.from_numpy(weight), rtn, torch.from_numpy(hessian)))
    assert packed_compatible(result)
    ordered = mk.gptq(mk.int(4, group=64), refit=64, act_order=True)(torch.from_numpy(weight), Ctx(H=torch.from_numpy(hessian)))
    assert not packed_compatible(ordered) and ordered.params["permutation"] is not None


def test_error_feedback_validation():
    with pytest.raises(ValueError, match="multiple of step"):
        mk.ldlq(mk.int(4), step=8, block_size=12)
    with pytest.raises(ValueError, match="Hessian dimensions"):
        mk.gptq(mk.int(4))(torch.randn(4, 16), Ctx(H=torch.eye(8)))
    with pytest.raises(ValueError, match="positive definite"):
        mk.gptq(mk.int(4), damp=0.0)(torch.randn(4, 16), Ctx(H=-torch.eye(16)))
    with pytest.raises(RuntimeError, match="calibration statistic"):
        mk.gptq(mk.int(4))(torch.randn(4, 16))


def test_layout_predicate_and_packed_compatibility():
    assert packed_kernels.layout_for(4, 4096, 128).tile_codes == 128
    assert packed_kernels.layout_for(3, 250, 50) is None
    assert packed_kernels.layout_for(9, 256, 64) is None
    assert packed_kernels.sample_tile_for(5) == 8
    weight = torch.from_numpy(helpers.normal_weight(8, 64, seed=25))
    assert packed_compatible(mk.int(4, group=32)(weight))
    assert not packed_compatible(mk.int(12, group=32)(weight))
    assert not packed_compatible(mk.Q(weight))


def test_capability_report_strings_on_the_host():
    report = mk.capabilities(mk.int(4, group=128), device="cpu")
    assert report.bits_per_weight == 4.125 and report.codec == "scaled"
    assert report.checkpoint == "codes with a registered codec"
    assert report.error_feedback == "fused scalar kernel at step=1"
    assert report.packed_inference == "fused kernel" and report.online_activations == "fused kernel"
    assert "bits per weight     4.1250" in str(report)

    class Ternary(mk.Quantizer):
        def fit(self, weight, context):
            return mk.scaled(mk.grid.values(torch.tensor([-1.0, 0.0, 1.0]), bits=2), group=64).fit(weight, context)

    ternary = mk.capabilities(Ternary(), device="cpu")
    assert ternary.quantizer == "Ternary()" and ternary.bits_per_weight == 2.25
    assert ternary.online_activations.startswith("reference rounding")

    @mk.quantizer
    def sign(weight, context):
        return weight.sign() * weight.abs().mean()

    plain = mk.capabilities(sign, device="cpu")
    assert plain.bits_per_weight is None and plain.codec is None and plain.checkpoint == "dense reconstruction"
    assert plain.error_feedback.startswith("reference rounding") and plain.packed_inference == "no; dense weights"
    assert "unknown" in str(plain)
    assert mk.capabilities(mk.int(12), device="cpu").error_feedback == "reference rounding with the fitted rounder"
    feedback = mk.capabilities(mk.gptq(mk.int(4)), device="cpu")
    assert feedback.error_feedback == "not an inner format; it does not implement Quantizer.fit"
    assert feedback.packed_inference == "fused kernel"
    split = mk.capabilities(mk.int(3, group=50), shape=(16, 250), device="cpu")
    assert split.packed_inference.startswith("packed storage with dense execution")

    @mk.quantizer
    def truncated(weight, context):
        return weight[:, :-1]

    with pytest.raises(ValueError, match="invalid reconstruction"):
        mk.capabilities(truncated, device="cpu")


def test_checkpoint_layer_entries_round_trip():
    from mlkit_amd.checkpoints import layout

    weight = torch.from_numpy(helpers.normal_weight(16, 96, seed=26))
    first = mk.int(4, group=32, asym=True)(weight)
    second = mk.nf4(group=32)(weight * 2)
    dense = mk.Q(weight.clone(), bits=16 * weight.numel())
    tensors, layers = layout.describe_layers({"a": first, "b": second, "c": dense, "d": mk.int(4, group=32, asym=True)(weight)})
    assert tensors["a.codes"].numel() == 16 * 96 // 2 and tensors["a.params.scales"].dtype == torch.float16
    assert layers["a"]["params"]["group"] == {"value": 32} and layers["c"] == {"codec": None, "bits": dense.bits}
    assert layers["d"]["params"]["values"]["tensor"] == "a.params.values"      # identical tensors stored once
    assert "d.params.scales" not in tensors
    for name, original in (("a", first), ("b", second), ("c", dense)):
        restored = layout.restore_layer(tensors, name, layers[name])
        torch.testing.assert_close(restored.w, original.w, rtol=0, atol=0)
        assert restored.bits == original.bits
    assert (layout.FORMAT_VERSION, layout.MANIFEST_FILE, layout.WEIGHTS_FILE) == (1, "mlkit.json", "weights.safetensors")


def test_function_quantizers_bind_parameters():
    @mk.quantizer
    def clipped(w, ctx, *, limit=1.0):
        return w.clamp(-limit, limit)

    tight = clipped(limit=0.1)
    assert repr(tight) == "clipped(limit=0.1)"
    assert float(tight(torch.ones(2, 2) * 5, Ctx()).w.max()) == pytest.approx(0.1)
    with pytest.raises(TypeError):
        clipped(unknown=3)
    assert isinstance(nn.Linear(2, 2), nn.Module)


@pytest.mark.parametrize("shape", [(32, 64), (28, 96), (12, 20)])
def test_incoherent_identity_and_basis_codec(shape):
    torch.manual_seed(3)
    weights = torch.randn(*shape)
    identity = mk.incoherent(lambda w, ctx: mk.Q(w, bits=32 * w.numel()))(weights)
    torch.testing.assert_close(identity.w, weights, rtol=1e-5, atol=1e-5)
    coded = mk.incoherent(mk.int(8, group=None))(weights, Ctx("layer.0"))
    assert coded.codec == "basis" and coded.params["inner_codec"] == "scaled"
    assert coded.params["right_seed"] == (coded.params["left_seed"] + 1) % 2**32
    assert coded.metadata["trainable"] == ["inner_scales"] and coded.metadata["parameter_formats"]["inner_scales"] == "fp16"
    assert float((coded.w - weights).abs().max()) < 0.08 * float(weights.abs().max())
    # one-sided and calibrated variants
    right_only = mk.incoherent(mk.int(8, group=None), left=None)(weights)
    assert right_only.params["left_seed"] is None
    inputs = torch.randn(4 * shape[1], shape[1])
    with_feedback = mk.incoherent(mk.gptq(mk.int(4, group=None), refit=None))(weights, Ctx("l", X=inputs))
    assert with_feedback.codec == "basis" and with_feedback.params["inner_codec"] == "feedback"
    assert torch.isfinite(with_feedback.w).all()
    with pytest.raises(ValueError, match="rht or None"):
        mk.incoherent(mk.int(4), left="dct")


# ---- vector grids on host tensors -------------------------------------------------------------------


def test_vector_grid_validation_and_nearest_on_the_host(rng):
    from oracle import lattice as oracle_lattice

    with pytest.raises(ValueError, match="nonempty finite matrix"):
        mk.grid.vector(torch.zeros(0, 4))
    with pytest.raises(ValueError, match="exceeds the declared bit capacity"):
        mk.grid.vector(torch.randn(20, 4), bits=4)
    grid = mk.grid.vector(torch.randn(20, 4))
    assert (grid.bits, grid.dim, grid.name) == (5, 4, "vector")
    lattice = mk.grid.e8p()
    assert (lattice.bits, lattice.dim, lattice.name) == (16, 8, "e8p") and lattice.values.shape == (65536, 8)
    codebook = rng.standard_normal((300, 8)).astype(np.float32)
    codebook[200] = codebook[7]
    samples = rng.standard_normal((500, 8)).astype(np.float32)
    samples[0] = codebook[7]
    found = mk.nearest(torch.from_numpy(samples), torch.from_numpy(codebook), return_indices=True, codebook_chunk=128)
    expected = oracle_lattice.nearest_codes(samples, codebook)
    assert (found.numpy() == expected).mean() > 0.99 and found[0] == 7
    rounded = lattice(torch.from_numpy(samples))
    codes = oracle_lattice.nearest_e8p_codes(samples)
    np.testing.assert_array_equal(rounded.numpy(), oracle_lattice.e8p_points()[codes])
    with pytest.raises(ValueError, match="eight-dimensional"):
        lattice(torch.zeros(3, 4))
    with pytest.raises(ValueError, match="asymmetric quantization requires an explicit scalar grid"):
        mk.scaled(lattice, asym=True)
    with pytest.raises(ValueError, match="divisible by the vector grid dimension"):
        mk.scaled(lattice, group=12)(torch.randn(4, 48))


def test_vector_grid_and_feedback_on_the_host():
    # /root/reference/tests/quantization/test_algorithms.py:60-66, and the decoders
    weights = torch.randn(16, 64)
    codebook = torch.randn(32, 8)
    quantization = mk.scaled(mk.grid.vector(codebook), group=None)
    context = Ctx("layer", H=torch.eye(64))
    result = mk.ldlq(quantization, step=8)(weights, context)
    assert result.w.shape == weights.shape and result.codec == "vector_feedback"
    assert result.bits == 5 * weights.numel() / 8 + 16 * weights.shape[0]
    assert context.additional_bits == 32 * 8 * 32          # the codebook, counted once
    assert quantization.logical_bits((16, 64)) == result.bits
    torch.testing.assert_close(codecs.decoder("vector_feedback")(result.codes, **result.params), result.w, rtol=0, atol=0)
    # with an identity Hessian no error is fed back: the sweep equals direct rounding
    direct = quantization(weights, Ctx("layer"))
    assert direct.codec == "vector_scaled" and direct.codes.dtype == torch.int32
    assert torch.equal(direct.codes, result.codes)
    lattice = mk.scaled(mk.grid.e8p(), group=32)(weights)
    assert lattice.params["values"] is None and lattice.params["dim"] == 8
    from oracle import lattice as oracle_lattice

    expected = oracle_lattice.decode_vector_scaled(lattice.codes.numpy(), lattice.params["scales"].numpy(),
                                                   oracle_lattice.e8p_points(), 32, 8)
    np.testing.assert_array_equal(lattice.w.numpy(), expected)
    joined = mk.concatenate_rows([mk.scaled(mk.grid.e8p(), group=32)(weights[:8]), mk.scaled(mk.grid.e8p(), group=32)(weights[8:])])
    torch.testing.assert_close(joined.w, lattice.w, rtol=0, atol=0)
    with pytest.raises(ValueError, match="step equal to its dimension"):
        mk.ldlq(quantization, step=8, backend="hip")(weights, Ctx("layer", H=torch.eye(64)))


def test_rotation_of_separate_blocks_on_the_host():
    """``rht(value, seed, block=b)`` transforms blocks of b values one by one: per block the
    oracle's stagewise transform of value * signs, its own inverse, and an error for blocks
    that do not tile the width as powers of two.  ``mk.rotate(seed, block=b)`` records the
    block length with the layer and leaves layers the blocks do not tile to the whole-row
    transform."""
    from oracle import transforms as oracle_transforms
    from mlkit_amd.conversion import RotateInputs

    torch.manual_seed(3)
    value = torch.randn(5, 768)
    rotated = mk.rht(value, seed=9, block=256)
    signs = host_transforms.random_signs(768, 9, "cpu").numpy()
    expected = oracle_transforms.fwht((value.numpy() * signs).reshape(5, 3, 256)).reshape(5, 768)
    np.testing.assert_allclose(rotated.numpy(), expected, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(mk.rht(rotated, seed=9, inverse=True, block=256).numpy(), value.numpy(), rtol=1e-5, atol=1e-5)
    with pytest.raises(ValueError, match="do not tile"):
        mk.rht(value, seed=9, block=512)
    with pytest.raises(ValueError, match="do not tile"):
        mk.rht(value, seed=9, block=96)
    module = nn.ModuleDict({"down_proj": nn.Linear(768, 8), "o_proj": nn.Linear(96, 8)})
    inputs = torch.randn(2, 768)
    before = module["down_proj"](inputs)
    mk.rotate(seed=1, block=256)(module)
    descriptors = {entry["name"]: entry for entry in module._mlkit_transforms}
    assert descriptors["down_proj"]["block"] == 256 and "block" not in descriptors["o_proj"]
    hook, = (h for h in module["down_proj"]._forward_pre_hooks.values() if isinstance(h, RotateInputs))
    assert hook.rotation.block == 256
    torch.testing.assert_close(module["down_proj"](inputs), before, rtol=1e-4, atol=1e-5)


def test_copies_of_an_online_rotation_prepare_their_own_plans():
    """Prepared plans close over device addresses; copies and pickles carry the seed and block only."""
    import copy
    import pickle

    from mlkit_amd.quantization.transforms import OnlineRotation

    rotation = OnlineRotation(5, 2048)
    value = torch.randn(2, 4096)
    expected = rotation(value)
    assert rotation._plans
    for other in (copy.deepcopy(rotation), pickle.loads(pickle.dumps(rotation))):
        assert (other.seed, other.block) == (5, 2048) and not other._plans
        assert torch.equal(other(value), expected)
