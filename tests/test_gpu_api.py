"""GPU tests of the public API on HIP tensors: the kernels behind ``mk.scaled``, ``mk.gptq``,
``mk.rht``, ``PackedLinear`` and ``mk.optimize`` against the oracle (bit for bit where the
arithmetic is fixed) and with the reference's own module-level assertions
(tests/inference/test_packed_linear.py, tests/evaluation/test_capability_report.py,
tests/conversion/test_head_quantization.py:76-81, tests/checkpoints/test_checkpoints.py in
/root/reference)."""

import copy

import numpy as np
import pytest
import torch
from torch import nn
import torch.nn.functional as functional

import mlkit_amd as mk
from mlkit_amd.quantization.core import Ctx
from oracle import feedback as oracle_feedback, scaling, transforms as oracle_transforms

import helpers

pytestmark = pytest.mark.gpu

F32 = np.float32
SEVEN = np.array([-1, -0.5, -0.25, 0, 0.25, 0.5, 1], dtype=F32)


def dev(array):
    return torch.from_numpy(np.ascontiguousarray(array)).cuda()


def host(tensor):
    torch.cuda.synchronize()
    return tensor.detach().cpu().numpy()


@pytest.mark.parametrize("name,make,values,integer,kwargs", [
    ("int4-asym-g128", lambda: mk.int(4, group=128, asym=True), scaling.int_values(4), True, dict(group=128, asym=True)),
    ("int2-g64", lambda: mk.int(2, group=64), scaling.int_values(2), True, dict(group=64)),
    ("int3-g64", lambda: mk.int(3, group=64), scaling.int_values(3), True, dict(group=64)),
    ("nf4-g64", lambda: mk.nf4(group=64), scaling.NF4_VALUES, False, dict(group=64)),
    ("cb3-g64-mse", lambda: mk.scaled(mk.grid.values(SEVEN, bits=3), group=64, scale="mse"), SEVEN, False,
     dict(group=64, scale="mse")),
    ("int4-g128-mse", lambda: mk.int(4, group=128, scale="mse"), scaling.int_values(4), True, dict(group=128, scale="mse")),
    ("int4-rowwise-bf16", lambda: mk.int(4, group=None, scale_fmt="bf16"), scaling.int_values(4), True,
     dict(group=None, fmt="bf16")),
])
def test_scaled_formats_match_oracle_bit_for_bit(name, make, values, integer, kwargs):
    weight = helpers.normal_weight(96, 1024, seed=31, student_t=True)
    result = make()(dev(weight))
    expected = scaling.quantize(weight, values, integer=integer, **kwargs)
    np.testing.assert_array_equal(host(result.params["scales"]), expected["scales"])
    np.testing.assert_array_equal(host(result.codes), expected["codes"])
    if expected["zero"] is not None:
        np.testing.assert_array_equal(host(result.params["zero"]), expected["zero"])
    dense = scaling.decode_grouped(expected["codes"], expected["scales"], values, expected["group"], expected["zero"])
    np.testing.assert_array_equal(host(result.w), dense)
    assert result.bits == make().logical_bits(weight.shape)


def test_scaled_rejects_non_finite_weights_on_device():
    weight = torch.randn(8, 256, device="cuda")
    weight[3, 17] = float("nan")
    with pytest.raises(ValueError, match="finite"):
        mk.int(4)(weight)


def test_online_activation_reconstruction_equals_quantize_dequantize():
    x = torch.randn(5, 512, device="cuda").half()
    fmt = mk.int(8, group=128)
    torch.testing.assert_close(fmt.reconstruct_activations(x), fmt(x.float()).w.half(), rtol=0, atol=0)


@pytest.mark.parametrize("values,integer,asym,group,refit,block", [
    (scaling.int_values(4), True, False, 128, 128, 128),
    (scaling.int_values(4), True, True, 64, 128, 64),      # two tiles per region
    (scaling.NF4_VALUES, False, False, 64, 64, 128),
    (scaling.int_values(3), True, False, 32, None, 128),   # one region: no refits
    # one kernel per 128-column region (pending solve + scale fit + sweep), every group width it takes
    (scaling.int_values(4), True, True, 64, 128, 128),
    (scaling.int_values(4), True, False, 16, 128, 128),
    (scaling.int_values(3), True, True, 32, 128, 256),
    (scaling.int_values(8), True, True, 128, 128, 128),
    # tables of up to sixteen values in the same one-kernel-per-region path (NF4, FP4 and a ragged table)
    (scaling.NF4_VALUES, False, False, 64, 128, 128),
    (scaling.NF4_VALUES, False, True, 32, 128, 128),
    (np.array([-6, -4, -3, -2, -1.5, -1, -0.5, 0, 0.5, 1, 1.5, 2, 3, 4, 6], dtype=np.float32), False, False, 32, 128, 256),
    (np.array([-1, -0.5, -0.25, 0, 0.25, 0.5, 1], dtype=np.float32), False, False, 128, 128, 128),
    (scaling.NF4_VALUES, False, False, 64, 96, 96),        # regions that are not whole tiles
    # tables of 17 to 256 values take the one-kernel-per-region path too (a row's sixteen lanes search together)
    (np.sinh(np.linspace(-3, 3, 256)).astype(np.float32), False, False, 64, 128, 128),
    (np.sinh(np.linspace(-3, 3, 256)).astype(np.float32), False, True, 128, 128, 256),
    ((np.linspace(-1, 1, 40) ** 3).astype(np.float32), False, False, 32, 128, 128),
    ((np.linspace(-1, 1, 40) ** 3).astype(np.float32), False, False, 64, 96, 96),   # tiles of 96 columns
])
def test_gptq_on_device_matches_oracle_sweep(values, integer, asym, group, refit, block, rng):
    rows, width = 80, 512
    weight = helpers.normal_weight(rows, width, seed=32)
    inputs = rng.standard_normal((1536, width)).astype(F32)
    inputs[:, ::9] *= 5
    inputs[:, 100] = 0
    hessian = (inputs.T @ inputs / 1536).astype(F32)
    grid = mk.grid.int(int(np.log2(len(values)))) if integer else mk.grid.values(values, bits=max(4, int(np.ceil(np.log2(len(values))))))
    inner = mk.scaled(grid, group=group, asym=asym)
    quantizer = mk.gptq(inner, refit=refit, block_size=block)
    context = Ctx("layer", H=dev(hessian))
    result = quantizer(dev(weight), context)
    # the coefficient matrix is an input of the sweep: hand the oracle the very same one
    coeff = host(mk.feedback_coefficients(dev(hessian).clone(), 1)[0])
    expected = oracle_feedback.sweep(weight, coeff, values, group=group, integer=integer, refit=refit, block=block,
                                     asym=asym, dead=np.diag(hessian) == 0, update_mode=0)
    np.testing.assert_array_equal(host(result.params["scales"]), expected["scales"])
    np.testing.assert_array_equal(host(result.codes), expected["codes"])
    np.testing.assert_array_equal(host(result.w), expected["w"])
    assert result.codec == "feedback"
    loss = float(mk.proxy_loss(dev(weight), result.w, dev(hessian)))
    assert loss < float(mk.proxy_loss(dev(weight), inner(dev(weight)).w, dev(hessian)))
    assert loss == pytest.approx(oracle_feedback.proxy_loss(weight, expected["w"], hessian), rel=1e-3)


def test_config4_gptq_int4_g128_4096x11008_rows_match_oracle():
    """The whole 4096 x 11008 layer of the benchmark configuration on the device (Hessian from
    16384 tokens with 1 % of the channels x30, damp 0.01, block = refit = group = 128, natural
    order).  Rows are independent, so the oracle sweeps 16 rows spread over the matrix with the
    same coefficient matrix; codes, scales and reconstruction must equal it bit for bit, and
    the decoded result must equal the sweep's output."""
    rows, width = 4096, 11008
    checked = np.linspace(0, rows - 1, 16).astype(np.int64)
    generator = torch.Generator(device="cuda").manual_seed(33)
    weight = (torch.randn((rows, width), device="cuda", generator=generator) * 0.02).half().float()
    inputs = torch.randn((16384, width), device="cuda", generator=generator).half()
    hot = torch.randperm(width, device="cuda", generator=generator)[: width // 100]
    inputs[:, hot] *= 30
    hessian = torch.zeros((width, width), device="cuda")
    for band in inputs.split(2048):                       # X^T X / n without a 721 MB fp32 copy of X
        hessian.addmm_(band.float().T, band.float())
    hessian /= inputs.shape[0]
    del inputs
    result = mk.gptq(mk.int(4, group=128))(weight, Ctx("down_proj", H=hessian))
    coeff = host(mk.feedback_coefficients(hessian.clone(), 1)[0])
    picked = torch.from_numpy(checked).cuda()
    expected = oracle_feedback.sweep(host(weight[picked]), coeff, scaling.int_values(4), group=128, integer=True,
                                     refit=128, block=128)
    del coeff
    np.testing.assert_array_equal(host(result.codes[picked]), expected["codes"])
    np.testing.assert_array_equal(host(result.params["scales"][picked]), expected["scales"])
    np.testing.assert_array_equal(host(result.w[picked]), expected["w"])
    assert result.params["scales"].shape == (rows, width // 128) and result.codes.shape == (rows, width)
    rtn = mk.int(4, group=128)(weight).w
    loss = float(mk.proxy_loss(weight, result.w, hessian))
    assert loss < 0.9 * float(mk.proxy_loss(weight, rtn, hessian))
    sampled = oracle_feedback.proxy_loss(host(weight[picked]), expected["w"], host(hessian))
    assert float(mk.proxy_loss(weight[picked], result.w[picked], hessian)) == pytest.approx(sampled, rel=1e-3)


@pytest.mark.parametrize("values,integer,asym,group,refit", [
    (scaling.int_values(4), True, False, 128, 128),
    (scaling.int_values(4), True, True, 64, 128),
    (scaling.NF4_VALUES, False, False, 64, 64),
])
def test_gptq_activation_order_on_device_matches_oracle(values, integer, asym, group, refit, rng):
    """act_order=True: columns are swept by descending Hessian diagonal (dead channels count as
    1).  The oracle sweeps the permuted weights with the device's coefficient matrix of the
    permuted Hessian; codes and scales stay in sweep order, the reconstruction is returned in
    the original column order (algorithms/error_feedback.py:276-283,196-197,228-232 in
    /root/reference)."""
    rows, width = 80, 512
    weight = helpers.normal_weight(rows, width, seed=34)
    inputs = rng.standard_normal((1536, width)).astype(F32)
    inputs *= np.linspace(0.5, 3.0, width, dtype=F32)[rng.permutation(width)]
    inputs[:, 77] = 0
    hessian = (inputs.T @ inputs / 1536).astype(F32)
    grid = mk.grid.int(4) if integer else mk.grid.values(values, bits=4)
    quantizer = mk.gptq(mk.scaled(grid, group=group, asym=asym), refit=refit, act_order=True)
    context = Ctx("layer", H=dev(hessian))
    result = quantizer(dev(weight), context)
    permutation = host(result.params["permutation"])
    diagonal = np.diag(hessian).copy()
    diagonal[diagonal == 0] = 1
    assert sorted(permutation.tolist()) == list(range(width))
    assert (np.diff(diagonal[permutation]) <= 0).all()                       # descending activation energy
    coeff = host(mk.feedback_coefficients(dev(hessian).clone(), 1, permutation=dev(permutation))[0])
    dead = (np.diag(hessian) == 0)
    expected = oracle_feedback.sweep(weight[:, permutation], coeff, values, group=group, integer=integer,
                                     refit=refit, block=128, asym=asym, dead=dead[permutation])
    np.testing.assert_array_equal(host(result.codes), expected["codes"])
    np.testing.assert_array_equal(host(result.params["scales"]), expected["scales"])
    if asym:
        np.testing.assert_array_equal(host(result.params["zero"]), expected["zero"])
    np.testing.assert_array_equal(host(result.w), expected["w"][:, np.argsort(permutation)])
    if not asym:   # an asymmetric grid need not contain zero
        assert float(np.abs(host(result.w)[:, 77]).max()) == 0
    plain = mk.gptq(mk.scaled(grid, group=group, asym=asym), refit=refit)(dev(weight), Ctx("layer", H=dev(hessian)))
    assert result.bits == plain.bits and context.additional_bits == width * 9   # K * ceil(log2 K) bits of order
    from mlkit_amd.inference.packed_linear import packed_compatible
    assert not packed_compatible(result)


@pytest.mark.parametrize("width", [28, 96, 896, 4864, 4096, 14336])
def test_rht_round_trip_and_oracle(width):
    value = torch.randn((6, width), device="cuda")
    rotated = mk.rht(value, seed=5)
    torch.testing.assert_close(mk.rht(rotated, seed=5, inverse=True), value, rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(rotated.norm(dim=1), value.norm(dim=1), rtol=1e-5, atol=0)
    from mlkit_amd.quantization.transforms import random_signs

    signs = host(random_signs(width, 5, "cuda"))
    np.testing.assert_allclose(host(rotated), oracle_transforms.randomized(host(value), signs), rtol=1e-5, atol=2e-5)


def test_rotated_layer_keeps_its_outputs():
    """Offline rotation of the weight columns plus online rotation of the inputs leaves the
    product unchanged (14336-wide down projection, 28 x 512 Paley factorisation)."""
    weight = torch.randn((256, 14336), device="cuda") * 0.02
    x = torch.randn((2, 14336), device="cuda")
    torch.testing.assert_close(mk.rht(x, seed=9) @ mk.rht(weight, seed=9).T, x @ weight.T, rtol=1e-3, atol=2e-3)
    half = mk.rht(x.half(), seed=9)
    assert half.dtype == torch.float16
    torch.testing.assert_close(half.float(), mk.rht(x.half().float(), seed=9), rtol=2e-3, atol=2e-3)


# ---- module level: mirrors of the reference's PackedLinear tests ---------------------------

def packed_and_reference(fmt, *, input_width=256, output_width=37, dtype=torch.float32, calibration=None):
    torch.manual_seed(40)
    module = nn.Sequential(nn.Linear(input_width, output_width, dtype=dtype))
    converted = mk.quantize(module, fmt, calib=None if calibration is None else [calibration], cache_dir=None)
    packed = mk.optimize(converted, backend="packed")
    assert isinstance(packed.module[0], mk.PackedLinear)
    return packed, converted


@pytest.mark.parametrize("name", ["int4", "nf4"])
@pytest.mark.parametrize("batch", [1, 3, 7])
def test_packed_linear_matches_dense(name, batch):
    fmt = {"int4": mk.int(4, group=32), "nf4": mk.nf4(group=32)}[name]
    torch.manual_seed(41)
    module = nn.Sequential(nn.Linear(130, 71, dtype=torch.float16))
    converted = mk.quantize(module, fmt, calib=None)
    packed = mk.optimize(converted, backend="packed")
    inputs = torch.randn(batch, 130, dtype=torch.float16)
    with torch.inference_mode():
        torch.testing.assert_close(packed(inputs), converted(inputs), rtol=0.002, atol=0.002)
    assert isinstance(packed.module[0], mk.PackedLinear)
    assert packed.module[0].packed.numel() == (130 * 71 + 1) // 2
    assert packed.execution_backend == "packed:1"


@pytest.mark.parametrize("rows", [1, 2, 5, 8, 9, 33])
def test_packed_linear_handles_every_row_count(rows):
    packed, converted = packed_and_reference(mk.int(4, group=64))
    inputs = torch.randn(rows, 256)
    with torch.inference_mode():
        torch.testing.assert_close(packed(inputs), converted(inputs), rtol=1e-4, atol=1e-5)
        nested = inputs.reshape(1, rows, 256)
        torch.testing.assert_close(packed(nested), converted(nested), rtol=1e-4, atol=1e-5)


def test_packed_linear_applies_asymmetric_offsets():
    packed, converted = packed_and_reference(mk.int(4, group=64, asym=True))
    assert packed.module[0].zeros is not None
    for rows in (1, 3, 20):
        inputs = torch.randn(rows, 256)
        with torch.inference_mode():
            torch.testing.assert_close(packed(inputs), converted(inputs), rtol=1e-4, atol=1e-5)


def test_packed_linear_executes_error_feedback_codecs():
    calibration = torch.randn(512, 256)
    packed, converted = packed_and_reference(mk.gptq(mk.int(4, group=64), refit=64), calibration=calibration)
    assert converted.quantized["0"].codec == "feedback"
    inputs = torch.randn(3, 256)
    with torch.inference_mode():
        torch.testing.assert_close(packed(inputs), converted(inputs), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("input_width,group", [(255, 64), (256, 5), (250, 20)])
def test_layouts_that_split_a_packing_word_use_dense_reconstruction(input_width, group):
    packed, converted = packed_and_reference(mk.int(4, group=group), input_width=input_width)
    layer = packed.module[0]
    assert layer.layout is None and layer.maximum_fused_rows == 0
    inputs = torch.randn(2, input_width)
    with torch.inference_mode():
        torch.testing.assert_close(packed(inputs), converted(inputs), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(layer.weight, converted.module[0].weight, rtol=1e-6, atol=1e-7)


def test_packed_weight_reconstruction_matches_the_converted_layer():
    for fmt in (mk.int(4, group=64), mk.nf4(group=32), mk.int(4, group=64, asym=True)):
        packed, converted = packed_and_reference(fmt)
        torch.testing.assert_close(packed.module[0].weight, converted.module[0].weight, rtol=1e-6, atol=1e-7)


def test_packed_linear_can_be_copied_and_cast_after_launching():
    packed, converted = packed_and_reference(mk.int(4, group=64), dtype=torch.float16)
    inputs = torch.randn(1, 256, dtype=torch.float16)
    with torch.inference_mode():
        expected = packed(inputs)
        duplicate = copy.deepcopy(packed)
        torch.testing.assert_close(duplicate(inputs), expected, rtol=0, atol=0)
        single = duplicate.module[0].float()
        result = single(inputs.float().cuda())
        torch.testing.assert_close(result, expected.float(), rtol=2e-3, atol=2e-3)
        assert result.dtype == torch.float32


def test_packed_linear_follows_replaced_side_buffers():
    """After a launch, new `scales`, `zeros` and `bias` tensors (assignment, a partial
    load_state_dict(assign=True), re-registration) must be the ones the next launch reads."""
    packed, _ = packed_and_reference(mk.int(4, group=64, asym=True), dtype=torch.float16)
    layer = packed.module[0]
    inputs = torch.randn(2, 256, dtype=torch.float16, device="cuda")

    def dense_product():
        return functional.linear(inputs.float(), layer.weight.float(),
                                 None if layer.bias is None else layer.bias.float())

    with torch.inference_mode():
        torch.testing.assert_close(layer(inputs).float(), dense_product(), rtol=2e-3, atol=2e-3)
        before = layer(inputs).clone()
        layer.scales = (layer.scales.float() * 1.5).half()                      # plain assignment
        torch.testing.assert_close(layer(inputs).float(), dense_product(), rtol=2e-3, atol=2e-3)
        assert not torch.allclose(layer(inputs), before, rtol=1e-2, atol=1e-3)
        state = {"zeros": (layer.zeros.float() + 0.01).half(), "bias": torch.full_like(layer.bias, 0.25)}
        layer.load_state_dict(state, strict=False, assign=True)                 # partial reload
        torch.testing.assert_close(layer(inputs).float(), dense_product(), rtol=2e-3, atol=2e-3)
        layer.register_buffer("scales", (layer.scales.float() * 0.5).half())   # re-registration
        torch.testing.assert_close(layer(inputs).float(), dense_product(), rtol=2e-3, atol=2e-3)


class Attention(nn.Module):
    """q / k / v read the same hidden state; o reads something else."""

    def __init__(self, width=896, heads_kv=128):
        super().__init__()
        self.q_proj = nn.Linear(width, width, bias=True)
        self.k_proj = nn.Linear(width, heads_kv, bias=True)
        self.v_proj = nn.Linear(width, heads_kv, bias=True)
        self.o_proj = nn.Linear(width, width, bias=False)

    def forward(self, x):
        q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        mixed = q * (k.sum(-1, keepdim=True) + v.mean(-1, keepdim=True))
        return self.o_proj(mixed)


def test_sibling_layers_share_one_launch():
    """optimize(group_siblings=True): q / k / v (same parent, same input width and codec) are
    linked; the model's output equals the ungrouped packed model bit for bit, for fp16 rows 1..8,
    under inference_mode and plain no_grad, when an input is modified in place between calls,
    when a member is called alone, after deepcopy, and after a buffer is replaced."""
    torch.manual_seed(49)
    module = Attention().half().cuda()
    converted = mk.quantize(module, mk.int(4, group=128), calib=None)
    plain = mk.optimize(converted, backend="packed")
    grouped = mk.optimize(converted, backend="packed", group_siblings=True)
    attention = grouped.module
    assert attention.q_proj._siblings is attention.k_proj._siblings is attention.v_proj._siblings is not None
    assert attention.o_proj._siblings is None and len(attention.q_proj._siblings.layers) == 3
    for context in (torch.inference_mode, torch.no_grad):
        for rows in (1, 2, 5, 8, 12):
            x = torch.randn(rows, 896, device="cuda").half()
            with context():
                assert torch.equal(grouped(x), plain(x)), (context, rows)
    with torch.no_grad():
        x = torch.randn(2, 896, device="cuda").half()
        q = attention.q_proj(x)                      # leaves k and v pending for this x
        x.mul_(2)                                    # the version changes: pending outputs must not be used
        assert torch.equal(attention.k_proj(x), plain.module.k_proj(x))
        assert torch.equal(q * 0 + attention.q_proj(x), plain.module.q_proj(x))
        other = torch.randn(2, 896, device="cuda").half()
        # another tensor while v's output for x still waits: v does not share its siblings' input and leaves the group
        assert torch.equal(attention.v_proj(other), plain.module.v_proj(other))
        assert attention.v_proj._siblings is None and attention.q_proj._siblings.layers == (attention.q_proj, attention.k_proj)
        assert torch.equal(attention.v_proj(other), plain.module.v_proj(other))
        assert torch.equal(attention.k_proj(other), plain.module.k_proj(other))   # no output waiting: a new launch
        assert torch.equal(attention.k_proj(other), plain.module.k_proj(other))   # a member called twice
        assert len(attention.q_proj._siblings.layers) == 2
    duplicate = copy.deepcopy(grouped)
    assert duplicate.module.q_proj._siblings is not attention.q_proj._siblings
    assert duplicate.module.q_proj._siblings.layers[1] is duplicate.module.k_proj
    with torch.inference_mode():
        x = torch.randn(1, 896, device="cuda").half()
        assert torch.equal(duplicate(x), plain(x))
        attention.k_proj.scales = (attention.k_proj.scales.float() * 2).half()     # a replaced buffer is picked up
        plain.module.k_proj.scales = (plain.module.k_proj.scales.float() * 2).half()
        assert torch.equal(grouped(x), plain(x))


def test_a_layer_that_reads_another_input_leaves_its_sibling_group():
    """q / k / v / o with one input width and codec are all linked at first; o is called with the mixed
    tensor while its output for the hidden state still waits, so it leaves the group on the first forward
    and the later forwards multiply q / k / v in one launch and o in its own."""
    torch.manual_seed(53)
    module = Attention(heads_kv=896)
    module.q_proj.bias = module.k_proj.bias = module.v_proj.bias = None
    module = module.half().cuda()
    converted = mk.quantize(module, mk.int(4, group=128), calib=None)
    plain = mk.optimize(converted, backend="packed")
    grouped = mk.optimize(converted, backend="packed", group_siblings=True)
    attention = grouped.module
    group = attention.q_proj._siblings
    assert attention.o_proj._siblings is group and len(group.layers) == 4
    x = torch.randn(2, 896, device="cuda").half()
    with torch.inference_mode():
        assert torch.equal(grouped(x), plain(x))
    assert attention.o_proj._siblings is None and group.layers == (attention.q_proj, attention.k_proj, attention.v_proj)
    launches = []
    bound = group._bound
    group._bound = lambda: (launches.append(1), bound())[1]
    with torch.inference_mode():
        for _ in range(3):
            x = torch.randn(1, 896, device="cuda").half()
            assert torch.equal(grouped(x), plain(x))
    assert len(launches) == 3 and group._pending is None
    # two layers, one of which never shares: the group dissolves
    pair = SiblingLaunchPair().half().cuda()
    linked = mk.optimize(mk.quantize(pair, mk.int(4, group=128), calib=None), backend="packed", group_siblings=True)
    first, second = linked.module.first, linked.module.second
    assert first._siblings is second._siblings is not None
    with torch.inference_mode():
        y = linked(x)
        assert torch.equal(y, second(first(x)))
    assert first._siblings is None and second._siblings is None


class SiblingLaunchPair(nn.Module):
    """Two layers of one shape in a chain: same parent, same codec, never the same input."""

    def __init__(self):
        super().__init__()
        self.first = nn.Linear(896, 896, bias=False)
        self.second = nn.Linear(896, 896, bias=False)

    def forward(self, x):
        return self.second(self.first(x))


WIDTH_FORMATS = {
    "int2": lambda: mk.int(2, group=64),
    "int3": lambda: mk.int(3, group=64),
    "int5": lambda: mk.int(5, group=64),
    "int6": lambda: mk.int(6, group=32),
    "int7": lambda: mk.int(7, group=64),
    "int8": lambda: mk.int(8, group=128),
    "int3-asymmetric": lambda: mk.int(3, group=64, asym=True),
    "e4m3": lambda: mk.scaled(mk.grid.fp("e4m3"), group=64),
    "codebook3": lambda: mk.scaled(mk.grid.values(torch.linspace(-1, 1, 7).pow(3), bits=3), group=32),
}


@pytest.mark.parametrize("name", WIDTH_FORMATS)
@pytest.mark.parametrize("rows", [1, 3, 20])
def test_packed_linear_executes_every_code_width(name, rows):
    packed, converted = packed_and_reference(WIDTH_FORMATS[name]())
    layer = packed.module[0]
    bits = converted.quantized["0"].metadata["code_bits"]
    assert layer.layout is not None
    assert layer.packed.numel() == 37 * 256 * bits // 8
    inputs = torch.randn(rows, 256)
    with torch.inference_mode():
        torch.testing.assert_close(packed(inputs), converted(inputs), rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(layer.weight, converted.module[0].weight, rtol=1e-6, atol=1e-7)


def test_three_bit_rows_that_split_a_word_use_dense_reconstruction():
    packed, converted = packed_and_reference(mk.int(3, group=50), input_width=250)
    assert packed.module[0].layout is None
    inputs = torch.randn(2, 250)
    with torch.inference_mode():
        torch.testing.assert_close(packed(inputs), converted(inputs), rtol=1e-4, atol=1e-5)


def test_wide_codes_remain_dense():
    converted = mk.quantize(nn.Sequential(nn.Linear(64, 16)), mk.int(12, group=32), calib=None)
    packed = mk.optimize(converted, backend="packed")
    assert isinstance(packed.module[0], nn.Linear)
    assert packed.execution_backend == "packed:0"
    assert mk.optimize(converted, backend="dense").execution_backend == "dense"
    with pytest.raises(ValueError, match="backend must be"):
        mk.optimize(converted, backend="other")
    with pytest.raises(ValueError, match="QModel"):
        mk.optimize(nn.Linear(4, 4), backend="packed")


def test_packed_linear_input_validation():
    packed, _ = packed_and_reference(mk.int(4, group=64))
    layer = packed.module[0]
    with pytest.raises(ValueError, match="input width"):
        layer(torch.randn(1, 128, device="cuda"))
    with pytest.raises(ValueError, match="CUDA inputs"):
        layer(torch.randn(1, 256))
    with pytest.raises(RuntimeError, match="autograd"):
        layer(torch.randn(1, 256, device="cuda", requires_grad=True))
    with pytest.raises(ValueError, match="PackedLinear requires"):
        mk.PackedLinear(nn.Linear(8, 8).cuda(), mk.Q(torch.zeros(8, 8)))


class TiedHead(nn.Module):
    def __init__(self, vocabulary=300, width=128):
        super().__init__()
        self.embed = nn.Embedding(vocabulary, width)
        self.head = nn.Linear(width, vocabulary, bias=False)
        self.head.weight = self.embed.weight

    def forward(self, tokens):
        return self.head(self.embed(tokens))


def test_embedding_tied_to_a_packed_head_reads_the_packed_rows():
    torch.manual_seed(42)
    converted = mk.quantize(TiedHead(), mk.int(4, group=64), calib=None, head=mk.int(4, group=64))
    assert converted.tied_weights == {"embed.weight": "head"}
    packed = mk.optimize(converted, backend="packed")
    assert isinstance(packed.module.embed, mk.PackedEmbedding) and isinstance(packed.module.head, mk.PackedLinear)
    tokens = torch.tensor([[0, 5, 299], [17, 17, 1]], device="cuda")
    dense = converted.quantized["head"].w.cuda()
    torch.testing.assert_close(packed.module.embed(tokens), dense[tokens], rtol=0, atol=0)
    with torch.inference_mode():
        torch.testing.assert_close(packed(tokens), converted(tokens), rtol=1e-4, atol=1e-4)


def test_checkpoint_round_trip(tmp_path):
    torch.manual_seed(43)
    module = nn.Sequential(nn.Linear(64, 48), nn.ReLU(), nn.Linear(48, 16, bias=False))
    converted = mk.quantize(module, mk.int(4, group=16, asym=True), calib=None)
    inputs = torch.randn(4, 64)
    expected = converted(inputs)
    mk.save(converted, tmp_path / "checkpoint")
    with pytest.raises(FileExistsError):
        mk.save(converted, tmp_path / "checkpoint")
    restored = mk.load_checkpoint(tmp_path / "checkpoint",
                                  model=lambda: nn.Sequential(nn.Linear(64, 48), nn.ReLU(), nn.Linear(48, 16, bias=False)))
    torch.testing.assert_close(restored(inputs), expected, rtol=0, atol=0)
    assert restored.quantized["0"].codec == "scaled" and restored.quantized["0"].bits == converted.quantized["0"].bits
    packed = mk.optimize(restored)
    assert packed.execution_backend == "packed:2"
    with torch.inference_mode():
        torch.testing.assert_close(packed(inputs), expected, rtol=1e-4, atol=1e-5)
    mk.save(converted, tmp_path / "checkpoint", overwrite=True)
    assert (tmp_path / "checkpoint" / "mlkit.json").exists() and (tmp_path / "checkpoint" / "weights.safetensors").exists()


def test_capabilities_on_device():
    report = mk.capabilities(mk.int(4, group=128))
    assert report.bits_per_weight == 4.125 and report.codec == "scaled"
    assert report.error_feedback == "fused scalar kernel at step=1"
    assert report.packed_inference == "fused kernel" and report.online_activations == "fused kernel"
    assert mk.capabilities(mk.gptq(mk.int(4))).packed_inference == "fused kernel"
    assert mk.capabilities(mk.int(3, group=50), shape=(16, 250)).packed_inference.startswith("packed storage with dense")
    # vector grids (/root/reference/tests/evaluation/test_capability_report.py:47-72)
    lattice = mk.capabilities(mk.scaled(mk.grid.e8p(), group=None))
    assert lattice.error_feedback == "fused vector kernel at step=8" and lattice.packed_inference == "no; dense weights"
    assert lattice.codec == "vector_scaled" and lattice.bits_per_weight == pytest.approx(2 + 16 / 256)
    quadruples = mk.capabilities(mk.scaled(mk.grid.vector(torch.randn(600, 4)), group=16))
    assert quadruples.error_feedback == "fused vector kernel at step=4"
    assert mk.capabilities(mk.int(12)).error_feedback == "reference rounding with the fitted rounder"


@pytest.mark.parametrize("rows,width", [(70, 1000), (256, 1024)])
def test_whole_sweep_entry_point_equals_the_region_by_region_loop(rows, width, rng):
    """`mk_feedback_sweep` (one call) against the same kernels issued region by region from
    Python (a subclass of Scaled is not eligible for the single call). The second shape is
    whole 128 x 128 tiles, where the single call updates from the deviations its sweep kept."""
    from mlkit_amd.quantization.scaled import Scaled

    class Plain(Scaled):
        pass

    weight = dev(helpers.normal_weight(rows, width, seed=50))   # (70, 1000): ragged last region and tile
    inputs = rng.standard_normal((2048, width)).astype(F32)
    inputs[:, ::11] *= 4
    hessian = dev((inputs.T @ inputs / 2048).astype(F32))
    for asym, refit, block in ((False, 128, 128), (True, 128, 128), (True, 256, 64), (False, None, 128), (True, 96, 128)):
        single = mk.gptq(Scaled(mk.grid.int(4), 32, asym=asym), refit=refit, block_size=block)(weight, Ctx(H=hessian))
        looped = mk.gptq(Plain(mk.grid.int(4), 32, asym=asym), refit=refit, block_size=block)(weight, Ctx(H=hessian))
        assert torch.equal(single.codes, looped.codes)
        assert torch.equal(single.params["scales"], looped.params["scales"])
        assert (single.params["zero"] is None) == (looped.params["zero"] is None)
        if asym:
            assert torch.equal(single.params["zero"], looped.params["zero"])
        assert single.bits == looped.bits and single.params["group"] == looped.params["group"]
        assert single.params["refit"] == looped.params["refit"] and single.metadata == looped.metadata
        assert torch.equal(single.w, looped.w)


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_packed_linear_under_torch_compile(backend):
    """A compiled module holds the fused matvec as the operator `mlkit_amd::packed_matvec`."""
    packed, converted = packed_and_reference(mk.int(4, group=64), dtype=torch.float16)
    inputs = torch.randn(2, 256, dtype=torch.float16, device="cuda")
    with torch.inference_mode():
        expected = packed.module(inputs)
        compiled = torch.compile(packed.module, backend=backend)
        for _ in range(3):
            torch.testing.assert_close(compiled(inputs), expected, rtol=0, atol=0)


def test_optimize_with_compilation_replays_correctly():
    """`mk.optimize(compile=True)` (mode "reduce-overhead": HIP graphs): every replay, with
    eager work between replays, matches the eager packed model."""
    torch.manual_seed(44)
    module = nn.Sequential(nn.Linear(256, 96, dtype=torch.float16), nn.Linear(96, 64, dtype=torch.float16))
    converted = mk.quantize(module, mk.int(4, group=32), calib=None)
    eager = mk.optimize(converted, backend="packed")
    compiled = mk.optimize(converted, backend="packed", compile=True)
    assert compiled.execution_backend == "packed:2+compiled"
    with torch.inference_mode():
        for step in range(5):
            inputs = torch.randn(1, 256, dtype=torch.float16, device="cuda") * (step + 1)
            expected = eager(inputs).clone()
            torch.cuda.synchronize()
            torch.testing.assert_close(compiled(inputs).clone(), expected, rtol=0, atol=0)


class Block(nn.Module):
    def __init__(self, width=896, hidden=4864):
        super().__init__()
        self.up_proj = nn.Linear(width, hidden, bias=False)
        self.down_proj = nn.Linear(hidden, width, bias=False)

    def forward(self, x):
        return self.down_proj(torch.relu(self.up_proj(x)))


def test_online_rotation_survives_quantization_packing_and_checkpoints(tmp_path):
    """Rotated down projection (4864 = 76 x 64, Paley order 76): same function before
    quantization; after quantization the packed model keeps the input rotation, and a checkpoint
    restores both the codes and the rotation."""
    torch.manual_seed(45)
    module = Block().cuda()
    inputs = torch.randn(3, 896, device="cuda")
    expected = module(inputs)
    mk.rotate(seed=7)(module)
    assert module._mlkit_transforms == [{"kind": "rotation", "name": "down_proj",
                                         "seed": mk.layer_seed("down_proj", 7)}]
    torch.testing.assert_close(module(inputs), expected, rtol=1e-4, atol=1e-4)
    converted = mk.quantize(module, mk.int(4, group=64), calib=None)
    assert converted.transforms == module._mlkit_transforms
    quantized_output = converted(inputs)
    packed = mk.optimize(converted, backend="packed")
    down = packed.module.down_proj   # the packed layer runs the rotation itself (one library call per forward)
    assert isinstance(down, mk.PackedLinear) and not down._forward_pre_hooks and down._rotation is not None
    with torch.inference_mode():
        torch.testing.assert_close(packed(inputs), quantized_output, rtol=1e-4, atol=1e-4)
    mk.save(converted, tmp_path / "rotated")
    restored = mk.load_checkpoint(tmp_path / "rotated", model=Block)
    assert restored.transforms == converted.transforms
    torch.testing.assert_close(restored(inputs), quantized_output, rtol=0, atol=0)


@pytest.mark.parametrize("rows,width", [(4096, 14336), (14336, 4096)])
def test_config5_rotated_int4_layer_end_to_end(rows, width):
    """Offline rotation of the weight columns (14336 -> 28 x 512 Paley blocks, 4096 -> one
    FWHT), INT4-g128 quantization, online rotation of fp16 activations and the fused matvec:
    against the oracle's rotated path (the matvec at 1e-3 of the output range on the activations the
    device rotated, those within one fp16 unit in the last place of the oracle's rotation and all but a
    few per cent identical), and against the unrotated fp32 product within quantization error."""
    from mlkit_amd.kernels import hadamard
    from mlkit_amd.quantization.transforms import OnlineRotation, random_signs

    torch.manual_seed(46)
    layer = nn.Linear(width, rows, bias=False, dtype=torch.float16)
    with torch.no_grad():
        layer.weight.normal_(0, 0.02)
    module = nn.ModuleDict({"down_proj": layer}).cuda()
    plain = layer.weight.detach().float().clone()
    mk.rotate(seed=3)(module)
    seed = mk.layer_seed("down_proj", 3)
    converted = mk.quantize(module, mk.int(4, group=128), calib=None)
    packed = mk.optimize(converted, backend="packed", inplace=True)
    fused = packed.module["down_proj"]
    assert isinstance(fused, mk.PackedLinear) and fused.layout is not None
    q = converted.quantized["down_proj"]
    signs = host(random_signs(width, seed, "cuda"))
    dense = scaling.decode_grouped(host(q.codes), host(q.params["scales"]), scaling.int_values(4), 128)
    for samples in (1, 8):
        x = torch.randn(samples, width, device="cuda").half()
        with torch.inference_mode():
            y = fused(x)
        # what the layer's own call rotates (one sample of a power-of-two width inside the matvec kernel, with the
        # stagewise transform's sums; otherwise the row-rotation kernel's), rounded to fp16
        if samples == 1 and width & (width - 1) == 0:
            device_rotated = hadamard.transform(x.float(), signs_before=random_signs(width, seed, "cuda")).half()
        else:
            device_rotated = OnlineRotation(seed)(x)
        helpers.check_rotated_layer(host(y.float()), {"dense": dense}, device_rotated,
                                    oracle_transforms.randomized(host(x.float()), signs), torch.float16)
        exact = host(x.float() @ plain.T)
        relative = np.linalg.norm(host(y.float()) - exact) / np.linalg.norm(exact)
        assert relative < 0.15, relative   # 4-bit rounding noise of a Gaussian layer


@pytest.mark.parametrize("rows,width", [(256, 4096), (512, 14336), (64, 896)])
def test_packed_layer_absorbs_its_online_rotation(rows, width):
    """mk.optimize turns the rotate_inputs pre-hook of a rotated layer into a rotation inside
    PackedLinear.forward: one library call (rotation kernel + matvec) for up to eight rows.
    The result equals hook-then-matvec bit for bit (the same two kernels), for fp16 and bf16,
    for more than eight rows (dense path) and after deepcopy / state reload.  One sample
    of a power-of-two width is rotated inside the matvec kernel, with the sums of the stagewise
    transform: there the result equals the matvec of that transform's output, and the hook's
    (the same sums in another order) to rounding."""
    from mlkit_amd.conversion import RotateInputs
    from mlkit_amd.kernels import hadamard
    from mlkit_amd.quantization.transforms import OnlineRotation, random_signs

    torch.manual_seed(48)
    layer = nn.Linear(width, rows, bias=True, dtype=torch.float16)
    module = nn.ModuleDict({"down_proj": layer}).cuda()
    mk.rotate(seed=4)(module)
    assert any(isinstance(hook, RotateInputs) for hook in module["down_proj"]._forward_pre_hooks.values())
    converted = mk.quantize(module, mk.int(4, group=128), calib=None)
    packed = mk.optimize(converted, backend="packed")
    fused = packed.module["down_proj"]
    assert isinstance(fused, mk.PackedLinear) and not fused._forward_pre_hooks and fused._rotation is not None
    seed = mk.layer_seed("down_proj", 4)
    hook = OnlineRotation(seed)
    plain = copy.deepcopy(fused)
    plain._rotation = None                       # the unrotated layer, fed rotated inputs by hand
    for dtype in (torch.float16, torch.bfloat16):
        for samples in (1, 3, 8, 20):
            if samples > 8 and dtype != layer.weight.dtype:
                continue   # the dense path multiplies in the layer's own dtype (bias included)
            x = torch.randn(samples, width, device="cuda").to(dtype)
            inside = samples == 1 and width & (width - 1) == 0
            with torch.inference_mode():
                rotated = hook(x)
                if inside:
                    stagewise = hadamard.transform(x.float(), signs_before=random_signs(width, seed, "cuda")).to(dtype)
                    assert (stagewise.float() - rotated.float()).abs().max() <= 1.6e-2 * rotated.float().abs().max()
                    rotated = stagewise
                assert torch.equal(fused(x), plain(rotated)), (dtype, samples)
                assert torch.equal(fused(x.view(1, samples, width)), plain(rotated).view(1, samples, rows))
    duplicate = copy.deepcopy(packed).module["down_proj"]
    x = torch.randn(2, width, device="cuda").half()
    with torch.inference_mode():
        assert torch.equal(duplicate(x), fused(x))


@pytest.mark.parametrize("width", [4096, 896])
def test_copies_of_a_rotated_layer_bind_their_own_launch_arguments(width, tmp_path):
    """The bound launch arguments of a layer are raw device addresses.  A deep copy and a pickled layer
    (torch.save of the module) must not carry them: the copy's signs and basis live elsewhere, and in
    another process the addresses mean nothing."""
    import pickle

    torch.manual_seed(52)
    module = nn.ModuleDict({"down_proj": nn.Linear(width, 128, bias=True, dtype=torch.float16)}).cuda()
    mk.rotate(seed=9)(module)
    packed = mk.optimize(mk.quantize(module, mk.int(4, group=128), calib=None), backend="packed")
    fused = packed.module["down_proj"]
    x = torch.randn(2, width, device="cuda").half()
    with torch.inference_mode():
        expected = fused(x)
    assert fused._launch is not None and fused._rotation_launch is not None and fused._rotation_launch[1] is not None
    duplicate = copy.deepcopy(fused)
    torch.save(fused, tmp_path / "layer.pt")
    reloaded = torch.load(tmp_path / "layer.pt", weights_only=False)     # a file this test wrote
    unpickled = pickle.loads(pickle.dumps(fused))
    for other in (duplicate, reloaded, unpickled):
        assert other._launch is None and other._rotation_launch is None and not other._rotation._plans
        with torch.inference_mode():
            assert torch.equal(other(x), expected)
        (order, power, basis, signs, scale), keep = other._rotation_launch[2:]
        assert signs == keep[0].data_ptr() and (basis is None or basis == keep[1].data_ptr())
        assert other._launch[0][0] == other.packed.data_ptr() != fused.packed.data_ptr()
    # a bound tuple whose tensors are not the ones its addresses name is rebuilt, not used
    stale = fused._rotation_launch
    fused._rotation_launch = (stale[0], stale[1], stale[2], tuple(tensor.clone() for tensor in stale[3]))
    with torch.inference_mode():
        assert torch.equal(fused(x), expected)
    (order, power, basis, signs, scale), keep = fused._rotation_launch[2:]
    assert signs == keep[0].data_ptr()


def test_rotation_of_separate_blocks_end_to_end(tmp_path):
    """mk.rotate(seed, block=2048): the down projection's 14336 input features are rotated as
    seven blocks of 2048 (offline on the weight columns, online on the activations).  The
    rotated float layer reproduces the original outputs; quantised and packed, one fp16 row
    goes through one launch and equals the pre-hook followed by the unrotated packed layer bit
    for bit; the block length travels through the checkpoint manifest."""
    from mlkit_amd.conversion import RotateInputs
    from mlkit_amd.quantization.transforms import OnlineRotation

    torch.manual_seed(50)
    rows, width = 256, 14336
    module = nn.ModuleDict({"down_proj": nn.Linear(width, rows, bias=True, dtype=torch.float16)}).cuda()
    x = torch.randn(3, width, device="cuda").half()
    with torch.inference_mode():
        expected = module["down_proj"](x)
    mk.rotate(seed=4, block=2048)(module)
    assert module._mlkit_transforms[0]["block"] == 2048
    hooks = [hook for hook in module["down_proj"]._forward_pre_hooks.values() if isinstance(hook, RotateInputs)]
    assert len(hooks) == 1 and hooks[0].rotation.block == 2048
    with torch.inference_mode():
        rotated_output = module["down_proj"](x)
    assert (rotated_output.float() - expected.float()).abs().max() <= 2e-2 * expected.float().abs().max()
    converted = mk.quantize(module, mk.int(4, group=128), calib=None)
    packed = mk.optimize(converted, backend="packed")
    fused = packed.module["down_proj"]
    assert isinstance(fused, mk.PackedLinear) and fused._rotation is not None and fused._rotation.block == 2048
    plain = copy.deepcopy(fused)
    plain._rotation = None
    hook = OnlineRotation(mk.layer_seed("down_proj", 4), 2048)
    for samples in (1, 2, 8, 20):
        inputs = torch.randn(samples, width, device="cuda").half()
        with torch.inference_mode():
            assert torch.equal(fused(inputs), plain(hook(inputs))), samples
    for samples in (1, 3):   # bf16 activations into the fp16 layer: the same launches in the other type
        inputs = torch.randn(samples, width, device="cuda").bfloat16()
        with torch.inference_mode():
            assert torch.equal(fused(inputs), plain(hook(inputs))), samples
    converted.save(tmp_path / "blocks")
    restored = mk.load_checkpoint(tmp_path / "blocks",
                                  model=lambda: nn.ModuleDict({"down_proj": nn.Linear(width, rows, dtype=torch.float16)}))
    assert restored.transforms[0]["block"] == 2048
    with torch.inference_mode():
        assert torch.equal(restored.module["down_proj"](x), converted.module["down_proj"](x))


def test_checkpoint_mirrors_of_the_reference_tests(tmp_path):
    import json

    def create_model():
        return nn.Sequential(nn.Linear(32, 16), nn.ReLU(), nn.Linear(16, 8))

    torch.manual_seed(47)
    source = create_model()
    before = source[0].weight.detach().clone()
    converted = mk.quantize(source, mk.int(4, group=8), calib=None)
    assert torch.equal(source[0].weight, before)          # the source model is left alone
    directory = tmp_path / "checkpoint"
    converted.save(directory)
    restored = mk.load_checkpoint(directory, model=create_model)
    inputs = torch.randn(4, 32)
    torch.testing.assert_close(restored(inputs), converted(inputs), rtol=0, atol=0)
    assert restored.bpw == converted.bpw
    manifest = json.loads((directory / "mlkit.json").read_text())
    assert manifest["tensor_bytes"] < sum(v.numel() * v.element_size() for v in converted.module.state_dict().values())
    converted.save(directory, overwrite=True)
    restored.save(tmp_path / "restored")
    assert json.loads((tmp_path / "restored" / "mlkit.json").read_text())["tensor_bytes"] == manifest["tensor_bytes"]

    custom = mk.quantize(nn.Sequential(nn.Linear(8, 4)), lambda w, ctx: w.round(), calib=None)
    custom.save(tmp_path / "custom")
    reloaded = mk.load_checkpoint(tmp_path / "custom", model=lambda: nn.Sequential(nn.Linear(8, 4)))
    assert reloaded.bpw is None
    torch.testing.assert_close(custom.module[0].weight, reloaded.module[0].weight)

    root = mk.quantize(nn.Linear(32, 16, bias=False), mk.int(4, group=8), calib=None)
    root.save(tmp_path / "root")
    again = mk.load_checkpoint(tmp_path / "root", model=lambda: nn.Linear(32, 16, bias=False))
    sample = torch.randn(3, 32)
    torch.testing.assert_close(again(sample), root(sample), rtol=0, atol=0)
    packed = mk.optimize(again, inplace=True)
    assert isinstance(packed.module, mk.PackedLinear)
    torch.testing.assert_close(packed(sample), root(sample), rtol=1e-5, atol=1e-6)


def test_checkpoint_stores_tied_weights_and_shared_parameters_once(tmp_path):
    import json

    class TiedLanguageModel(nn.Module):
        def __init__(self):
            super().__init__()
            self.embedding = nn.Embedding(32, 16)
            self.projections = nn.Sequential(nn.Linear(16, 16), nn.Linear(16, 16))
            self.lm_head = nn.Linear(16, 32, bias=False)
            self.lm_head.weight = self.embedding.weight

        def forward(self, tokens):
            return self.lm_head(self.projections(self.embedding(tokens)))

    converted = mk.quantize(TiedLanguageModel(), mk.int(4, group=8), calib=None)
    converted.save(tmp_path / "shared")
    manifest = json.loads((tmp_path / "shared" / "mlkit.json").read_text())
    assert manifest["state_aliases"] == {"lm_head.weight": "embedding.weight"}
    first = manifest["layers"]["projections.0"]["params"]["values"]["tensor"]
    assert first == manifest["layers"]["projections.1"]["params"]["values"]["tensor"]
    restored = mk.load_checkpoint(tmp_path / "shared", model=TiedLanguageModel)
    tokens = torch.randint(32, (2, 7))
    torch.testing.assert_close(restored(tokens), converted(tokens), rtol=0, atol=0)
    assert restored.module.embedding.weight is restored.module.lm_head.weight


def test_row_chunked_conversion_of_a_wide_head_equals_whole_conversion(monkeypatch):
    import mlkit_amd.models as models

    torch.manual_seed(48)
    layer = nn.Linear(256, 1000, bias=False)
    whole = mk.quantize(layer, mk.int(4, group=64), calib=None).quantized[""]
    monkeypatch.setattr(models, "CHUNKED_CONVERSION_ELEMENTS", 1000)
    monkeypatch.setattr(models, "ROW_CHUNK_ELEMENTS", 256 * 96)
    chunked = mk.quantize(layer, mk.int(4, group=64), calib=None).quantized[""]
    assert torch.equal(chunked.codes, whole.codes) and torch.equal(chunked.params["scales"], whole.params["scales"])
    assert chunked.bits == whole.bits and chunked.codec == "scaled"


def test_incoherent_quantization_on_device_and_checkpoint(tmp_path):
    """Two-sided rotation (896 = 28 x 32 Paley rows, 4864 = 76 x 64 columns) around INT4: the
    basis codec decodes on the device, beats plain INT4 on a layer with outlier columns, and
    survives a checkpoint bit for bit."""
    torch.manual_seed(49)
    layer = nn.Linear(4864, 896, bias=False)
    with torch.no_grad():
        layer.weight.normal_(0, 0.02)
        layer.weight[:, ::97] *= 15
    identity = mk.incoherent(lambda w, ctx: mk.Q(w, bits=32 * w.numel()))(layer.weight.detach().cuda())
    torch.testing.assert_close(identity.w, layer.weight.detach().cuda(), rtol=1e-4, atol=1e-5)
    converted = mk.quantize(layer, mk.incoherent(mk.int(4, group=64)), calib=None)
    q = converted.quantized[""]
    assert q.codec == "basis" and q.params["inner_codec"] == "scaled" and q.codes.dtype == torch.uint8
    original = layer.weight.detach().cuda()
    plain = mk.int(4, group=64)(original).w
    assert float((q.w - original).norm()) < 0.8 * float((plain - original).norm())
    assert not mk.packed_compatible(q)
    converted.save(tmp_path / "basis")
    restored = mk.load_checkpoint(tmp_path / "basis", model=lambda: nn.Linear(4864, 896, bias=False))
    torch.testing.assert_close(restored.module.weight, converted.module.weight, rtol=0, atol=0)
    assert restored.quantized[""].params["right_seed"] == q.params["right_seed"]


@pytest.mark.parametrize("width", [4096, 14336, 896, 12])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_online_rotation_hook_equals_rht(width, dtype):
    """The prepared launch of the forward pre-hook against ``mk.rht`` on the same input.  Up to
    64 rows take the per-block kernel (mix, then transform: the same linear map summed in
    another order), so results agree to fp32 rounding: fp32 outputs to 1e-5, 16-bit outputs
    identical except where the rounding of the output sits on a near-tie.  Taller inputs take
    ``rht``'s own kernels and are equal bit for bit; so is a width without a kernel."""
    from mlkit_amd.quantization.transforms import OnlineRotation

    rotation = OnlineRotation(seed=11)
    generator = torch.Generator(device="cuda").manual_seed(width)

    def close(ours, theirs):
        if width < 32:
            return torch.equal(ours, theirs)
        if dtype == torch.float32:
            return torch.allclose(ours, theirs, rtol=1e-5, atol=2e-5)
        step = 2.0 ** (-10 if dtype == torch.float16 else -7) * float(theirs.float().abs().max())
        return float((ours.float() - theirs.float()).abs().max()) <= step and float((ours == theirs).float().mean()) > 0.99

    for rows in (1, 8, 300):
        value = torch.randn((rows, width), device="cuda", generator=generator).to(dtype)
        if rows > 64:
            assert torch.equal(rotation(value), mk.rht(value, seed=11))
        else:
            assert close(rotation(value), mk.rht(value, seed=11))
    wide = torch.randn((4, 2 * width), device="cuda", generator=generator).to(dtype)
    view = wide[:, :width]
    assert close(rotation(view), mk.rht(view, seed=11))
    batched = torch.randn((2, 3, width), device="cuda", generator=generator).to(dtype)
    assert close(rotation(batched), mk.rht(batched, seed=11))
    assert rotation(batched).shape == batched.shape


class GatedBlock(nn.Module):
    """q / k / v on one input, an output projection, and a gated MLP whose down projection is rotated."""

    def __init__(self, hidden: int = 896, inner: int = 2048) -> None:
        super().__init__()
        self.q_proj = nn.Linear(hidden, hidden, bias=True)
        self.k_proj = nn.Linear(hidden, 128, bias=True)
        self.v_proj = nn.Linear(hidden, 128, bias=True)
        self.o_proj = nn.Linear(hidden, hidden, bias=False)
        self.gate_proj = nn.Linear(hidden, inner, bias=False)
        self.up_proj = nn.Linear(hidden, inner, bias=False)
        self.down_proj = nn.Linear(inner, hidden, bias=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        mixed = self.o_proj(q * (k.sum(-1, keepdim=True) + v.mean(-1, keepdim=True)))
        hidden = x + mixed
        return hidden + self.down_proj(torch.nn.functional.silu(self.gate_proj(hidden)) * self.up_proj(hidden))


@pytest.mark.parametrize("group_siblings", [False, True])
@pytest.mark.parametrize("rows", [1, 4])
def test_forward_of_packed_layers_captured_in_a_hip_graph(group_siblings, rows):
    """Serving code captures a decoder block once and replays it.  A block of seven packed layers (three
    siblings on one input, gate / up on another, a down projection with an online rotation of 2048 points) is
    captured with torch.cuda.graph; every replay, with new values in the static input and eager work and
    synchronisations between the replays, equals the eager forward of the same values bit for bit."""
    torch.manual_seed(61)
    module = GatedBlock().half().cuda()
    mk.rotate(seed=5)(nn.ModuleDict({"down_proj": module.down_proj}))
    converted = mk.quantize(module, mk.int(4, group=128), calib=None)
    packed = mk.optimize(converted, backend="packed", group_siblings=group_siblings)
    block = packed.module
    assert isinstance(block.down_proj, mk.PackedLinear) and block.down_proj._rotation is not None
    static = torch.randn(rows, 896, device="cuda").half()
    with torch.inference_mode():
        for _ in range(3):   # binds the launch arguments and the rotation buffers before the capture
            block(static)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = block(static)
        for trial in range(4):
            fresh = torch.randn(rows, 896, device="cuda").half() * (1 + trial)
            static.copy_(fresh)
            graph.replay()
            torch.cuda.synchronize()
            result = captured.clone()
            eager = block(fresh.clone())     # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(result, eager), (group_siblings, rows, trial)


SWEEP_TABLES = [
    (scaling.int_values(4), True), (scaling.int_values(3), True), (scaling.int_values(8), True), (scaling.NF4_VALUES, False),
    (np.array([-1, -.5, -.25, 0, .25, .5, 1], dtype=np.float32), False), ((np.linspace(-1, 1, 40) ** 3).astype(np.float32), False),
    (np.sinh(np.linspace(-3, 3, 256)).astype(np.float32), False), (np.linspace(-1, 1, 17).astype(np.float32), False),
    (np.tanh(np.linspace(-2, 2, 100)).astype(np.float32), False),
]


@pytest.mark.parametrize("seed", [21, 22])
def test_random_gptq_configurations_match_the_oracle_sweep(seed):
    """Twenty-five configurations per seed drawn over grids and tables (7 to 256 values), scale groups, block and
    refit widths (regions that are and are not whole 128-column tiles), offsets, row counts and widths: every sweep
    kernel the dispatch can choose; codes, scales and reconstruction equal the oracle's bit for bit."""
    rng = np.random.default_rng(seed)
    for trial in range(25):
        values, integer = SWEEP_TABLES[rng.integers(len(SWEEP_TABLES))]
        width = int(rng.choice([256, 384, 512, 640, 1024]))
        rows = int(rng.choice([5, 64, 80, 130]))
        group = int(rng.choice([g for g in (16, 32, 64, 128) if width % g == 0]))
        block = int(rng.choice([64, 96, 128, 256]))
        refit = [None, block, 2 * block, 128][rng.integers(4)]
        asym = bool(rng.integers(2))
        weight = helpers.normal_weight(rows, width, seed=100 * seed + trial)
        inputs = rng.standard_normal((3 * width, width)).astype(F32)
        inputs[:, ::9] *= 5
        hessian = (inputs.T @ inputs / (3 * width)).astype(F32)
        bits = int(np.log2(len(values))) if integer else max(4, int(np.ceil(np.log2(len(values)))))
        grid = mk.grid.int(bits) if integer else mk.grid.values(values, bits=bits)
        quantizer = mk.gptq(mk.scaled(grid, group=group, asym=asym), refit=refit, block_size=block)
        result = quantizer(dev(weight), Ctx("layer", H=dev(hessian)))
        coeff = host(mk.feedback_coefficients(dev(hessian).clone(), 1)[0])
        expected = oracle_feedback.sweep(weight, coeff, values, group=group, integer=integer, refit=refit, block=block,
                                         asym=asym, dead=np.diag(hessian) == 0, update_mode=0)
        case = (trial, len(values), integer, rows, width, group, block, refit, asym)
        np.testing.assert_array_equal(host(result.params["scales"]), expected["scales"], err_msg=str(case))
        np.testing.assert_array_equal(host(result.codes), expected["codes"], err_msg=str(case))
        np.testing.assert_array_equal(host(result.w), expected["w"], err_msg=str(case))
