"""GPU parity of the packed matvec (through the C ABI) against the oracle's
reconstruct-then-matmul.  Tolerances: fp16/bf16 activations, max |y - y_ref| <= 1e-3 * max |y_ref|
(fp32 accumulate) against a float64 yardstick, plus the reference's own allclose bounds
(tests/inference/test_packed_linear.py:13-24,91-98,162-186)."""

import ctypes
import functools

import numpy as np
import pytest
import torch

from oracle import bitstream as oracle_bitstream, matvec as oracle_matvec, scaling

import helpers

pytestmark = pytest.mark.gpu


def run_matvec(layer, x, bias=None, scale_dtype=torch.float16):
    from mlkit_amd.kernels import packed_linear

    tensors = helpers.to_device(layer, scale_dtype)
    rows, width = layer["shape"]
    layout = packed_linear.layout_for(layer["bits"], width, layer["group"])
    assert layout is not None
    uniform, minimum, step = helpers.uniform_grid(layer["values"])
    inputs = x.cuda().contiguous()
    output = torch.empty((inputs.shape[0], rows), dtype=inputs.dtype, device="cuda")
    packed_linear.matrix_vector(
        inputs, tensors["packed"], tensors["scales"], tensors["values"], tensors["zeros"],
        None if bias is None else bias.cuda(), output, layer["group"], layout,
        uniform_grid=uniform, grid_minimum=minimum, grid_step=step)
    torch.cuda.synchronize()
    return output.float().cpu().numpy()


def check(y, layer, x, bias=None, relative=1e-3):
    reference = oracle_matvec.reconstruct_then_matmul_f64(
        x.float().numpy(), layer["dense"], None if bias is None else bias.float().numpy())
    scale = np.abs(reference).max()
    error = np.abs(y - reference).max() / scale
    assert error <= relative, f"max error {error:.3e} of the output range"
    return error


INT4 = scaling.int_values(4)


def test_config1_int4_asym_g128_4096x4096():
    weight = helpers.normal_weight(4096, 4096, seed=1)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True, asym=True)
    x = helpers.activations(1, 4096, seed=2)
    y = run_matvec(layer, x)
    check(y, layer, x)
    fp32_reference = oracle_matvec.reconstruct_then_matmul(
        x.float().numpy(), layer["packed"], 4, layer["shape"], layer["scales"], layer["values"],
        128, layer["zero"])
    np.testing.assert_allclose(y, fp32_reference, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("shape", [(896, 896), (128, 896), (4864, 896), (896, 4864)])
@pytest.mark.parametrize("samples", [1, 2, 4, 8])
def test_config2_decoder_shapes_int4_g128(shape, samples):
    weight = helpers.normal_weight(*shape, seed=3, outlier_fraction=0.001)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True)
    x = helpers.activations(samples, shape[1], seed=4)
    check(run_matvec(layer, x), layer, x)


@pytest.mark.parametrize("rows,width", [
    (5120 + 5, 8192),    # 320 tiles of sixteen long rows: a last round a quarter full
    (6144 + 11, 4096),   # 384 tiles of two wavefronts
    (8192 + 3, 2048),    # 512 tiles of one wavefront
    (3584 + 2, 3584),    # fewer tiles than compute units: tall tiles from three samples on
    (3072 + 7, 8192),
    (3072 + 7, 11008),   # six wavefronts: sixteen-row tiles of two spans (the sub-matrix: eight-row tiles)
    (2560 + 9, 12288),   # too few tiles for two spans: the streaming kernel's wavefronts hand over their terms
    (6144 + 3, 14336),   # seven wavefronts: 256 tiles of 24 rows of two spans
    (5120 + 5, 13824),   # 256 tiles of twenty rows
    (7168 + 3, 12288),   # 256 tiles of 28 rows
    (3584 + 5, 11008),   # 256 tiles of fourteen rows
])
@pytest.mark.parametrize("asym", [False, True])
def test_tile_heights_chosen_by_layer_shape(rows, width, asym):
    """Layers for which the launcher leaves its default tile of sixteen (or four) rows: tiles of eight rows where
    sixteen would leave SIMDs idle or the last round sparse, walked by as many workgroups as the GPU holds from
    three samples on, and tall tiles on small layers with several samples.  Every sample count, fp16 and bf16,
    ragged row counts, with bias; with one and two samples every row equals the same row of a launch on a
    sub-matrix that takes the default tiles, bit for bit, since a row's sums do not depend on its tile (nor, for
    rows of six and seven wavefronts, on whether the two-span kernel or the streaming kernel sums them)."""
    weight = helpers.normal_weight(rows, width, seed=rows % 97)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True, asym=asym)
    bias = helpers.activations(1, rows, seed=3)[0]
    part = 2048 if rows < 4096 else 4096
    head = dict(layer, packed=layer["packed"][: part * width // 2], scales=layer["scales"][:part],
                zero=None if layer["zero"] is None else layer["zero"][:part], dense=layer["dense"][:part],
                shape=(part, width))
    for dtype in (torch.float16, torch.bfloat16):
        for samples in (1, 2, 3, 4, 5, 8):
            x = helpers.activations(samples, width, seed=40 + samples, dtype=dtype)
            y = run_matvec(layer, x, bias.to(dtype))
            check(y, layer, x.float(), bias.to(dtype).float(), relative=1e-3 if dtype == torch.float16 else 8e-3)
            if samples <= 2:   # (from three samples on the split of a row over wavefronts depends on the shape too)
                np.testing.assert_array_equal(y[:, :part], run_matvec(head, x, bias[:part].to(dtype)))


@pytest.mark.parametrize("rows,width,group,asym", [
    (4096 + 5, 18944, 128, False),   # sixteen-row tiles, four wavefronts of three spans: two of them have a third span, one partly past the row
    (300, 22016, 64, True),          # eleven spans: three wavefronts of three, one of two
    (67, 24576, 128, False),         # twelve spans, the longest row of three spans per wavefront
    (260, 28672, 128, True),         # four-row tiles, seven wavefronts
    (5120 + 9, 18944, 128, True),    # 256 tiles of twenty rows
    (3072 + 3, 18944, 128, False),   # 256 tiles of twelve rows
    (70, 32768, 64, True),           # the longest row
    (48, 16384 + 32, 32, False),     # one chunk in the second span
    (37, 53248, 128, True),          # beyond two spans: the table kernel's turns
])
def test_rows_of_more_than_16384_codes(rows, width, group, asym):
    """Down projections of the larger decoders (K = 18944, 28672): every wavefront owns two or three spans of 2048 codes.
    One to eight samples, fp16 and bf16 activations, 16-bit and fp32 scales, offsets and bias, against the float64
    product."""
    weight = helpers.normal_weight(rows, width, seed=width % 89)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=group, integer=True, asym=asym)
    bias = helpers.activations(1, rows, seed=3)[0]
    for dtype, scale_dtype in ((torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32)):
        for samples in (1, 2, 3, 4, 5, 8):
            x = helpers.activations(samples, width, seed=50 + samples, dtype=dtype)
            y = run_matvec(layer, x, bias.to(dtype), scale_dtype=scale_dtype)
            sides = {key: None if layer[key] is None else torch.from_numpy(layer[key]).to(scale_dtype).float().numpy()
                     for key in ("scales", "zero")}
            check(y, layer if scale_dtype != torch.bfloat16 else dict(layer, dense=scaling.decode_grouped(
                layer["codes"], sides["scales"], layer["values"], layer["group"], sides["zero"])),
                x.float(), bias.to(dtype).float(), relative=1e-3 if dtype == torch.float16 else 8e-3)


def test_config2_tied_output_head():
    weight = helpers.normal_weight(151936, 896, seed=5, outlier_fraction=0.001)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True)
    for samples in (1, 2, 4, 8):
        x = helpers.activations(samples, 896, seed=6 + samples)
        check(run_matvec(layer, x), layer, x)
    # fp32 activations on the same layer: 9496 tiles of rows, more than the GPU holds workgroups, so a workgroup
    # prepares its digit planes once and walks several tiles with them
    for samples in (1, 2, 3):
        x = helpers.activations(samples, 896, seed=16 + samples, dtype=torch.float32)
        y = run_matvec(layer, x, scale_dtype=torch.float16)
        reference = oracle_matvec.reconstruct_then_matmul_f64(x.double().numpy(), layer["dense"], None)
        np.testing.assert_allclose(y, reference, rtol=1e-4, atol=1e-5)


CODECS = {
    "int2-g64": dict(values=scaling.int_values(2), bits=2, group=64, integer=True),
    "int3-g64": dict(values=scaling.int_values(3), bits=3, group=64, integer=True),
    "nf4-g64": dict(values=scaling.NF4_VALUES, bits=4, group=64, integer=False),
    "cb3-g64-mse": dict(values=np.array([-1, -.5, -.25, 0, .25, .5, 1], dtype=np.float32), bits=3,
                        group=64, integer=False, scale="mse"),
}


@functools.lru_cache(maxsize=1)
def config3_weight(shape):
    return helpers.normal_weight(*shape, seed=7, student_t=True)


@pytest.mark.parametrize("name", CODECS)
@pytest.mark.parametrize("shape", [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)])
def test_config3_sub_byte_and_codebook_codecs(name, shape):
    """Every config-3 layer at its full size (all rows), one and eight samples: the float64
    yardstick at 1e-3 of the output range and the reference's own fp16 bound
    (tests/inference/test_packed_linear.py:13-24 in /root/reference) against the fp32 product."""
    options = dict(CODECS[name])
    values = options.pop("values")
    layer = helpers.quantised_layer(config3_weight(shape), values, **options)
    assert layer["packed"].size == shape[0] * shape[1] * options["bits"] // 8
    for samples in (1, 8):
        x = helpers.activations(samples, shape[1], seed=8 + samples)
        y = run_matvec(layer, x)
        check(y, layer, x)
        fp32_reference = oracle_matvec.reconstruct_then_matmul(x.float().numpy(), None, None, None, None, None,
                                                               None, dense=layer["dense"])
        np.testing.assert_allclose(y, fp32_reference, rtol=2e-3, atol=2e-3)


LONG_ROW_CODECS = dict(CODECS, **{
    "int8-g128": dict(values=scaling.int_values(8), bits=8, group=128, integer=True),
    "int5-g32": dict(values=scaling.int_values(5), bits=5, group=32, integer=True),
    "int6-g64-asym": dict(values=scaling.int_values(6), bits=6, group=64, integer=True, asym=True),
    "int2-g64-asym": dict(values=scaling.int_values(2), bits=2, group=64, integer=True, asym=True),
})


@pytest.mark.parametrize("name", LONG_ROW_CODECS)
@pytest.mark.parametrize("rows,width", [(1040 + 3, 18944), (100, 28672), (48, 16384 + 64), (40, 32768), (35, 53248)])
def test_rows_of_more_than_16384_codes_of_every_codec(name, rows, width):
    """The table kernels cover rows of more than 16384 codes in several turns of the workgroup's width, adding the
    turns' row sums before the reduction.  Every codec, one to eight samples, fp16 and bf16, with bias, ragged
    row counts (rows past the last whole tile), against the float64 product."""
    options = dict(LONG_ROW_CODECS[name])
    values = options.pop("values")
    layer = helpers.quantised_layer(helpers.normal_weight(rows, width, seed=width % 83, student_t=True), values, **options)
    bias = helpers.activations(1, rows, seed=4)[0]
    for dtype in (torch.float16, torch.bfloat16):
        for samples in (1, 2, 3, 4, 5, 8):
            x = helpers.activations(samples, width, seed=70 + samples, dtype=dtype)
            y = run_matvec(layer, x, bias.to(dtype), scale_dtype=dtype)
            sides = {key: None if layer[key] is None else torch.from_numpy(layer[key]).to(dtype).float().numpy()
                     for key in ("scales", "zero")}
            rounded = dict(layer, dense=scaling.decode_grouped(layer["codes"], sides["scales"], layer["values"], layer["group"], sides["zero"]))
            check(y, rounded, x.float(), bias.to(dtype).float(), relative=1e-3 if dtype == torch.float16 else 8e-3)


def test_metric_shape_int4_g128_4096x14336_all_row_counts():
    weight = helpers.normal_weight(4096, 14336, seed=9)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True)
    for samples in (1, 2, 4, 8):
        x = helpers.activations(samples, 14336, seed=10 + samples)
        y = run_matvec(layer, x)
        check(y, layer, x)
        fp32_reference = oracle_matvec.reconstruct_then_matmul(x.float().numpy(), None, None, None, None, None,
                                                               None, dense=layer["dense"])
        np.testing.assert_allclose(y, fp32_reference, rtol=2e-3, atol=2e-3)   # the reference's fp16 bound


@pytest.mark.parametrize("scale_dtype", [torch.float16, torch.bfloat16])
def test_metric_shape_with_bf16_activations(scale_dtype):
    """The same layer in a bf16 model: one and two rows take the bf16 variant of the INT4
    streaming kernel (seven-bit mantissas: one nibble per half and shift), more rows the table kernel."""
    weight = helpers.normal_weight(4096, 14336, seed=9)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True,
                                    fmt="fp16" if scale_dtype == torch.float16 else "bf16")
    for samples in (1, 2, 5):
        x = helpers.activations(samples, 14336, seed=40 + samples, dtype=torch.bfloat16)
        check(run_matvec(layer, x, scale_dtype=scale_dtype), layer, x, relative=8e-3)


def test_down_projection_14336x4096():
    weight = helpers.normal_weight(14336, 4096, seed=11)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True)
    for samples in (1, 8):
        x = helpers.activations(samples, 4096, seed=12)
        check(run_matvec(layer, x), layer, x)


WIDTHS = {
    "int2": (scaling.int_values(2), 2, 64, True),
    "int3": (scaling.int_values(3), 3, 64, True),
    "int5": (scaling.int_values(5), 5, 64, True),
    "int6": (scaling.int_values(6), 6, 32, True),
    "int7": (scaling.int_values(7), 7, 64, True),
    "int8": (scaling.int_values(8), 8, 128, True),
    "codebook3": (np.linspace(-1, 1, 7, dtype=np.float32) ** 3, 3, 32, False),
    "int4-g16": (scaling.int_values(4), 4, 16, True),
    "int3-g48": (scaling.int_values(3), 3, 48, True),
}


@pytest.mark.parametrize("name", WIDTHS)
@pytest.mark.parametrize("samples", [1, 3, 8, 20])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_every_code_width_and_activation_dtype(name, samples, dtype):
    values, bits, group, integer = WIDTHS[name]
    width = 288 if group == 48 else 256
    weight = helpers.normal_weight(37, width, seed=13, scale=1.0)
    for asym in (False, True):
        layer = helpers.quantised_layer(weight, values, bits=bits, group=group, integer=integer,
                                        asym=asym, fmt="fp32")
        assert layer["packed"].size == 37 * width * bits // 8
        x = helpers.activations(samples, width, seed=14, dtype=dtype)
        bias = helpers.activations(1, 37, seed=15, dtype=dtype)[0]
        y = run_matvec(layer, x, bias=bias, scale_dtype=torch.float32)
        if dtype == torch.float32:
            reference = oracle_matvec.reconstruct_then_matmul(
                x.numpy(), layer["packed"], bits, layer["shape"], layer["scales"], layer["values"],
                group, layer["zero"], bias.numpy())
            np.testing.assert_allclose(y, reference, rtol=1e-4, atol=1e-4)
        else:
            check(y, layer, x, bias, relative=1e-3 if dtype == torch.float16 else 8e-3)


def test_rejects_layouts_that_split_a_word():
    from mlkit_amd import native

    lib = native.library()
    assert lib.mk_packed_layout_supported(4, 255, 64) == 0
    assert lib.mk_packed_layout_supported(3, 250, 50) == 0
    assert lib.mk_packed_layout_supported(4, 4096, 128) == 1
    x = torch.zeros(1, 250, device="cuda")
    status = lib.mk_packed_matvec(
        x.data_ptr(), 0, x.data_ptr(), x.data_ptr(), 0, x.data_ptr(), 8, None, None, 0, x.data_ptr(),
        1, 16, 250, 50, 3, 1, 0.0, 1.0, None)
    assert status == native.MK_ERR_UNSUPPORTED
    assert "packing word" in native.last_error()


@pytest.mark.parametrize("name,values,bits,integer", [
    ("int2", scaling.int_values(2), 2, True), ("int3", scaling.int_values(3), 3, True),
    ("nf4", scaling.NF4_VALUES, 4, False), ("e2m1", np.array([-6, -4, -3, -2, -1.5, -1, -.5, 0, .5, 1, 1.5, 2, 3, 4, 6],
                                                             dtype=np.float32), 4, False),
    ("codebook7", np.array([-1, -.5, -.25, 0, .25, .5, 1], dtype=np.float32), 3, False),
])
@pytest.mark.parametrize("group", [32, 128, 2048])
def test_pair_table_kernel_offsets_bias_and_ragged_rows(name, values, bits, integer, group, width=2048):
    """fp16 activations and scales at K = 2048: the LDS pair-table kernel covers rows 0..31 and
    the word kernel rows 32..39; asymmetric offsets, bias and every sample tile."""
    weight = helpers.normal_weight(40, 2048, seed=16, student_t=True)
    for asym in (False, True):
        layer = helpers.quantised_layer(weight, values, bits=bits, group=group, integer=integer, asym=asym)
        for samples in (1, 2, 3, 8, 11):
            x = helpers.activations(samples, 2048, seed=17 + samples)
            bias = helpers.activations(1, 40, seed=18)[0]
            check(run_matvec(layer, x, bias=bias), layer, x, bias)


@pytest.mark.parametrize("width", [32, 896, 2080, 4864])
@pytest.mark.parametrize("bits,values,integer", [(4, INT4, True), (3, scaling.int_values(3), True),
                                                 (4, scaling.NF4_VALUES, False)])
def test_streaming_kernels_on_rows_that_do_not_fill_a_wavefront(width, bits, values, integer):
    """K a multiple of 32 but not of 2048: the trailing lanes of the last wavefront idle."""
    weight = helpers.normal_weight(50, width, seed=19, student_t=True)
    for asym in (False, True):
        layer = helpers.quantised_layer(weight, values, bits=bits, group=32, integer=integer, asym=asym)
        for samples in (1, 4, 8):
            x = helpers.activations(samples, width, seed=20 + samples)
            check(run_matvec(layer, x), layer, x)


@pytest.mark.parametrize("name", WIDTHS)
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("width", [256, 288, 264])
def test_packed_decode_is_exact(name, out_dtype, width):
    """packed -> dense: fp32 output equals the oracle's decode bit for bit, half-precision
    outputs equal its rounding (multiply and add kept separate); 256/288 take the chunk
    kernel, 264 the word kernel."""
    from mlkit_amd.kernels import packed_linear

    values, bits, group, integer = WIDTHS[name]
    if width % group and group != 48:
        group = 8 if bits in (4, 8, 2) else 24 if bits in (3, 6) else 8 * bits if width % (8 * bits) == 0 else group
    layout = packed_linear.layout_for(bits, width, group)
    if layout is None:
        pytest.skip("no fused layout for this combination")
    weight = helpers.normal_weight(21, width, seed=30, scale=1.0)
    for asym in (False, True):
        layer = helpers.quantised_layer(weight, values, bits=bits, group=group, integer=integer, asym=asym)
        tensors = helpers.to_device(layer)
        uniform, minimum, step = helpers.uniform_grid(layer["values"])
        dense = torch.empty((21, width), dtype=out_dtype, device="cuda")
        packed_linear.decode(tensors["packed"], tensors["scales"], tensors["values"], tensors["zeros"], dense,
                             layer["group"], layout, uniform, minimum, step)
        torch.cuda.synchronize()
        expected = torch.from_numpy(layer["dense"]).to(out_dtype)
        assert torch.equal(dense.cpu(), expected)


def test_packed_decode_full_layer_matches_matvec_input():
    """4096 x 14336 INT4-g128 -> fp16: spot rows against the oracle, and the dense product
    agrees with the fused matvec."""
    from mlkit_amd.kernels import packed_linear

    weight = helpers.normal_weight(4096, 14336, seed=31)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True)
    tensors = helpers.to_device(layer)
    dense = torch.empty((4096, 14336), dtype=torch.float16, device="cuda")
    packed_linear.decode(tensors["packed"], tensors["scales"], tensors["values"], None, dense, 128,
                         packed_linear.layout_for(4, 14336, 128), True, -8.0, 1.0)
    torch.cuda.synchronize()
    rows = [0, 1, 777, 4095]
    assert torch.equal(dense[rows].cpu(), torch.from_numpy(layer["dense"][rows]).half())
    x = helpers.activations(2, 14336, seed=32)
    fused = run_matvec(layer, x)
    np.testing.assert_allclose((x.cuda().float() @ dense.float().T).cpu().numpy(), fused, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("bits,values,integer", [(4, INT4, True), (2, scaling.int_values(2), True),
                                                 (3, scaling.int_values(3), True), (4, scaling.NF4_VALUES, False)])
@pytest.mark.parametrize("scale_dtype", [torch.float16, torch.bfloat16])
def test_bf16_activations(bits, values, integer, scale_dtype):
    """bf16 activations (bf16 outputs) with fp16 or bf16 scales; integer grids are exact in the
    bf16 table, so the error is the bf16 rounding of inputs and outputs only."""
    weight = helpers.normal_weight(48, 4096, seed=21, student_t=True)
    for asym in (False, True):
        layer = helpers.quantised_layer(weight, values, bits=bits, group=128, integer=integer, asym=asym,
                                        fmt="fp16" if scale_dtype == torch.float16 else "bf16")
        for samples in (1, 2, 8):
            x = helpers.activations(samples, 4096, seed=22 + samples, dtype=torch.bfloat16)
            check(run_matvec(layer, x, scale_dtype=scale_dtype), layer, x, relative=8e-3)


@pytest.mark.parametrize("width", [256, 512, 896, 1024, 1056, 4864])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name,values,bits,integer", [
    ("int4", INT4, 4, True), ("int2", scaling.int_values(2), 2, True), ("int3", scaling.int_values(3), 3, True),
    ("nf4", scaling.NF4_VALUES, 4, False),
])
def test_short_rows_on_the_streaming_and_block_kernels(width, dtype, name, values, bits, integer):
    """Rows of at most 512 / 1024 codes change the work split (two rows per wavefront step,
    one or two sub-slices per wavefront); 1056 and 4864 leave part of the last wavefront
    empty.  Symmetric and asymmetric, every row count up to eight, 48 and 4112 rows (the
    four-row and the sixteen-row tiling)."""
    tolerance = 1e-3 if dtype == torch.float16 else 8e-3
    for rows in (48, 4112):
        if rows == 4112 and (width not in (896, 1056) or name not in ("int4", "nf4")):
            continue
        weight = helpers.normal_weight(rows, width, seed=50 + width % 97, student_t=True)
        for asym in (False, True):
            layer = helpers.quantised_layer(weight, values, bits=bits, group=32, integer=integer, asym=asym)
            for samples in (1, 2, 3, 4, 7, 8):
                x = helpers.activations(samples, width, seed=60 + samples, dtype=dtype)
                check(run_matvec(layer, x), layer, x, relative=tolerance)


E4M3 = np.array(sorted({s * (m / 8 * 2.0 ** -6 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7))
                        for s in (-1, 1) for e in range(15) for m in range(8)}), dtype=np.float32)


@pytest.mark.parametrize("name,values,bits,integer", [
    ("int5", scaling.int_values(5), 5, True), ("int6", scaling.int_values(6), 6, True),
    ("int7", scaling.int_values(7), 7, True), ("int8", scaling.int_values(8), 8, True),
    ("e4m3", E4M3, 8, False),
])
@pytest.mark.parametrize("width", [2048, 4096, 896])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_wide_codes_on_the_table_kernel(name, values, bits, integer, width, dtype):
    """5- to 8-bit codes with 16-bit activations: single-value or pair tables by width."""
    weight = helpers.normal_weight(40, width, seed=23, student_t=True)
    tolerance = 1e-3 if dtype == torch.float16 else 8e-3
    for asym in (False, True):
        layer = helpers.quantised_layer(weight, values, bits=bits, group=32, integer=integer, asym=asym)
        for samples in (1, 8):
            x = helpers.activations(samples, width, seed=24 + samples, dtype=dtype)
            check(run_matvec(layer, x), layer, x, relative=tolerance)


@pytest.mark.parametrize("name,values,bits,integer", [
    ("int4", INT4, 4, True), ("int3", scaling.int_values(3), 3, True), ("nf4", scaling.NF4_VALUES, 4, False),
    ("int6", scaling.int_values(6), 6, True),
])
def test_widest_rows_fill_the_lds_of_the_block_kernels(name, values, bits, integer, width=16384):
    """K = 16384: eight wavefronts per workgroup, each parking the slices of four samples in
    LDS beside the value table (the largest LDS footprint the matvec kernels ask for)."""
    weight = helpers.normal_weight(48, width, seed=31, student_t=True)
    layer = helpers.quantised_layer(weight, values, bits=bits, group=128, integer=integer, asym=False)
    for samples in (1, 4, 8):
        x = helpers.activations(samples, width, seed=32 + samples)
        check(run_matvec(layer, x), layer, x)


def run_group(layers, x, biases=None, scale_dtype=torch.float16):
    from mlkit_amd.kernels import packed_linear

    first = layers[0]
    width = first["shape"][1]
    layout = packed_linear.layout_for(first["bits"], width, first["group"])
    uniform, minimum, step = helpers.uniform_grid(first["values"])
    tensors = [helpers.to_device(layer, scale_dtype) for layer in layers]
    biases = [None] * len(layers) if biases is None else [None if b is None else b.cuda() for b in biases]
    launch = packed_linear.GroupLaunch(
        [t["packed"] for t in tensors], [t["scales"] for t in tensors], tensors[0]["values"],
        [t["zeros"] for t in tensors], biases, [layer["shape"][0] for layer in layers], width, first["group"], layout,
        uniform_grid=uniform, grid_minimum=minimum, grid_step=step)
    inputs = x.cuda().contiguous()
    outputs = [torch.full((inputs.shape[0], layer["shape"][0]), float("nan"), dtype=inputs.dtype, device="cuda")
               for layer in layers]
    launch(inputs, outputs)
    torch.cuda.synchronize()
    return outputs


@pytest.mark.parametrize("width,rows,asym", [
    (4096, (4096, 1024, 1024), False),      # q / k / v of an 8B-class decoder
    (4096, (14336, 14336), False),          # gate / up
    (896, (896, 128, 128), True),           # q / k / v of the 0.5B-class decoder, short rows, offsets
    (896, (4864, 4864), False),
    (2080, (50, 37, 16), False),            # ragged: rows past the last whole tile, partly filled wavefront
    (14336, (4096, 1040 + 13, 48 + 7), True),   # rows of seven wavefronts: the two-span kernel in the group and (first member) alone; ragged members
    (11008, (2048 + 6, 3000), False),           # six wavefronts; neither member takes the two-span kernel alone
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_grouped_launch_equals_separate_launches(width, rows, asym, dtype):
    """One launch over sibling matrices sharing the activations returns, bit for bit, what one
    launch per matrix returns (which the tests above hold against the oracle), for every row
    count, with and without bias; and the first member is checked against the oracle directly.
    (Both calls give the rows past a member's last whole tile to four-row tiles and only the last rows % 4 to
    the word kernel, whatever tiles the rest of the member takes.  The promise is for one and two samples; with
    more the kernels may split a row by the launch's size, and these shapes are ones where they do not.)"""
    layers = [helpers.quantised_layer(helpers.normal_weight(n, width, seed=70 + i, outlier_fraction=0.001), INT4,
                                      bits=4, group=32 if width % 128 else 128, integer=True, asym=asym)
              for i, n in enumerate(rows)]
    for samples in (1, 2, 3, 4, 8):
        x = helpers.activations(samples, width, seed=80 + samples, dtype=dtype)
        biases = [helpers.activations(1, n, seed=90 + i, dtype=dtype)[0] if i != 1 else None for i, n in enumerate(rows)]
        for with_bias in (False, True):
            chosen = biases if with_bias else None
            grouped = run_group(layers, x, chosen)
            for index, layer in enumerate(layers):
                bias = None if chosen is None else chosen[index]
                separate = run_matvec(layer, x, bias=bias)
                assert np.array_equal(grouped[index].float().cpu().numpy(), separate), (index, samples, with_bias)
            check(grouped[0].float().cpu().numpy(), layers[0], x, None if chosen is None else chosen[0],
                  relative=1e-3 if dtype == torch.float16 else 8e-3)


GROUP_CODECS = {
    "int2": (scaling.int_values(2), 2, True), "int3": (scaling.int_values(3), 3, True),
    "nf4": (scaling.NF4_VALUES, 4, False), "codebook7": (np.array([-1, -.5, -.25, 0, .25, .5, 1], dtype=np.float32), 3, False),
    "int8": (scaling.int_values(8), 8, True),
}


@pytest.mark.parametrize("name", GROUP_CODECS)
@pytest.mark.parametrize("width,rows", [(2048, (64, 40, 16)), (896, (128, 128)), (8192, (48, 32))])
def test_grouped_launch_of_table_codecs(name, width, rows):
    """Sub-byte, codebook and 8-bit codecs through the grouped entry point (one launch of the
    table kernels, members of different heights, rows past a member's last whole tile): equal
    to separate launches bit for bit for every row count, with and without offsets; the first
    member is also held against the oracle."""
    values, bits, integer = GROUP_CODECS[name]
    for asym in (False, True):
        layers = [helpers.quantised_layer(helpers.normal_weight(n, width, seed=75 + i, student_t=True), values, bits=bits,
                                          group=64, integer=integer, asym=asym) for i, n in enumerate(rows)]
        for samples in (1, 2, 3, 8):
            x = helpers.activations(samples, width, seed=76 + samples)
            grouped = run_group(layers, x)
            for index, layer in enumerate(layers):
                assert np.array_equal(grouped[index].float().cpu().numpy(), run_matvec(layer, x)), (index, samples, asym)
            check(grouped[0].float().cpu().numpy(), layers[0], x)


def test_grouped_launch_with_fp32_activations():
    """fp32 activations through the grouped entry point: INT4 uniform grids run as one launch of the digit-plane
    kernel (members of different heights, rows past a member's last whole tile, every sample count), other
    layouts (3-bit codes here) as one launch of the generic kernel per matrix; both equal mk_packed_matvec bit for
    bit, and the first member is held against the float64 product."""
    for values, bits, width, group in ((INT4, 4, 2048, 128), (INT4, 4, 256, 64), (scaling.int_values(3), 3, 256, 64)):
        layers = [helpers.quantised_layer(helpers.normal_weight(n, width, seed=77 + i), values, bits=bits, group=group,
                                          integer=True, fmt="fp32") for i, n in enumerate((37, 21, 64))]
        for samples in (1, 2, 3, 5, 8):
            x = helpers.activations(samples, width, seed=78 + samples, dtype=torch.float32)
            grouped = run_group(layers, x, scale_dtype=torch.float32)
            for index, layer in enumerate(layers):
                assert np.array_equal(grouped[index].cpu().numpy(), run_matvec(layer, x, scale_dtype=torch.float32)), (bits, width, samples, index)
            reference = oracle_matvec.reconstruct_then_matmul_f64(x.double().numpy(), layers[0]["dense"], None)
            np.testing.assert_allclose(grouped[0].cpu().numpy(), reference, rtol=1e-4, atol=1e-5)


def test_grouped_launch_of_tall_members_with_fp32_activations():
    """Four tall members and eight fp32 samples: more (tile, pass, member) units than the GPU holds workgroups, so
    the workgroups of the matrix-core kernel walk their member's tiles; members of different heights (one ends
    inside a tile), offsets and bias.  Equal to the separate launches bit for bit."""
    width, group = 2048, 128
    heights = (8192, 4096 + 16 + 5, 6144, 8192 + 16)
    layers = [helpers.quantised_layer(helpers.normal_weight(n, width, seed=91 + i), INT4, bits=4, group=group,
                                      integer=True, asym=True, fmt="fp32") for i, n in enumerate(heights)]
    for samples in (4, 8):
        x = helpers.activations(samples, width, seed=92 + samples, dtype=torch.float32)
        grouped = run_group(layers, x, scale_dtype=torch.float32)
        for index, layer in enumerate(layers):
            assert np.array_equal(grouped[index].cpu().numpy(), run_matvec(layer, x, scale_dtype=torch.float32)), (samples, index)
        reference = oracle_matvec.reconstruct_then_matmul_f64(x.double().numpy(), layers[1]["dense"], None)
        np.testing.assert_allclose(grouped[1].cpu().numpy(), reference, rtol=1e-4, atol=1e-5)


def test_grouped_launch_validation():
    from mlkit_amd import native

    lib = native.library()
    x = torch.zeros(1, 256, device="cuda", dtype=torch.float16)
    pointers = (ctypes.c_void_p * 9)(*([x.data_ptr()] * 9))
    widths = (ctypes.c_int * 9)(*([16] * 9))
    arguments = lambda count: (pointers, 1, count, pointers, pointers, 1, None, 0, None, None, 0, pointers, widths,  # noqa: E731
                               1, 256, 128, 4, 1, -8.0, 1.0, None)
    assert lib.mk_packed_matvec_group(*arguments(9)) == native.MK_ERR_INVALID
    assert "1 to 8 matrices" in native.last_error()
    assert lib.mk_packed_matvec_group(*arguments(0)) == native.MK_ERR_INVALID


def test_grouped_launch_with_activations_per_matrix():
    """The experts of a mixture-of-experts layer: eight 4096 x 14336 INT4-g128 matrices (two
    distinct weight sets, reused, to bound the oracle's work), each multiplied with its own
    activation row in one launch; every output equals the separate launch and the oracle."""
    from mlkit_amd.kernels import packed_linear

    layers = [helpers.quantised_layer(helpers.normal_weight(4096, 14336, seed=95 + i), INT4, bits=4, group=128,
                                      integer=True) for i in range(2)]
    tensors = [helpers.to_device(layer) for layer in layers]
    members = [tensors[i % 2] for i in range(8)]
    layout = packed_linear.layout_for(4, 14336, 128)
    launch = packed_linear.GroupLaunch([t["packed"] for t in members], [t["scales"] for t in members], members[0]["values"],
                                       [None] * 8, [None] * 8, [4096] * 8, 14336, 128, layout, uniform_grid=True,
                                       grid_minimum=-8.0, grid_step=1.0)
    for samples in (1, 4):
        inputs = [helpers.activations(samples, 14336, seed=120 + i).cuda() for i in range(8)]
        outputs = [torch.full((samples, 4096), float("nan"), dtype=torch.float16, device="cuda") for _ in range(8)]
        launch(inputs, outputs)
        torch.cuda.synchronize()
        for i in range(8):
            separate = run_matvec(layers[i % 2], inputs[i].cpu())
            assert np.array_equal(outputs[i].float().cpu().numpy(), separate), i
        check(outputs[5].float().cpu().numpy(), layers[1], inputs[5].cpu())


@pytest.mark.parametrize("rows,width,asym,with_bias,with_signs", [
    (4096, 4096, False, False, True),      # the rotated down-projection's shape class: sixteen-row tiles
    (256, 2048, True, True, True),         # four-row tiles, one wavefront per workgroup (no exchange through LDS)
    (512, 8192, False, True, False),       # four wavefronts: two exchange stages; no sign vector
    (4096, 16384, True, False, True),      # eight wavefronts, the widest row
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_rotation_inside_the_matvec_kernel(rows, width, asym, with_bias, with_signs, dtype):
    """One fp16 or bf16 sample of an INT4 layer with a power-of-two row: mk_rotated_packed_matvec runs
    the Walsh-Hadamard rotation inside the matvec kernel.  Its stages and sums are the stagewise
    transform's, so the result equals, bit for bit, mk_packed_matvec on activations rotated by
    mk_fwht and rounded to the activation type; and it is the rotated layer of the oracle within tolerance."""
    from mlkit_amd import native
    from mlkit_amd.kernels import hadamard
    from oracle import transforms as oracle_transforms

    weight = helpers.normal_weight(rows, width, seed=rows + width)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True, asym=asym)
    tensors = helpers.to_device(layer, dtype)
    code = native.DTYPE_CODES[dtype]
    x = helpers.activations(1, width, seed=5, dtype=dtype).cuda()
    signs = torch.from_numpy(oracle_transforms.deterministic_signs(width, seed=3)).cuda() if with_signs else None
    bias = helpers.activations(1, rows, seed=6, dtype=dtype)[0].cuda() if with_bias else None
    scale = hadamard.normaliser(width)
    rotated = hadamard.transform(x.float(), signs_before=signs).to(dtype)     # stagewise, scaled, rounded once
    lib = native.library()
    outputs = [torch.full((1, rows), float("nan"), dtype=dtype, device="cuda") for _ in range(2)]
    workspace = torch.full((1, width), float("nan"), dtype=dtype, device="cuda")
    matvec = (tensors["packed"].data_ptr(), tensors["scales"].data_ptr(), native.dtype_code(tensors["scales"]),
              tensors["values"].data_ptr(), 16, native.pointer(tensors["zeros"]), native.pointer(bias), code)
    shape = (1, rows, width, 128, 4, 1, -8.0, 1.0, native.current_stream(x.device))
    native.check(lib.mk_rotated_packed_matvec(x.data_ptr(), code, workspace.data_ptr(), 1, width, None,
                                              native.pointer(signs), scale, *matvec, outputs[0].data_ptr(), *shape))
    native.check(lib.mk_packed_matvec(rotated.data_ptr(), code, *matvec, outputs[1].data_ptr(), *shape))
    torch.cuda.synchronize()
    assert torch.isnan(workspace).all()          # the buffer was not needed
    assert torch.equal(outputs[0], outputs[1])
    host_signs = np.ones(width, dtype=np.float32) if signs is None else signs.cpu().numpy()
    # the stagewise device transform is the oracle's bit for bit: no rotated activation differs at all
    _, differing = helpers.check_rotated_layer(outputs[0].float().cpu().numpy(), layer, rotated,
                                               oracle_transforms.randomized(x.float().cpu().numpy(), host_signs), dtype, bias)
    assert differing == 0.0


@pytest.mark.parametrize("rows,width,block,asym,with_bias,with_signs", [
    (4096, 14336, 2048, False, True, True),     # seven blocks, one per wavefront: no exchange between wavefronts
    (512, 14336, 512, True, False, True),       # four blocks per wavefront: the last lane stages are left out
    (4096, 12288, 4096, False, False, False),   # three blocks of two wavefronts each
    (256, 6144, 64, True, True, True),          # the shortest block: one lane stage
])
def test_rotation_of_separate_blocks_inside_the_matvec_kernel(rows, width, block, asym, with_bias, with_signs):
    """order > 1 without a basis: every block of `power` values is Walsh-Hadamard transformed for
    itself.  One fp16 sample of whole 2048-code slices runs in ONE launch, the transform inside
    the matvec kernel with the stages above the block length left out: bit for bit
    mk_packed_matvec on mk_fwht's output (rows of `block` values) rounded to fp16, the buffer
    untouched.  Two samples take mk_fwht and mk_packed_matvec behind each other and equal the same."""
    from mlkit_amd import native
    from mlkit_amd.kernels import hadamard
    from oracle import transforms as oracle_transforms

    weight = helpers.normal_weight(rows, width, seed=rows + width)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True, asym=asym)
    tensors = helpers.to_device(layer, torch.float16)
    signs = torch.from_numpy(oracle_transforms.deterministic_signs(width, seed=3)).cuda() if with_signs else None
    bias = helpers.activations(1, rows, seed=6)[0].cuda() if with_bias else None
    lib = native.library()
    matvec = (tensors["packed"].data_ptr(), tensors["scales"].data_ptr(), native.dtype_code(tensors["scales"]),
              tensors["values"].data_ptr(), 16, native.pointer(tensors["zeros"]), native.pointer(bias), native.MK_F16)
    for samples in (1, 2):
        x = helpers.activations(samples, width, seed=5 + samples).cuda()
        rotated = hadamard.transform(x.float().view(samples, width // block, block), signs_before=signs).half().view(samples, width)
        outputs = [torch.full((samples, rows), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2)]
        workspace = torch.full((samples, width), float("nan"), dtype=torch.float16, device="cuda")
        shape = (samples, rows, width, 128, 4, 1, -8.0, 1.0, native.current_stream(x.device))
        native.check(lib.mk_rotated_packed_matvec(x.data_ptr(), native.MK_F16, workspace.data_ptr(), width // block, block,
                                                  None, native.pointer(signs), hadamard.normaliser(block), *matvec,
                                                  outputs[0].data_ptr(), *shape))
        native.check(lib.mk_packed_matvec(rotated.data_ptr(), native.MK_F16, *matvec, outputs[1].data_ptr(), *shape))
        torch.cuda.synchronize()
        if samples == 1:
            assert torch.isnan(workspace).all()      # one launch: the buffer was not needed
        else:
            assert torch.equal(workspace, rotated)   # mk_fwht wrote the rotated activations there
        assert torch.equal(outputs[0], outputs[1])
        host_signs = np.ones(width, dtype=np.float32) if signs is None else signs.cpu().numpy()
        blocks = (x.float().cpu().numpy() * host_signs).reshape(samples, width // block, block)
        _, differing = helpers.check_rotated_layer(outputs[0].float().cpu().numpy(), layer, rotated,
                                                   oracle_transforms.fwht(blocks).reshape(samples, width), torch.float16, bias)
        assert differing == 0.0



@pytest.mark.parametrize("rows,width,asym,with_bias,scale_dtype", [
    (64, 14336, False, True, torch.float16),
    (4096 + 23, 4096, True, False, torch.float16),   # 7 rows beyond the last whole tile
    (48, 4864, False, True, torch.bfloat16),      # 38 groups of 128 codes
    (32, 16384, True, True, torch.float16),       # the widest row of the streaming kernels
    (16, 2048, False, False, torch.float16),
    (80, 8192, False, False, torch.float16),
    (32, 8320, False, False, torch.float16),      # 65 groups
    (4096 + 13, 2048, True, True, torch.float16),    # tiles of eight rows (one wavefront per row, many rows), 5 rows beyond
    (4096 + 8, 896, False, False, torch.float16),    # the same with two rows per wavefront step
])
def test_two_to_eight_samples_on_rows_of_many_lengths(rows, width, asym, with_bias, scale_dtype):
    """INT4 with one scale per 128 codes, fp16 activations, every sample count from two to eight, on rows from
    2048 to 16384 codes (ragged tiles of rows, odd numbers of 128-code groups): against the float64 product of
    the oracle's reconstruction at 1e-3 of the output range and the reference's own fp16 bound."""
    weight = helpers.normal_weight(rows, width, seed=rows + width)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True, asym=asym)
    bias = helpers.activations(1, rows, seed=8)[0] if with_bias else None
    for samples in (2, 3, 4, 5, 7, 8):
        x = helpers.activations(samples, width, seed=40 + samples)
        y = run_matvec(layer, x, bias, scale_dtype=scale_dtype)
        if scale_dtype == torch.float16:
            check(y, layer, x, bias)
            fp32_reference = oracle_matvec.reconstruct_then_matmul(
                x.float().numpy(), layer["packed"], 4, layer["shape"], layer["scales"], layer["values"], 128, layer["zero"],
                None if bias is None else bias.float().numpy())
            np.testing.assert_allclose(y, fp32_reference, rtol=2e-3, atol=2e-3)
        else:   # the oracle's scales rounded to bf16: compare with the kernel for one sample, which they also serve
            single = np.concatenate([run_matvec(layer, x[m:m + 1], bias, scale_dtype=scale_dtype) for m in range(samples)])
            assert np.abs(y - single).max() <= 1e-3 * np.abs(single).max()


def test_small_and_large_activations_keep_the_tolerance():
    """Rows of activations a hundred times smaller or two thousand times larger than the usual ones, and a row
    with every second value small: the error stays within the tolerance of each row's output range.  One
    sample at a time the activations meet the codes unscaled, and a row ten thousand times smaller than usual
    (fp16 values near the end of the normal range) keeps the tolerance as well."""
    weight = helpers.normal_weight(64, 4096, seed=77)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True)
    x = helpers.activations(4, 4096, seed=3).float()
    x[0] *= 1e-2
    x[1] *= 2000.0
    x[2, ::2] *= 1e-3
    x = x.half()
    y = run_matvec(layer, x)
    for m in range(4):
        check(y[m:m + 1], layer, x[m:m + 1])
    tiny = (helpers.activations(2, 4096, seed=4).float() * 1e-4).half()
    for samples in (1, 2):
        y = run_matvec(layer, tiny[:samples])
        for m in range(samples):
            check(y[m:m + 1], layer, tiny[m:m + 1])


@pytest.mark.parametrize("rows,width,group,asym,with_bias", [
    (4096, 14336, 128, False, False),   # the metric shape
    (4096 + 5, 4096, 128, True, True),
    (64, 896, 128, False, True),        # two rows per wavefront step
    (48, 2080, 32, True, False),        # a ragged last slice, one scale per chunk
    (32, 256, 256, False, False),       # one scale per row
])
@pytest.mark.parametrize("scale_format", ["fp32", "fp16"])
def test_fp32_activations_on_the_streaming_kernel(rows, width, group, asym, with_bias, scale_format):
    """INT4 with fp32 activations, one to eight samples (what the reference's own matvec tests run,
    tests/inference/test_packed_linear.py:91-98): chunks of 32 activations are scaled by a power of two, rounded
    to 22-bit integers and multiplied with the codes exactly, as planes of 4-bit digits (v_dot8_i32_i4) or, from
    three samples and 1025 codes a row on, of bytes (integer matrix-core blocks).  Against the float64
    product within 1.5e-7 of sum |w| |x| (an fp32 dot product of these lengths measures 2e-8 to 4.5e-8 of it on the
    CPU, this path 1.5e-8 to 8.5e-8), and against the oracle's fp32 reconstruct-then-matmul at the reference's own
    bound (rtol 1e-4, atol 1e-5); with fp32 and with fp16 scales; activations spanning sixty
    times 1e-30 and 1e30, and rows of zeros, keep the bound; activations spanning sixty powers of two inside a
    chunk (which keeps 22 bits of its LARGEST value) keep 1e-6 of the outputs' range."""
    weight = helpers.normal_weight(rows, width, seed=rows + width)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=group, integer=True, asym=asym, fmt=scale_format)
    bias = helpers.activations(1, rows, seed=8, dtype=torch.float32)[0] if with_bias else None
    for samples in (1, 2, 3, 4, 5, 8) + ((9, 33) if rows <= 64 else ()):   # the C ABI takes any count: passes of four
        x = helpers.activations(samples, width, seed=60 + samples, dtype=torch.float32)
        spread = torch.ones(width)
        spread[: width // 2] = 2.0 ** torch.randint(-30, 30, (width // 2,), generator=torch.Generator().manual_seed(3)).float()
        for scaled in (x, x * 1e-30, x * 1e30, torch.zeros_like(x), x * spread):
            y = run_matvec(layer, scaled, bias, scale_dtype=torch.float32 if scale_format == "fp32" else torch.float16)
            reference = oracle_matvec.reconstruct_then_matmul_f64(
                scaled.double().numpy(), layer["dense"], None if bias is None else bias.double().numpy())
            budget = 1.5e-7 * (np.abs(scaled.double().numpy()) @ np.abs(layer["dense"]).T.astype(np.float64)) + 1e-7 * np.abs(reference) + 1e-30
            if torch.equal(scaled, x * spread) and not torch.equal(scaled, x):
                # the error is bounded against the outputs' range, which the large values make
                assert np.abs(y - reference).max() <= 1e-6 * np.abs(reference).max()
                continue
            worst = float((np.abs(y - reference) / budget).max())
            assert worst <= 1.0, (samples, worst)
            if scaled is x:
                fp32_reference = oracle_matvec.reconstruct_then_matmul(
                    x.numpy(), layer["packed"], 4, layer["shape"], layer["scales"], layer["values"], group, layer["zero"],
                    None if bias is None else bias.numpy())
                np.testing.assert_allclose(y, fp32_reference, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("scale_format", ["fp32", "fp16"])
def test_fp32_activations_on_layers_taller_than_the_gpu_holds_workgroups(scale_format):
    """Five to eight fp32 samples of a layer with more tiles of sixteen rows, times two passes of four samples, than
    the GPU holds workgroups at once: every workgroup of the matrix-core kernel prepares its activations once and
    walks several tiles.  With offsets and bias, against the float64 product at the bound of the test above."""
    rows, width, group = 8192 + 16 + 3, 8192, 128
    weight = helpers.normal_weight(rows, width, seed=31)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=group, integer=True, asym=True, fmt=scale_format)
    bias = helpers.activations(1, rows, seed=9, dtype=torch.float32)[0]
    for samples in (5, 8):
        x = helpers.activations(samples, width, seed=80 + samples, dtype=torch.float32)
        y = run_matvec(layer, x, bias, scale_dtype=torch.float32 if scale_format == "fp32" else torch.float16)
        reference = oracle_matvec.reconstruct_then_matmul_f64(x.double().numpy(), layer["dense"], bias.double().numpy())
        budget = 1.5e-7 * (np.abs(x.double().numpy()) @ np.abs(layer["dense"]).T.astype(np.float64)) + 1e-7 * np.abs(reference) + 1e-30
        worst = float((np.abs(y - reference) / budget).max())
        assert worst <= 1.0, (samples, worst)


def test_fp32_activations_that_are_not_finite_stay_so():
    """The reference's fp32 matmul answers an infinite or NaN activation with outputs that are not finite; the digit
    planes answer with NaN for every row (the chunk's factor becomes NaN), and other samples are not touched."""
    weight = helpers.normal_weight(64, 4096, seed=9)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=128, integer=True, asym=False, fmt="fp16")
    for samples in (1, 2, 4):
        for poison in (float("inf"), float("-inf"), float("nan")):
            x = helpers.activations(samples, 4096, seed=70 + samples, dtype=torch.float32)
            clean = run_matvec(layer, x, None, scale_dtype=torch.float16)
            x[0, 1234] = poison
            y = run_matvec(layer, x, None, scale_dtype=torch.float16)
            assert not np.isfinite(y[0]).any()
            np.testing.assert_array_equal(y[1:], clean[1:])


def test_fp32_activations_with_bf16_scales():
    """fp32 activations against bf16 scales and offsets (the digit-plane kernel converts the sides itself): against
    the float64 product of the weights that those rounded scales and offsets give."""
    rows, width, group = 80, 4096, 128
    weight = helpers.normal_weight(rows, width, seed=21)
    layer = helpers.quantised_layer(weight, INT4, bits=4, group=group, integer=True, asym=True)
    scales = torch.from_numpy(layer["scales"]).bfloat16().double().numpy()
    zeros = torch.from_numpy(layer["zero"]).bfloat16().double().numpy()
    codes = oracle_bitstream.unpack(layer["packed"], 4, layer["shape"]).astype(np.float64)
    dense = (codes + float(layer["values"][0])) * np.repeat(scales, group, axis=1) + np.repeat(zeros, group, axis=1)
    for samples in (1, 2, 4):
        x = helpers.activations(samples, width, seed=22 + samples, dtype=torch.float32)
        y = run_matvec(layer, x, scale_dtype=torch.bfloat16)
        np.testing.assert_allclose(y, x.double().numpy() @ dense.T, rtol=1e-4, atol=1e-5)


SWEEP_CODECS = [
    (scaling.int_values(4), 4, True), (scaling.int_values(2), 2, True), (scaling.int_values(3), 3, True),
    (scaling.int_values(8), 8, True), (scaling.NF4_VALUES, 4, False),
    (np.array([-1, -.5, -.25, 0, .25, .5, 1], dtype=np.float32), 3, False), (scaling.int_values(5), 5, True),
    (scaling.int_values(6), 6, True),
]


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_layouts_against_the_oracle(seed):
    """Forty layers per seed drawn over the codecs, row lengths (32 ... 16384), scale groups, row counts (ragged
    tiles, short and tall matrices), offsets, bias, the three activation types and one to nine samples: every kernel
    the dispatch can choose, against the float64 product at the tolerance of the activation type."""
    rng = np.random.default_rng(seed)
    for trial in range(40):
        values, bits, integer = SWEEP_CODECS[rng.integers(len(SWEEP_CODECS))]
        width = int(rng.choice([32, 64, 96, 256, 512, 896, 1024, 1536, 2048, 2080, 3072, 4096, 4864, 6144, 8192, 11008, 14336, 16384]))
        group = int(rng.choice([g for g in (32, 64, 128, 256) if width % g == 0] + [width]))
        tall = [1, 3, 16, 37, 64, 130, 260, 1024, 4096 + 5, 4100, 6144, 9000]
        rows = int(rng.choice(tall)) if width <= 4096 else int(rng.choice([3, 16, 40, 4096 + 7]))
        asym, with_bias = bool(rng.integers(2)), bool(rng.integers(2))
        dtype = [torch.float16, torch.bfloat16, torch.float32][rng.integers(3)]
        samples = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9]))
        weight = helpers.normal_weight(rows, width, seed=100 * seed + trial)
        layer = helpers.quantised_layer(weight, values, bits=bits, group=group, integer=integer, asym=asym)
        x = helpers.activations(samples, width, seed=1000 + trial, dtype=dtype)
        bias = helpers.activations(1, rows, seed=5, dtype=dtype)[0] if with_bias else None
        y = run_matvec(layer, x, bias)
        reference = oracle_matvec.reconstruct_then_matmul_f64(
            x.double().numpy(), layer["dense"], None if bias is None else bias.double().numpy())
        tolerance = {torch.float16: 1e-3, torch.bfloat16: 8e-3, torch.float32: 2e-5}[dtype]
        error = np.abs(y - reference).max() / max(np.abs(reference).max(), 1e-30)
        assert error <= tolerance, (trial, bits, integer, rows, width, group, asym, with_bias, dtype, samples, error)


@pytest.mark.parametrize("seed", range(8))
def test_random_shapes_alone_and_grouped(seed):
    """Seeded random layers (any width that is a multiple of 32 up to 14336 and some up to 32768, ragged row counts,
    fp16 / bf16, offsets, bias, one to eight samples): every output within the tolerance of the float64 product; with
    one and two samples a sub-matrix of whole tiles (which takes other tiles or another kernel) and a grouped launch
    over the layer and that sub-matrix return the same bits as the layer alone."""
    rng = np.random.default_rng(1000 + seed)
    width = int(rng.integers(1, 14336 // 32 + 1)) * 32 if seed % 4 else int(rng.integers(16384 // 32 + 1, 32768 // 32 + 1)) * 32
    group = int(rng.choice([32, 64, 128, width]))
    if width % group:
        group = 32
    rows = int(rng.integers(40, max(41, min(2600, 24_000_000 // width))))
    asym = bool(rng.integers(2))
    dtype = (torch.float16, torch.bfloat16)[int(rng.integers(2))]
    layer = helpers.quantised_layer(helpers.normal_weight(rows, width, seed=seed), INT4, bits=4, group=group, integer=True, asym=asym)
    if dtype == torch.bfloat16:   # the layer as the kernel sees it: scales and offsets rounded to bf16
        sides = {key: None if layer[key] is None else torch.from_numpy(layer[key]).to(dtype).float().numpy() for key in ("scales", "zero")}
        layer = dict(layer, dense=scaling.decode_grouped(layer["codes"], sides["scales"], layer["values"], group, sides["zero"]))
    part = (rows // 3) // 16 * 16
    head = dict(layer, packed=layer["packed"][: part * width // 2], scales=layer["scales"][:part],
                zero=None if layer["zero"] is None else layer["zero"][:part], dense=layer["dense"][:part], shape=(part, width))
    bias = helpers.activations(1, rows, seed=3, dtype=dtype)[0]
    for samples in (1, 2, int(rng.choice([3, 4, 5, 8]))):
        x = helpers.activations(samples, width, seed=20 + samples, dtype=dtype)
        y = run_matvec(layer, x, bias, scale_dtype=dtype)
        check(y, layer, x.float(), bias.float(), relative=1e-3 if dtype == torch.float16 else 8e-3)
        if samples <= 2 and part >= 16:
            alone = run_matvec(head, x, bias[:part], scale_dtype=dtype)
            np.testing.assert_array_equal(y[:, :part], alone)
            grouped = run_group([layer, head], x, [bias, bias[:part]], scale_dtype=dtype)
            np.testing.assert_array_equal(grouped[0].float().cpu().numpy(), y)
            np.testing.assert_array_equal(grouped[1].float().cpu().numpy(), alone)
