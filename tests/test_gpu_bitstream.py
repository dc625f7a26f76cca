"""GPU parity of the bit-stream kernels (mk_pack / mk_unpack through mk.pack / mk.unpack on
device tensors) and of the row-gather decode (mk_packed_decode_rows) against the oracle:
bit-exact, every code width, ragged counts (tests/quantization/test_operations.py:65-88 in
/root/reference hold the same round trips and error cases on the host)."""

import numpy as np
import pytest
import torch

import mlkit_amd as mk
from oracle import bitstream, scaling

import helpers

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", range(1, 17))
@pytest.mark.parametrize("count", [0, 1, 7, 17, 31, 32, 33, 64, 1021, 4096 * 7 + 5])
def test_pack_and_unpack_match_the_oracle_on_device(bits, count):
    rng = np.random.default_rng(100 * bits + count % 97)
    codes = rng.integers(0, 1 << bits, count, dtype=np.int64)
    expected = bitstream.pack(codes, bits)
    for dtype in (torch.uint8, torch.int16, torch.int32, torch.int64):
        if (dtype == torch.uint8 and bits > 8) or (dtype == torch.int16 and bits > 15):
            continue   # the dtype cannot hold every code of this width
        packed = mk.pack(torch.from_numpy(codes).to(dtype).cuda(), bits)
        assert packed.dtype == torch.uint8 and packed.numel() == (count * bits + 7) // 8
        np.testing.assert_array_equal(packed.cpu().numpy(), expected)
    restored = mk.unpack(torch.from_numpy(expected).cuda(), bits, (count,))
    assert restored.dtype == (torch.uint8 if bits <= 8 else torch.int32)
    np.testing.assert_array_equal(restored.cpu().numpy().astype(np.int64), codes)
    np.testing.assert_array_equal(bitstream.unpack(expected, bits, (count,)).astype(np.int64), codes)


def test_pack_of_a_whole_layer_and_unaligned_streams():
    """4096 x 14336 INT4 and INT3 codes (the stream PackedLinear holds), and streams that start
    at an odd byte of their allocation (the byte-wise variants of both kernels)."""
    rng = np.random.default_rng(5)
    for bits in (4, 3):
        codes = rng.integers(0, 1 << bits, (4096, 14336), dtype=np.uint8)
        packed = mk.pack(torch.from_numpy(codes).cuda(), bits)
        assert packed.numel() == 4096 * 14336 * bits // 8
        expected = bitstream.pack(codes, bits)
        assert torch.equal(packed.cpu(), torch.from_numpy(expected))
        assert torch.equal(mk.unpack(packed, bits, codes.shape).cpu(), torch.from_numpy(codes))
        shifted = torch.empty(packed.numel() + 1, dtype=torch.uint8, device="cuda")
        shifted[1:] = packed
        assert torch.equal(mk.unpack(shifted[1:], bits, codes.shape).cpu(), torch.from_numpy(codes))
    from mlkit_amd import native

    codes = torch.from_numpy(rng.integers(0, 8, 1000, dtype=np.uint8)).cuda()
    target = torch.zeros(376, dtype=torch.uint8, device="cuda")
    native.check(native.library().mk_pack(codes.data_ptr(), 1, 1000, 3, target.data_ptr() + 1, None, None))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(target[1:].cpu().numpy(), bitstream.pack(codes.cpu().numpy(), 3))


def test_pack_error_cases_on_device():
    with pytest.raises(ValueError, match="capacity"):
        mk.pack(torch.tensor([0, 1, 16], device="cuda"), 4)
    with pytest.raises(ValueError, match="capacity"):
        mk.pack(torch.tensor([0, -1, 3], device="cuda"), 4)
    with pytest.raises(TypeError):
        mk.pack(torch.tensor([0.5], device="cuda"), 4)
    with pytest.raises(ValueError):
        mk.pack(torch.tensor([1], device="cuda"), 17)
    with pytest.raises(ValueError, match="byte count"):
        mk.unpack(torch.zeros(3, dtype=torch.uint8, device="cuda"), 4, (7,))


def test_deferred_overflow_flag_collects_the_range_checks():
    """pack(..., overflow=flag) does not read the flag back; one flag serves many calls and is checked once;
    optimize checks the codes of a whole model that way and still raises the reference's error."""
    import mlkit_amd as mk
    from mlkit_amd.quantization.bitstream import check_overflow
    from torch import nn

    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    good = torch.tensor([0, 7, 15, 3], dtype=torch.uint8, device="cuda")
    packed = mk.pack(good, 4, overflow=flag)
    assert packed.tolist() == [0x70, 0x3F]
    check_overflow(flag, 4)
    mk.pack(torch.tensor([1, 16], dtype=torch.uint8, device="cuda"), 4, overflow=flag)   # no error here
    mk.pack(good, 4, overflow=flag)                                                           # the flag stays set
    with pytest.raises(ValueError, match="capacity"):
        check_overflow(flag, 4)
    with pytest.raises(ValueError, match="one-element int32"):
        mk.pack(good, 4, overflow=torch.zeros(2, dtype=torch.int32, device="cuda"))
    assert mk.pack(torch.arange(256, dtype=torch.uint8, device="cuda"), 8).tolist() == list(range(256))
    # a model whose codes do not fit their declared width is refused by optimize
    module = nn.Sequential(nn.Linear(256, 32, dtype=torch.float16)).cuda()
    converted = mk.quantize(module, mk.int(4, group=128), calib=None)
    converted.quantized["0"].codes[3, 5] = 16
    with pytest.raises(ValueError, match="capacity"):
        mk.optimize(converted, backend="packed")


@pytest.mark.parametrize("name,values,bits,integer,group", [
    ("int4", scaling.int_values(4), 4, True, 128), ("int3", scaling.int_values(3), 3, True, 64),
    ("nf4", scaling.NF4_VALUES, 4, False, 64), ("int8", scaling.int_values(8), 8, True, 128),
])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("asym", [False, True])
def test_row_gather_decode_equals_rows_of_the_oracle_decode(name, values, bits, integer, group, out_dtype, asym):
    """The embedding lookup of a tied head: requested rows of the packed matrix, decoded, equal
    the same rows of the oracle's dense reconstruction bit for bit (repeated and unordered
    tokens, width 896 = the 0.5B decoder's hidden size, and a width of ragged wavefronts)."""
    from mlkit_amd import native

    for width in (896, 1056):
        weight = helpers.normal_weight(300, width, seed=90, student_t=True)
        layer = helpers.quantised_layer(weight, values, bits=bits, group=group if width % group == 0 else 32,
                                        integer=integer, asym=asym)
        tensors = helpers.to_device(layer)
        uniform, minimum, step = helpers.uniform_grid(layer["values"])
        # -1 and -300 index from the end as tensor indexing does; 300 and -301 lie outside the table: row 0
        tokens = torch.tensor([0, 299, 5, 5, 17, 128, 1, 299, 64, -1, -300, -7, 300, -301], device="cuda")
        out = torch.empty((tokens.numel(), width), dtype=out_dtype, device="cuda")
        native.check(native.library().mk_packed_decode_rows(
            tensors["packed"].data_ptr(), tensors["scales"].data_ptr(), native.dtype_code(tensors["scales"]),
            tensors["values"].data_ptr(), tensors["values"].numel(), native.pointer(tensors["zeros"]), tokens.data_ptr(),
            tokens.numel(), out.data_ptr(), native.dtype_code(out), 300, width, layer["group"], bits, int(uniform), minimum,
            step, None))
        torch.cuda.synchronize()
        wrapped = np.array([0, 299, 5, 5, 17, 128, 1, 299, 64, 299, 0, 293, 0, 0])
        assert (layer["dense"][np.array([-1, -300, -7])] == layer["dense"][wrapped[9:12]]).all()
        expected = torch.from_numpy(layer["dense"][wrapped]).to(out_dtype)
        assert torch.equal(out.cpu(), expected)
