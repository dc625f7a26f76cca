"""Pins oracle.bitstream / oracle.layout without the reference: closed forms, brute force,
round trips and the error cases of the reference's tests
(tests/quantization/test_operations.py:65-88, tests/inference/test_packed_linear.py:121-136,189-195)."""

import numpy as np
import pytest

from oracle import bitstream, layout


@pytest.mark.parametrize("bits", range(1, 17))
@pytest.mark.parametrize("elements", [0, 1, 7, 17, 64, 1021])
def test_round_trip_and_length(bits, elements, rng):
    codes = rng.integers(0, 2**bits, size=elements, dtype=np.int64).astype(np.int32)
    packed = bitstream.pack(codes, bits)
    assert packed.dtype == np.uint8 and packed.size == (elements * bits + 7) // 8
    restored = bitstream.unpack(packed, bits, codes.shape)
    assert restored.dtype == (np.uint8 if bits <= 8 else np.int32)
    assert np.array_equal(restored.astype(np.int32), codes)


@pytest.mark.parametrize("bits", range(1, 17))
def test_stream_equals_big_integer_packer(bits, rng):
    codes = rng.integers(0, 2**bits, size=37).tolist()
    expected = np.frombuffer(bitstream.pack_bitwise_python(codes, bits), dtype=np.uint8)
    assert np.array_equal(bitstream.pack(np.array(codes, dtype=np.int32), bits), expected)


def test_known_answers():
    # four bits: even index in the low nibble ("8 per little-endian int32")
    assert bitstream.pack(np.array([0x3, 0xA], dtype=np.uint8), 4).tolist() == [0xA3]
    word = bitstream.pack(np.arange(8, dtype=np.uint8), 4).view("<u4")[0]
    assert word == 0x76543210
    # three bits: eight codes in three bytes, code i at stream bits [3i, 3i+3)
    packed = bitstream.pack(np.arange(8, dtype=np.uint8), 3)
    assert packed.size == 3
    stream = int.from_bytes(packed.tobytes(), "little")
    assert [(stream >> (3 * i)) & 7 for i in range(8)] == list(range(8))
    # two bits, sixteen bits
    assert bitstream.pack(np.array([1, 2, 3, 0], dtype=np.uint8), 2).tolist() == [0b00111001]
    assert bitstream.pack(np.array([0x1234], dtype=np.int32), 16).tolist() == [0x34, 0x12]


def test_validation_errors():
    with pytest.raises(ValueError, match="capacity"):
        bitstream.pack(np.array([16]), 4)
    with pytest.raises(ValueError, match="byte count"):
        bitstream.unpack(np.zeros(1, dtype=np.uint8), 4, (4,))
    with pytest.raises(TypeError):
        bitstream.pack(np.array([0.5]), 4)
    with pytest.raises(ValueError):
        bitstream.pack(np.array([1]), 17)


def test_layout_table_and_negative_cases():
    # (bits, group) -> (bytes_per_word, codes_per_word, tile_words), K = 14336
    table = {
        (4, 128): (1, 2, 64), (4, 64): (1, 2, 32), (2, 64): (1, 4, 16),
        (3, 64): (3, 8, 8), (8, 128): (1, 1, 128), (6, 32): (3, 4, 8), (5, 64): (5, 8, 8),
        (7, 64): (7, 8, 8), (1, 128): (1, 8, 16),
    }
    for (bits, group), expected in table.items():
        found = layout.layout_for(bits, 14336, group)
        assert found is not None and tuple(found[1:]) == expected
        assert found.row_bytes(14336) == 14336 * bits // 8
    assert layout.layout_for(4, 14336, 128).tile_codes == 128
    for width, group in [(255, 64), (256, 5), (250, 20)]:
        assert layout.layout_for(4, width, group) is None
    assert layout.layout_for(3, 250, 50) is None
    assert layout.layout_for(9, 256, 64) is None and layout.layout_for(0, 256, 64) is None
    assert layout.layout_for(4, 256, 16) is not None and layout.layout_for(4, 256, 8) is None
    assert layout.layout_for(3, 96, 48) is not None
