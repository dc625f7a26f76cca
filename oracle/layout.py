"""Oracle (test infrastructure): word geometry of a packed code stream.

Restates ``kernels/packed_linear.py:43-79`` (``PackedLayout``/``layout_for``): a word
is the fewest whole bytes that hold a whole number of codes; a layer runs fused only if
every row and every scale group holds whole words and a tile has at least 16 codes.
"""

import math
from typing import NamedTuple


class Layout(NamedTuple):
    bits: int
    bytes_per_word: int
    codes_per_word: int
    tile_words: int

    @property
    def tile_codes(self) -> int:
        return self.tile_words * self.codes_per_word

    def row_bytes(self, width: int) -> int:
        return width // self.codes_per_word * self.bytes_per_word


def layout_for(bits: int, width: int, group: int) -> Layout | None:
    if bits < 1 or bits > 8:
        return None
    shared = math.gcd(bits, 8)
    codes_per_word, bytes_per_word = 8 // shared, bits // shared
    if width % codes_per_word != 0 or group % codes_per_word != 0:
        return None
    words_in_group = group // codes_per_word
    largest_power = words_in_group & -words_in_group
    tile_words = min(128 // codes_per_word, largest_power)
    if tile_words * codes_per_word < 16:
        return None
    return Layout(bits, bytes_per_word, codes_per_word, tile_words)
