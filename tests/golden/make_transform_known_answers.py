"""Writes tests/golden/transform_known_answers.json: known answers for the conventions of the
structured transforms, worked out with Python integers and hashlib only (no numpy, no torch, nothing
of the oracle or the package), by another route than the implementations take.

  python tests/golden/make_transform_known_answers.py

What each entry fixes, per operations/orthogonal_transforms.py:38-67, codecs/composition.py:14-20 and
quantization/context.py:11-13 in /root/reference:

* ``paley``: the sign pattern (entries times sqrt(order)) of the Paley matrices of order 12, 20, 28, 44.
  The Legendre symbol comes from Euler's criterion ``a^((q-1)/2) mod q`` instead of a table of squares.
  Paley I (q = 3 mod 4), order q + 1: row 0 all +1; rows 1.. have -1 in column 0 and
  ``chi(i - j) + [i == j]`` at (1 + i, 1 + j).  Paley II (q = 1 mod 4), order 2(q + 1): with the
  conference matrix C (C[0][0] = 0, ones in the rest of row and column 0, ``chi(i - j)`` inside) the four
  blocks are [[C + I, C - I], [C - I, -C - I]].
* ``signs``: the integer hash, one 32-bit step at a time, for a few (index + seed) values and the first
  sixteen signs of three seeds (one of them above 2^32, one that wraps past 2^32 inside the range).
* ``layer_seed``: sha256 of "seed:name", its first eight bytes little-endian, modulo 2^63 - 1.
"""

import hashlib
import json
import pathlib


def legendre(value: int, field: int) -> int:
    value %= field
    if value == 0:
        return 0
    return 1 if pow(value, (field - 1) // 2, field) == 1 else -1


def paley_one(field: int) -> list[list[int]]:
    order = field + 1
    rows = [[1] * order]
    for i in range(field):
        rows.append([-1] + [legendre(i - j, field) + (1 if i == j else 0) for j in range(field)])
    return rows


def paley_two(field: int) -> list[list[int]]:
    size = field + 1
    conference = [[0] + [1] * field] + [[1] + [legendre(i - j, field) for j in range(field)] for i in range(field)]
    eye = [[1 if i == j else 0 for j in range(size)] for i in range(size)]
    top = [[conference[i][j] + eye[i][j] for j in range(size)] + [conference[i][j] - eye[i][j] for j in range(size)]
           for i in range(size)]
    bottom = [[conference[i][j] - eye[i][j] for j in range(size)] + [-conference[i][j] - eye[i][j] for j in range(size)]
              for i in range(size)]
    return top + bottom


def hashed(value: int) -> int:
    mask = (1 << 32) - 1
    value &= mask
    value ^= value >> 16
    value = (value * 73244475) & mask          # 0x45D9F3B
    value ^= value >> 16
    value = (value * 73244475) & mask
    value ^= value >> 16
    return value


def signs(width: int, seed: int) -> list[int]:
    return [1 if hashed(index + seed) & 1 else -1 for index in range(width)]


def seed_of(name: str, seed: int) -> int:
    digest = hashlib.sha256((str(seed) + ":" + name).encode("utf-8")).hexdigest()
    first_eight = bytes.fromhex(digest[:16])
    value = sum(byte << (8 * position) for position, byte in enumerate(first_eight))
    return value % ((1 << 63) - 1)


def main() -> None:
    answers = {
        "paley": {"12": paley_one(11), "20": paley_one(19), "28": paley_two(13), "44": paley_one(43)},
        "hash": {str(value): hashed(value) for value in (0, 1, 2, 65536, 123456789, (1 << 32) - 1, (1 << 32) + 5)},
        "signs": [{"seed": seed, "first": signs(16, seed)} for seed in (0, 123456789, (1 << 32) - 8, (1 << 40) + 3)],
        "layer_seed": [{"name": name, "seed": seed, "value": seed_of(name, seed)}
                       for name, seed in (("x", 1), ("model.layers.0.mlp.down_proj", 3), ("", 0),
                                          ("model.layers.31.self_attn.o_proj", 0))],
    }
    path = pathlib.Path(__file__).resolve().parent / "transform_known_answers.json"
    path.write_text(json.dumps(answers, separators=(",", ":")) + "\n")


if __name__ == "__main__":
    main()
