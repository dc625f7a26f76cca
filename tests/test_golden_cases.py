"""The literal cases of the reference's tests (tests/golden/): the oracle, the host path and,
on a GPU, the kernels give the listed outputs."""

import json
import pathlib

import numpy as np
import pytest
import torch

import mlkit_amd as mk
from oracle import lattice as oracle_lattice

GOLDEN = pathlib.Path(__file__).resolve().parent / "golden"


def load(name):
    return json.loads((GOLDEN / name).read_text())


def test_nearest_keeps_the_original_order_among_ties_on_the_host():
    case = load("nearest_ties.json")
    samples, codebook = np.array(case["samples"], dtype=np.float32), np.array(case["codebook"], dtype=np.float32)
    distances = (samples - codebook.T) ** 2
    assert distances.tolist() == case["squared_distances"]            # the fixture is self-consistent
    assert distances.argmin(1).tolist() == case["indices"]
    assert oracle_lattice.nearest_codes(samples, codebook).tolist() == case["indices"]
    actual = mk.nearest(torch.tensor(case["samples"]), torch.tensor(case["codebook"]), return_indices=True)
    assert actual.tolist() == case["indices"]


@pytest.mark.gpu
def test_nearest_keeps_the_original_order_among_ties_on_the_device():
    case = load("nearest_ties.json")
    samples, codebook = torch.tensor(case["samples"], device="cuda"), torch.tensor(case["codebook"], device="cuda")
    assert mk.nearest(samples, codebook, return_indices=True).tolist() == case["indices"]
    # the same values as vectors of the dimensions the search kernel takes (every coordinate equal)
    for dimension in (2, 4, 8, 16):
        wide_samples, wide_codebook = samples.repeat(1, dimension).contiguous(), codebook.repeat(1, dimension).contiguous()
        assert mk.nearest(wide_samples, wide_codebook, return_indices=True).tolist() == case["indices"], dimension


@pytest.mark.parametrize("device", ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)])
def test_storage_validation_messages(device):
    case = load("storage_errors.json")
    with pytest.raises(ValueError, match=case["pack"]["message"]):
        mk.pack(torch.tensor(case["pack"]["codes"], device=device), case["pack"]["bits"])
    with pytest.raises(ValueError, match=case["unpack"]["message"]):
        mk.unpack(torch.zeros(case["unpack"]["bytes"], dtype=torch.uint8, device=device), case["unpack"]["bits"],
                  tuple(case["unpack"]["shape"]))
