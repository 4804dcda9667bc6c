"""The oracle against the golden vectors recorded from the reference's CPU backend (tests/golden/): every
output bit for bit, the f32 sums included, because the oracle restates the generic level's summation order."""

import sys
from pathlib import Path

import numpy as np
import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent / "golden"))
import cases  # noqa: E402

GOLDEN = Path(__file__).resolve().parent / "golden" / "reference_cpu_generic.npz"


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN, allow_pickle=False)


def test_every_case_is_recorded(golden):
    recorded = {k.split("/")[0] for k in golden.files}
    assert recorded == set(cases.CASES)


@pytest.mark.parametrize("name", sorted(cases.CASES))
def test_oracle_reproduces_the_reference_bits(oracle, golden, name):
    check, outputs = cases.run_case(oracle, name)
    assert check == int(golden[f"{name}/inputs_checksum"][0]), "the seeded inputs differ from the recorded run's"
    for key, value in outputs.items():
        want = torch.from_numpy(golden[f"{name}/{key}"])
        assert torch.equal(value, want), f"{name}/{key}: {(value != want).sum().item()} of {want.numel()} words differ"
