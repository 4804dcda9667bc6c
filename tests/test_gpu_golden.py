"""The GPU library against the golden vectors recorded from the reference's CPU backend (tests/golden/),
through the C ABI: codec bytes, dequantised bf16 and expert ids bit for bit; f32 sums, whose last bits depend
on the summation order, to a relative L2 error of 1e-2 at most (they come out near 1e-6)."""

import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from conftest import rel_l2

sys.path.insert(0, str(Path(__file__).resolve().parent / "golden"))
import cases  # noqa: E402

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).resolve().parent / "golden" / "reference_cpu_generic.npz"


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN, allow_pickle=False)


def as_float(bits):
    if bits.dtype == torch.int32:
        return bits.view(torch.float32)
    if bits.dtype == torch.int16:
        return bits.view(torch.bfloat16).float()
    return bits.float()


@pytest.mark.parametrize("name", sorted(cases.CASES))
def test_gpu_matches_the_reference(hip, golden, name):
    check, outputs = cases.run_case(hip, name)
    assert check == int(golden[f"{name}/inputs_checksum"][0]), "the seeded inputs differ from the recorded run's"
    for key, value in outputs.items():
        want = torch.from_numpy(golden[f"{name}/{key}"])
        if key in cases.EXACT:
            assert torch.equal(value, want), f"{name}/{key}: {(value != want).sum().item()} of {want.numel()} words differ"
        else:
            err = rel_l2(as_float(value), as_float(want))
            assert err <= 1e-2, f"{name}/{key}: relative L2 error {err:.3e}"
