"""Fixtures for the three libraries that speak the lx_* ABI.

    oracle   oracle/liboracle.so           this repository's plain-C restatement (host tensors)
    ref      oracle/_ref/libdromos_cpu.so  the reference's CPU backend where it was built (host tensors);
                                           tests that need it skip when it is absent
    hip      dromos_amd/lib/libdromos_hip.so   the product (device tensors); GPU tests only

Tests marked ``gpu`` need an MI355X; everything else runs on the CPU.
"""

import ctypes
import os
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(Path(__file__).resolve().parent))

from dromos_amd.abi import Kernels, hip_library_path  # noqa: E402

ORACLE_LIB = ROOT / "oracle" / "liboracle.so"
REF_LIB = ROOT / "oracle" / "_ref" / "libdromos_cpu.so"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    if not ORACLE_LIB.exists():
        pytest.fail(f"{ORACLE_LIB} is not built: run `python -m dromos_amd.build` (or make -C oracle oracle)")
    return Kernels(ORACLE_LIB, "cpu")


@pytest.fixture(scope="session")
def ref():
    """The reference's CPU backend. At its generic level (lx_set_arch_override(1)) its f32 sums use four
    lanes and unfused steps, which the oracle reproduces bit for bit."""
    if not REF_LIB.exists():
        pytest.skip("the reference CPU backend is not built here (make -C oracle ref needs /root/reference)")
    k = Kernels(REF_LIB, "cpu")
    k.lib.lx_set_arch_override.restype = ctypes.c_int
    k.lib.lx_set_arch_override.argtypes = [ctypes.c_int]
    return k


@pytest.fixture(scope="session")
def hip():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    # No fallback: a missing library is an error on a GPU box.
    return Kernels(hip_library_path(), "cuda")


def rel_l2(got, want):
    got, want = got.double().cpu().flatten(), want.double().cpu().flatten()
    denom = want.norm().item()
    return (got - want).norm().item() / (denom if denom > 0 else 1.0)


def close(actual, expected, atol, rtol=0.0):
    """Asserts |actual - expected| <= atol + rtol * |expected| elementwise; reports the worst element."""
    a, e = actual.double().cpu(), expected.double().cpu()
    err = (a - e).abs()
    bound = atol + rtol * e.abs()
    worst = (err - bound).argmax()
    assert bool((err <= bound).all()), (
        f"max abs err {err.max().item():.3e} at {worst.item()}: got {a.flatten()[worst].item():.6f}, "
        f"want {e.flatten()[worst].item():.6f}"
    )
