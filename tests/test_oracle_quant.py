"""Pins the oracle's quantisers and dequantiser: against the contract's rules restated in torch (IEEE
divisions, torch's own e4m3 cast), against known answers, and bit for bit against the reference's CPU backend
where that was built."""

import ctypes

import pytest
import torch

import checks
import ops
from dromos_amd.abi import W_BF16, W_FP8, W_INT8, W_NVFP4
from dromos_amd.formats import quantize_with, random_weight


@pytest.mark.parametrize("rows,cols", [(1, 8), (7, 2048), (300, 1000), (2048, 1024)])
def test_int8(oracle, rows, cols):
    checks.quantize_matches_rules(oracle, W_INT8, rows, cols, seed=rows + cols)
    checks.quantize_w8_matches(oracle, rows, cols, seed=rows * 3 + cols)


@pytest.mark.parametrize("rows,cols", [(1, 16), (7, 2048), (300, 1000), (2048, 1024)])
def test_fp8(oracle, rows, cols):
    checks.quantize_matches_rules(oracle, W_FP8, rows, cols, seed=rows * 3 + cols, spread=40.0, zero_row=True)


@pytest.mark.parametrize("rows,cols", [(1, 16), (7, 256), (300, 1024), (1024, 2048)])
def test_nvfp4(oracle, rows, cols):
    checks.quantize_matches_rules(oracle, W_NVFP4, rows, cols, seed=rows + cols * 7, spread=3.0, zero_block=True)


def test_known_answers(oracle):
    checks.int8_known_answers(oracle)
    checks.nvfp4_known_answers(oracle)


@pytest.mark.parametrize("fmt", [W_BF16, W_INT8, W_FP8, W_NVFP4])
@pytest.mark.parametrize("N,K", [(1, 16), (33, 512), (96, 1024)])
def test_dequantize(oracle, fmt, N, K):
    checks.dequantize_is_exact(oracle, fmt, N, K, seed=11 + fmt + N)


def test_dequantize_nvfp4_global_multiplies_once(oracle):
    w = random_weight(W_NVFP4, 64, 256, 3)
    a = ops.dequantize(oracle, w, 64, 256)
    w.glob *= 0.5
    b = ops.dequantize(oracle, w, 64, 256)
    assert torch.equal(b.float(), a.float() * 0.5)


def test_empty_and_invalid(oracle):
    w = torch.zeros(4, 16, dtype=torch.bfloat16)
    q = torch.zeros(4, 16, dtype=torch.int8)
    s = torch.zeros(4)
    assert oracle.status("quantize_w8", w, q, s, ctypes.c_int64(0), 16) == 0
    assert oracle.status("quantize_w8", w, q, s, ctypes.c_int64(4), 0) == 1
    assert oracle.status("quantize_w8", None, q, s, ctypes.c_int64(4), 16) == 1


@pytest.mark.parametrize("fmt", [W_INT8, W_FP8, W_NVFP4])
def test_bytes_equal_the_reference_backend(oracle, ref, fmt):
    g = torch.Generator().manual_seed(17 + fmt)
    w = (torch.randn(257, 1024, generator=g) * torch.rand(257, 1, generator=g) * 5).to(torch.bfloat16)
    w[3] = 0.0
    w[:, 32:48] = 0.0
    a, b = quantize_with(oracle, w, fmt), quantize_with(ref, w, fmt)
    assert torch.equal(a.data.view(torch.uint8), b.data.view(torch.uint8))
    assert torch.equal(a.scale.view(torch.uint8), b.scale.view(torch.uint8)) and a.glob == b.glob
    da, db = ops.dequantize(oracle, a, 257, 1024), ops.dequantize(ref, b, 257, 1024)
    assert torch.equal(da.view(torch.int16), db.view(torch.int16))


# ---- the per-token activation quantiser -------------------------------------------------------------------

ACT_SHAPES = [(1, 2048), (7, 1024), (300, 512), (64, 6400), (5, 4096), (3, 16)]


@pytest.mark.parametrize("pad", [0, 8])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("math", [1, 2, 3])
@pytest.mark.parametrize("M,K", ACT_SHAPES)
def test_quantize_act_matches_the_rules(oracle, M, K, math, x_dtype, pad):
    checks.quantize_act_case(oracle, math, M, K, seed=M * 31 + K + math, x_dtype=x_dtype, pad=pad * 2, x_pad=pad)


@pytest.mark.parametrize("math", [1, 2])
def test_quantize_act_odd_k(oracle, math):
    checks.quantize_act_case(oracle, math, 9, 1001, seed=5, x_pad=3, pad=7)


def test_quantize_act_fp4_extremes(oracle):
    checks.quantize_act_fp4_extremes(oracle)


@pytest.mark.parametrize("math", [1, 2, 3])
def test_quantize_act_equals_the_reference_backend(oracle, ref, math):
    g = torch.Generator().manual_seed(40 + math)
    x = (torch.randn(33, 1024, generator=g) * torch.rand(33, 1, generator=g) * 4).to(torch.bfloat16)
    x[4] = 0
    a, b = ops.quantize_act(oracle, x, math), ops.quantize_act(ref, x, math)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1].view(torch.int32), b[1].view(torch.int32))
    if math == 3:
        assert torch.equal(a[2], b[2])


def test_quantize_act_invalid(oracle):
    x = torch.zeros(4, 24)
    assert ops.quantize_act(oracle, x, 3, status=True) == 1  # FP4 needs K % 16 == 0
    assert ops.quantize_act(oracle, x, 0, status=True) == 1  # BF16 is not a quantised math
    assert ops.quantize_act(oracle, x[:0], 1, status=True) == 0
