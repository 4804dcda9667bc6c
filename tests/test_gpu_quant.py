"""GPU parity: the weight quantisers and the dequantiser through the C ABI, byte for byte against the contract's
rules restated in torch and against the CPU oracle (bit-exact is the bar for codec work)."""

import ctypes

import pytest
import torch

import checks
import ops
from dromos_amd.abi import W_BF16, W_FP8, W_INT8, W_NVFP4
from dromos_amd.formats import Weight, master_weight, quantize_with, random_weight

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols", [(1, 8), (7, 2048), (300, 1000), (2048, 1024), (131072, 1024)])
def test_int8(hip, rows, cols):
    checks.quantize_matches_rules(hip, W_INT8, rows, cols, seed=rows + cols)
    checks.quantize_w8_matches(hip, rows, cols, seed=rows * 3 + cols)


@pytest.mark.parametrize("rows,cols", [(1, 16), (7, 2048), (300, 1000), (2048, 1024), (131072, 1024)])
def test_fp8(hip, rows, cols):
    checks.quantize_matches_rules(hip, W_FP8, rows, cols, seed=rows * 3 + cols, spread=40.0, zero_row=True)


@pytest.mark.parametrize("rows,cols", [(1, 16), (7, 256), (300, 1024), (2048, 2048), (4096, 512)])
def test_nvfp4(hip, rows, cols):
    checks.quantize_matches_rules(hip, W_NVFP4, rows, cols, seed=rows + cols * 7, spread=3.0, zero_block=True)


def test_known_answers(hip):
    checks.int8_known_answers(hip)
    checks.nvfp4_known_answers(hip)


@pytest.mark.parametrize("fmt", [W_BF16, W_INT8, W_FP8, W_NVFP4])
@pytest.mark.parametrize("N,K", [(1, 16), (33, 512), (96, 1024)])
def test_dequantize(hip, fmt, N, K):
    checks.dequantize_is_exact(hip, fmt, N, K, seed=11 + fmt + N)


def test_dequantize_every_code(hip, oracle):
    # All 256 e4m3 codes (the two NaN codes included, which the reference reads as +-480) and all 16 e2m1 codes
    # with every block scale: the GPU's decode tables equal the oracle's bit for bit.
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat(2, 1)
    w = Weight(W_FP8, codes, torch.tensor([1.0, 0.37]))
    a, b = ops.dequantize(hip, w.to("cuda"), 2, 256), ops.dequantize(oracle, w, 2, 256)
    assert torch.equal(a.cpu().view(torch.int16), b.view(torch.int16))
    nib = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat(126, 1)[:, :128].contiguous()  # [126, 128] bytes = 256 k
    nib = (torch.arange(126 * 128, dtype=torch.int32) % 256).to(torch.uint8).view(126, 128)
    scales = (torch.arange(126 * 16, dtype=torch.int32) % 127).to(torch.uint8).view(126, 16)  # valid codes 0..0x7e
    w = Weight(W_NVFP4, nib, scales, glob=0.0371)
    a, b = ops.dequantize(hip, w.to("cuda"), 126, 256), ops.dequantize(oracle, w, 126, 256)
    assert torch.equal(a.cpu().view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("fmt", [W_INT8, W_FP8, W_NVFP4])
def test_baseline_shape_bytes_equal_the_oracle(hip, oracle, fmt):
    # N(0, 0.02) bf16 masters at a decode-sized row length, quantised on the GPU and by the oracle.
    g = torch.Generator().manual_seed(2000 + fmt)
    N, K = (512, 4096) if fmt != W_NVFP4 else (256, 14336)
    w = master_weight(N, K, g)
    a, b = quantize_with(hip, w.cuda(), fmt), quantize_with(oracle, w, fmt)
    assert torch.equal(a.data.cpu().view(torch.uint8), b.data.view(torch.uint8))
    assert torch.equal(a.scale.cpu().view(torch.uint8), b.scale.view(torch.uint8)) and a.glob == b.glob


def test_empty_and_invalid(hip):
    w = torch.zeros(4, 16, dtype=torch.bfloat16, device="cuda")
    q = torch.zeros(4, 16, dtype=torch.int8, device="cuda")
    s = torch.zeros(4, device="cuda")
    assert hip.status("quantize_w8", w, q, s, ctypes.c_int64(0), 16) == 0
    assert hip.status("quantize_w8", w, q, s, ctypes.c_int64(4), 0) == 1
    assert hip.status("quantize_w8", None, q, s, ctypes.c_int64(4), 16) == 1
    assert hip.lib.lx_rt_last_error() == 1 and hip.lib.lx_rt_last_error() == 0


# ---- the per-token activation quantiser -------------------------------------------------------------------

ACT_SHAPES = [(1, 2048), (7, 1024), (300, 512), (64, 6400), (5, 4096), (3, 16)]


@pytest.mark.parametrize("pad", [0, 8])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("math", [1, 2, 3])
@pytest.mark.parametrize("M,K", ACT_SHAPES)
def test_quantize_act_matches_the_rules(hip, M, K, math, x_dtype, pad):
    checks.quantize_act_case(hip, math, M, K, seed=M * 31 + K + math, x_dtype=x_dtype, pad=pad * 2, x_pad=pad)


@pytest.mark.parametrize("math", [1, 2])
def test_quantize_act_odd_k(hip, math):
    checks.quantize_act_case(hip, math, 9, 1001, seed=5, x_pad=3, pad=7)


def test_quantize_act_fp4_extremes(hip):
    checks.quantize_act_fp4_extremes(hip)


@pytest.mark.parametrize("math", [1, 2, 3])
def test_quantize_act_equals_the_oracle(hip, oracle, math):
    g = torch.Generator().manual_seed(40 + math)
    x = (torch.randn(257, 4096, generator=g) * torch.rand(257, 1, generator=g) * 4).to(torch.bfloat16)
    x[4] = 0
    a, b = ops.quantize_act(hip, x.cuda(), math), ops.quantize_act(oracle, x, math)
    assert torch.equal(a[0].cpu(), b[0]) and torch.equal(a[1].cpu().view(torch.int32), b[1].view(torch.int32))
    if math == 3:
        assert torch.equal(a[2].cpu(), b[2])


def test_quantize_act_invalid(hip):
    x = torch.zeros(4, 24, device="cuda")
    assert ops.quantize_act(hip, x, 3, status=True) == 1
    assert ops.quantize_act(hip, x, 0, status=True) == 1
    assert ops.quantize_act(hip, x[:0], 1, status=True) == 0
