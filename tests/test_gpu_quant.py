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
    # N(0, 0.02) bf16 masters at a BASELINE-sized row length, quantised on the GPU and by the oracle.
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
