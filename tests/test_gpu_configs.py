"""GPU parity at the full shapes of the benchmark configurations, through the C ABI: the CPU oracle on the same
inputs, and the bitwise contracts at the shapes where the row count chooses between kernels (a row's bits must not
depend on how many rows ride along, whichever kernel a row count lands on).

    C2  int8 / fp8 W 14336 x 4096, M in {1, 4, 16, 64}, default and batch-invariant mode
    C3  nvfp4 W 4096 x 14336
    C5  fp8, 32 rows: QKV 6144 x 4096, O 4096 x 4096, in_proj 16384 x 4096, out_proj 4096 x 8192, and the routed
        experts E = 128, L = 4096, I = 1536, top-8
"""

import os

import pytest
import torch

import ops
from conftest import rel_l2
from dromos_amd.abi import FORMATS, MATH_BF16, MATH_FP8, W_FP8
from dromos_amd.formats import Weight, alloc_quantized, master_weight, quantize_with, random_weight

pytestmark = pytest.mark.gpu
FMT = list(FORMATS)
ROWS = (1, 2, 4, 8, 16, 17, 64)


def bits(t):
    return t.view(torch.int32)


class invariant_mode:
    """LX_BATCH_INVARIANT=1 for the block (the library reads the variable on every call)."""

    def __enter__(self):
        os.environ["LX_BATCH_INVARIANT"] = "1"

    def __exit__(self, *exc):
        del os.environ["LX_BATCH_INVARIANT"]


# ---- a row's bits across row counts, at the shapes where the row count picks the kernel ----------------------


@pytest.mark.parametrize("N,K", [(14336, 4096), (16384, 4096)])
@pytest.mark.parametrize("fmt", FMT)
def test_rows_keep_their_bits_across_row_counts(hip, fmt, N, K):
    # engine/cuda/kernels.h:453-477: 896 and 1024 weight tiles; one row, a few rows, 16, 17 and 64 rows each take a
    # different kernel or a different shape of the same one.
    w = random_weight(FORMATS[fmt], N, K, N % 97).to("cuda")
    x = torch.randn(64, K, generator=torch.Generator().manual_seed(N)).to(torch.bfloat16).cuda()
    bias = torch.randn(N, generator=torch.Generator().manual_seed(K)).cuda()
    full = ops.gemm_skinny(hip, x, w, bias=bias)
    for M in ROWS:
        part = ops.gemm_skinny(hip, x[:M].contiguous(), w, bias=bias)
        assert torch.equal(bits(part), bits(full[:M])), f"lx_gemm_skinny: rows of an M={M} call differ from those of M=64"
        part = ops.gemm_w(hip, x[:M].contiguous(), w, MATH_BF16, bias=bias)
        assert torch.equal(bits(part), bits(full[:M])), f"lx_gemm_w: rows of an M={M} call differ from lx_gemm_skinny M=64"
    # a row somewhere in the middle, alone
    alone = ops.gemm_w(hip, x[37:38].contiguous(), w, MATH_BF16, bias=bias)
    assert torch.equal(bits(alone[0]), bits(full[37]))
    with invariant_mode():
        for M in (1, 2, 4, 8):
            y = ops.gemv_w(hip, x[:M].contiguous(), w, bias=bias)
            assert torch.equal(bits(y), bits(full[:M])), f"batch-invariant lx_gemv_w M={M} differs from lx_gemm_w M=64"
        assert torch.equal(bits(ops.gemm_w(hip, x, w, MATH_BF16, bias=bias)), bits(full))
    # The streaming GEMV (default mode) has its own sums; its rows do not depend on the row count either.
    y8 = ops.gemv_w(hip, x[:8].contiguous(), w, bias=bias)
    for M in (1, 2, 3, 4, 5):
        assert torch.equal(bits(ops.gemv_w(hip, x[:M].contiguous(), w, bias=bias)), bits(y8[:M])), f"lx_gemv_w M={M}"
    assert rel_l2(y8, full[:8]) < 1e-5


@pytest.mark.parametrize("N,K", [(14336, 4096), (16384, 4096)])
def test_fp8_math_rows_keep_their_bits_across_row_counts(hip, N, K):
    w = random_weight(W_FP8, N, K, 11).to("cuda")
    x = torch.randn(64, K, generator=torch.Generator().manual_seed(N + 1)).to(torch.bfloat16).cuda()
    full = ops.gemm_w(hip, x, w, MATH_FP8)
    for M in ROWS:
        part = ops.gemm_w(hip, x[:M].contiguous(), w, MATH_FP8)
        assert torch.equal(bits(part), bits(full[:M])), f"FP8 math: rows of an M={M} call differ from those of M=64"


# ---- C2 in batch-invariant mode ----------------------------------------------------------------------------------


@pytest.mark.parametrize("fmt", ["int8", "fp8"])
def test_c2_batch_invariant_mode(hip, oracle, fmt):
    N, K = 14336, 4096
    g = torch.Generator().manual_seed(1001)
    master = master_weight(N, K, g)
    x = torch.randn(64, K, generator=g).to(torch.bfloat16)
    w = quantize_with(hip, master.cuda(), FORMATS[fmt])
    xd = x.cuda()
    with invariant_mode():
        y64 = ops.gemm_w(hip, xd, w, MATH_BF16)
        y16 = ops.gemm_w(hip, xd[:16].contiguous(), w, MATH_BF16)
        y4 = ops.gemv_w(hip, xd[:4].contiguous(), w)
        y1 = ops.gemv_w(hip, xd[:1].contiguous(), w)
    assert torch.equal(bits(y16), bits(y64[:16])), "M=16 rows differ from M=64 rows"
    assert torch.equal(bits(y4), bits(y64[:4])), "M=4 rows (lx_gemv_w) differ from M=64 rows (lx_gemm_w)"
    assert torch.equal(bits(y1), bits(y64[:1])), "the M=1 row (lx_gemv_w) differs from the M=64 row (lx_gemm_w)"
    # Against the oracle (f32 sums of the same products in another order): relative L2 of 1e-2 is the path's bar, the
    # observed error is near 1e-6.
    want = ops.gemv_w(oracle, x[:4].contiguous(), w.to("cpu"))
    for got in (y4, y64[:4]):
        err = rel_l2(got.cpu(), want)
        assert err <= 1e-2 and err <= 1e-4, err
    # and the default mode at the same rows
    for M in (1, 4):
        err = rel_l2(ops.gemv_w(hip, xd[:M].contiguous(), w).cpu(), want[:M])
        assert err <= 1e-2 and err <= 1e-4, err


# ---- C5: the FP8 decode layer at 32 streams ----------------------------------------------------------------------

C5_DENSE = [("qkv", 6144, 4096), ("o", 4096, 4096), ("in_proj", 16384, 4096), ("out_proj", 4096, 8192)]


@pytest.mark.parametrize("name,N,K", C5_DENSE)
def test_c5_dense_projection(hip, oracle, name, N, K):
    g = torch.Generator().manual_seed(5000 + N % 13)
    master = master_weight(N, K, g)
    x = torch.randn(64, K, generator=g).to(torch.bfloat16)
    w = quantize_with(hip, master.cuda(), W_FP8)
    xd = x.cuda()
    y32 = ops.gemm_w(hip, xd[:32].contiguous(), w, MATH_BF16)
    want = ops.gemm_w(oracle, x[:32].contiguous(), w.to("cpu"), MATH_BF16)
    err = rel_l2(y32.cpu(), want)
    assert err <= 1e-2 and err <= 1e-4, f"{name}: {err}"
    y1 = ops.gemm_w(hip, xd[:1].contiguous(), w, MATH_BF16)
    y64 = ops.gemm_w(hip, xd, w, MATH_BF16)
    assert torch.equal(bits(y1), bits(y32[:1])), f"{name}: the M=1 row differs from the M=32 row"
    assert torch.equal(bits(y64[:32]), bits(y32)), f"{name}: M=64 rows differ from M=32 rows"
    with invariant_mode():
        assert torch.equal(bits(ops.gemv_w(hip, xd[:8].contiguous(), w)), bits(y32[:8])), f"{name}: batch-invariant lx_gemv_w"
        assert torch.equal(bits(ops.gemm_w(hip, xd[:32].contiguous(), w, MATH_BF16)), bits(y32))


@pytest.fixture(scope="module")
def c5_stacks(hip):
    """E = 128 experts of gate/up 4096 -> 1536 and down 1536 -> 4096 in fp8, quantised on the device from bf16
    masters ~ N(0, 0.02) drawn on the device (2.4 GB of fp8; drawn once for the module)."""
    import ctypes

    E, L, I = 128, 4096, 1536
    gen = torch.Generator(device="cuda").manual_seed(5032)
    pair = []
    for n, k in ((2 * I, L), (L, I)):
        out = alloc_quantized(W_FP8, E * n, k, "cuda")
        rows_per = 16 * n
        for r0 in range(0, E * n, rows_per):  # masters in slabs of 16 experts: they are not kept
            m = (torch.randn(rows_per, k, generator=gen, device="cuda") * 0.02).to(torch.bfloat16)
            part = Weight(W_FP8, out.data[r0 : r0 + rows_per], out.scale[r0 : r0 + rows_per])
            s = part.lx()
            hip("quantize_weight", m, ctypes.pointer(s), ctypes.c_int64(rows_per), k)
        pair.append(Weight(W_FP8, out.data.view(E, n, k), out.scale.view(E, n)))
    return pair


def test_c5_routed_experts(hip, oracle, c5_stacks):
    E, L, I, top_k, T = 128, 4096, 1536, 8, 32
    gu, dn = c5_stacks
    g = torch.Generator().manual_seed(5033)
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    ids, weights, _, _ = ops.route(hip, logits.cuda(), None, top_k)
    ids_o, weights_o, _, _ = ops.route(oracle, logits, None, top_k)
    assert torch.equal(ids.cpu(), ids_o)
    out = ops.experts_grouped(hip, latent.cuda(), ids, weights, gu, dn, I, E, top_k)
    want = ops.experts_grouped(oracle, latent, ids_o, weights_o, gu.to("cpu"), dn.to("cpu"), I, E, top_k)
    err = rel_l2(out.cpu(), want)
    assert err <= 1e-2 and err <= 2e-3, err
    # a token's bits do not depend on the batch, nor on the entry point's kernels for few tokens being others
    one = ops.experts_grouped(hip, latent[5:6].contiguous().cuda(), ids[5:6].contiguous(), weights[5:6].contiguous(), gu, dn, I, E, top_k)
    assert torch.equal(bits(one[0]), bits(out[5]))
    # the decode entry point at the same shape (8 tokens), against the same oracle rows
    dec = ops.experts_decode(hip, latent[:8].contiguous().cuda(), ids[:8].contiguous(), weights[:8].contiguous(), gu, dn, I, top_k)
    err = rel_l2(dec.cpu(), want[:8])
    assert err <= 1e-2 and err <= 2e-3, err


# ---- lx_moe_experts_decode_bf16 ----------------------------------------------------------------------------------


@pytest.mark.parametrize("T", [1, 3, 8])
def test_decode_bf16_entry_equals_the_decode_experts_on_bf16_stacks(hip, oracle, T):
    # engine/cuda/kernels.h:606-610: the bf16-stack form of lx_moe_experts_decode, bit-identical to it.
    E, L, I, top_k = 16, 1024, 512, 4
    g = torch.Generator().manual_seed(60 + T)
    gate_up = (torch.randn(E, 2 * I, L, generator=g) / L**0.5).to(torch.bfloat16)
    down = (torch.randn(E, L, I, generator=g) / I**0.5).to(torch.bfloat16)
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16)
    ids = torch.rand(T, E, generator=g).argsort(-1)[:, :top_k].to(torch.int32).contiguous()
    weights = torch.softmax(torch.randn(T, top_k, generator=g), -1).contiguous()

    def run(lib, dev):
        n = int(lib.size("moe_bf16x_workspace_bytes", T, I, top_k))
        assert n >= 2 * T * top_k * I
        ws = torch.full((n,), 0xFF, dtype=torch.uint8, device=dev)
        out = torch.full((T, L), float("nan"), device=dev)
        lib("moe_experts_decode_bf16", latent.to(dev), ids.to(dev), weights.to(dev), gate_up.to(dev), down.to(dev), out, ws, T, L, I, top_k)
        return out

    got = run(hip, "cuda")
    same = ops.experts_decode(hip, latent.cuda(), ids.cuda(), weights.cuda(), Weight(0, gate_up).to("cuda"), Weight(0, down).to("cuda"), I, top_k)
    assert torch.equal(bits(got), bits(same)), "lx_moe_experts_decode_bf16 differs from lx_moe_experts_decode on the same bf16 stacks"
    want = run(oracle, "cpu")
    err = rel_l2(got.cpu(), want)
    assert err <= 1e-2 and err <= 2e-3, err
    want64 = ops.experts_reference(latent, ids, weights, gate_up.double(), down.double())
    assert rel_l2(got.cpu(), want64) <= 2e-3


# ---- routing with masked experts -------------------------------------------------------------------------------


@pytest.mark.parametrize("E", [64, 200, 512, 2048])
def test_route_with_masked_experts(hip, oracle, E):
    # All but three logits are -inf (masked experts): the picks are the three finite ones, then the masked experts
    # from the lowest index up, every id once (engine/cpu/moe.cpp:367-381).
    top_k, T = 8, 5
    g = torch.Generator().manual_seed(E)
    logits = torch.full((T, E), float("-inf"))
    for t in range(T):
        keep = torch.randperm(E, generator=g)[:3]
        logits[t, keep] = torch.randn(3, generator=g)
    logits[T - 1] = float("-inf")
    logits[T - 1, E - 1] = 0.5  # one finite logit, at the end
    ids, weights, _, _ = ops.route(hip, logits.cuda(), None, top_k)
    ids_o, weights_o, _, _ = ops.route(oracle, logits, None, top_k)
    assert torch.equal(ids.cpu(), ids_o), (ids.cpu().tolist(), ids_o.tolist())
    for t in range(T):
        assert len(set(ids[t].tolist())) == top_k, f"token {t}: an expert was picked twice: {ids[t].tolist()}"
    assert torch.equal(torch.isnan(weights.cpu()), torch.isnan(weights_o))
    ok = ~torch.isnan(weights_o)
    assert (weights.cpu()[ok] - weights_o[ok]).abs().max().item() <= 1e-5


# ---- the two e4m3 codes no quantiser emits ------------------------------------------------------------------------


def test_fp8_codes_0x7f_and_0xff(hip):
    # e4m3fn calls 0x7f / 0xff NaN. The quantisers saturate at +-448 (0x7e / 0xfe) and never emit them
    # (tests/test_gpu_quant.py). lx_dequantize_weight reads them as the reference does (+-480,
    # engine/cpu/quant.cpp:12-18); the product kernels convert e4m3 in hardware, where they are NaN: a row that holds
    # one gives NaN, every other row is untouched.
    N, K = 32, 1024
    w = random_weight(W_FP8, N, K, 3)
    w.data[:, :] = w.data.clamp(max=0x7E) & 0x7F  # positive finite codes everywhere
    w.data[5, 17] = 0x7F
    w.data[9, 900] = 0xFF
    wd = w.to("cuda")
    x = torch.randn(20, K, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).cuda()
    deq = ops.dequantize(hip, wd, N, K).float().cpu()
    assert deq[5, 17].item() == pytest.approx(480.0 * w.scale[5].item(), rel=2**-8)
    assert deq[9, 900].item() == pytest.approx(-480.0 * w.scale[9].item(), rel=2**-8)
    clean = torch.ones(N, dtype=torch.bool)
    clean[5] = clean[9] = False
    for y in (ops.gemv_w(hip, x[:1].contiguous(), wd), ops.gemv_w(hip, x[:8].contiguous(), wd), ops.gemm_w(hip, x, wd, MATH_BF16)):
        y = y.cpu()
        assert bool(torch.isnan(y[:, ~clean]).all()), "a row holding an e4m3 NaN code gives NaN"
        assert bool(torch.isfinite(y[:, clean]).all())
