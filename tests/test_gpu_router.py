"""GPU parity: the calls either side of the experts in a decode layer (lx_spec_gemv_f32, lx_router_route,
lx_moe_summary, lx_moe_summary_history) and the legacy product forms (lx_moe_experts_w8, lx_gemm_bf16), through the C
ABI against the CPU oracle on the same inputs and float64 closed forms."""

import pytest
import torch

import checks
import ops
from conftest import close, rel_l2
from dromos_amd.abi import MATH_BF16, W_BF16, W_INT8
from dromos_amd.formats import Weight, random_stack

pytestmark = pytest.mark.gpu


def router_inputs(M, E, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    w = torch.randn(E, K, generator=g) / K**0.5
    bias = torch.randn(E, generator=g) * 0.1
    sel = torch.randn(E, generator=g) * 0.5
    return x, w, bias, sel


@pytest.mark.parametrize("M,N,K", [(1, 64, 2048), (8, 128, 2048), (8, 128, 4096), (3, 37, 130), (5, 1, 7), (2, 1024, 2048)])
def test_spec_gemv_f32(hip, oracle, M, N, K):
    x, w, bias, _ = router_inputs(M, N, K, M + N)
    y = ops.spec_gemv_f32(hip, x.cuda(), w.cuda(), bias.cuda())
    want = ops.spec_gemv_f32(oracle, x, w, bias)
    assert rel_l2(y, want) <= 1e-5  # f32 sums in another order
    close(y, x.double() @ w.double().T + bias.double(), atol=2e-6 * K**0.5 * max(want.abs().max().item(), 1.0))
    no_bias = ops.spec_gemv_f32(hip, x.cuda(), w.cuda(), None)
    assert rel_l2(no_bias, x.double() @ w.double().T) <= 1e-5
    # a row's bits do not depend on the rows beside it
    for m in range(M):
        alone = ops.spec_gemv_f32(hip, x[m : m + 1].contiguous().cuda(), w.cuda(), bias.cuda())
        assert torch.equal(alone[0].view(torch.int32), y[m].view(torch.int32)), f"row {m}"


@pytest.mark.parametrize("pad", [0, 3])
@pytest.mark.parametrize("M,N,K", [(1, 64, 2048), (9, 128, 2048), (33, 64, 2304), (70, 37, 130), (64, 1, 2048)])
def test_gemm_f32(hip, oracle, M, N, K, pad):
    # engine/cuda/kernels.h:72-76 (the reference tests it against float64 with rtol 1e-5, tests/kernels/test_gemm.py:67-80).
    x, w, bias, _ = router_inputs(M, N, K, M + N + pad)
    y = ops.gemm_f32(hip, x.cuda(), w.cuda(), bias.cuda(), pad=pad)
    want = ops.gemm_f32(oracle, x, w, bias, pad=pad)
    assert rel_l2(y[:, :N], want[:, :N]) <= 1e-5  # f32 sums in another order
    close(y[:, :N], x.double() @ w.double().T + bias.double(), atol=2e-6 * K**0.5 * max(want[:, :N].abs().max().item(), 1.0))
    assert torch.isnan(y[:, N:]).all(), "wrote past the N columns of y"
    # a row's bits are those of the decode-sized call, whatever the batch
    for m in (0, M // 2, M - 1):
        alone = ops.spec_gemv_f32(hip, x[m : m + 1].contiguous().cuda(), w.cuda(), bias.cuda())
        assert torch.equal(alone[0].view(torch.int32), y[m, :N].contiguous().view(torch.int32)), f"row {m}"
    no_bias = ops.gemm_f32(hip, x.cuda(), w.cuda(), None)
    assert rel_l2(no_bias, x.double() @ w.double().T) <= 1e-5


def test_gemm_f32_arguments(hip):
    w = torch.zeros(16, 64, device="cuda")
    assert ops.gemm_f32(hip, torch.zeros(0, 64, device="cuda"), w, None, status=True) == 0
    y = torch.zeros(4, 16, device="cuda")
    assert hip.status("gemm_f32", torch.zeros(4, 64, device="cuda"), 32, w, None, y, 16, 4, 16, 64) == 1  # ld_x < K
    assert hip.status("gemm_f32", torch.zeros(4, 64, device="cuda"), 64, w, None, y, 8, 4, 16, 64) == 1  # ld_y < N
    assert hip.status("gemm_f32", None, 64, w, None, y, 16, 4, 16, 64) == 1


def test_spec_gemv_f32_arguments(hip):
    w = torch.zeros(16, 64, device="cuda")
    assert ops.spec_gemv_f32(hip, torch.zeros(9, 64, device="cuda"), w, None, status=True) == 1
    assert ops.spec_gemv_f32(hip, torch.zeros(2, 64, device="cuda"), w, None, M=0, status=True) == 0


@pytest.mark.parametrize("M,E,K,top_k", [(1, 64, 2048, 8), (8, 128, 2048, 8), (5, 37, 130, 3), (3, 1024, 512, 32)])
def test_router_route(hip, oracle, M, E, K, top_k):
    x, w, bias, sel = router_inputs(M, E, K, E + K)
    xd, wd, bd, sd = x.cuda(), w.cuda(), bias.cuda(), sel.cuda()
    logits, ids, weights, entropy, confidence = ops.router_route(hip, xd, wd, bd, sd, top_k)
    # bit-identical to the two calls
    two = ops.spec_gemv_f32(hip, xd, wd, bd)
    assert torch.equal(logits.view(torch.int32), two.view(torch.int32))
    for u, v in zip((ids, weights, entropy, confidence), ops.route(hip, two, sd, top_k)):
        assert torch.equal(u, v)
    # and the routing is the oracle's on these logits
    want = ops.route(oracle, logits.cpu(), sel, top_k)
    assert torch.equal(ids.cpu(), want[0])
    for u, v in zip((weights, entropy, confidence), want[1:]):
        close(u, v, atol=1e-5)
    assert rel_l2(logits, ops.spec_gemv_f32(oracle, x, w, bias)) <= 1e-5


def test_router_route_arguments(hip):
    x, w, bias, sel = (t.cuda() for t in router_inputs(2, 16, 64, 1))
    assert ops.router_route(hip, torch.zeros(9, 64, device="cuda"), w, bias, sel, 4, status=True) == 1
    assert ops.router_route(hip, x, w, bias, sel, 17, status=True) == 1  # top_k > E
    assert ops.router_route(hip, x[:0], w, bias, sel, 4, status=True) == 0


@pytest.mark.parametrize("T,E,R,top_k", [(1, 64, 128, 8), (7, 37, 50, 3), (64, 128, 256, 4), (300, 64, 1024, 8)])
def test_summary(hip, oracle, T, E, R, top_k):
    g = torch.Generator().manual_seed(T + R)
    emb = torch.randn(E, R, generator=g).to(torch.bfloat16)
    _, ids, weights = checks.make_routing(T, E, 16, top_k, T)
    got = ops.moe_summary(hip, ids.cuda(), weights.cuda(), emb.cuda())
    want = ops.moe_summary(oracle, ids, weights, emb)
    assert torch.equal(got.cpu().view(torch.int32), want.view(torch.int32))  # the same multiplies and adds in the same order
    hist0 = torch.randn(T, R, generator=g)
    h, h_want = hist0.clone().cuda(), hist0.clone()
    got_h = ops.moe_summary(hip, ids.cuda(), weights.cuda(), emb.cuda(), history=h, a=0.9, b=0.1)
    ops.moe_summary(oracle, ids, weights, emb, history=h_want, a=0.9, b=0.1)
    assert torch.equal(got_h, got)
    assert torch.equal(h.cpu().view(torch.int32), h_want.view(torch.int32))


@pytest.mark.parametrize("T", [1, 8, 19])
def test_experts_w8(hip, oracle, T):
    E, L, I, top_k = 12, 1024, 512, 4
    gu, dn = random_stack(W_INT8, E, 2 * I, L, 81), random_stack(W_INT8, E, L, I, 82)
    latent, ids, weights = checks.make_routing(T, E, L, top_k, 83 + T)
    out = ops.experts_w8(hip, latent.cuda(), ids.cuda(), weights.cuda(), gu.to("cuda"), dn.to("cuda"), I, top_k)
    want = ops.experts_w8(oracle, latent, ids, weights, gu, dn, I, top_k)
    err = rel_l2(out, want)
    assert err <= 1e-2 and err <= 2e-3, err
    checks.experts_close(out, ops.experts_reference(latent, ids, weights, gu.dense(), dn.dense()))
    if T <= 8:  # the decode experts on the same int8 stacks: the same kernels, the same bits
        same = ops.experts_decode(hip, latent.cuda(), ids.cuda(), weights.cuda(), gu.to("cuda"), dn.to("cuda"), I, top_k)
        assert torch.equal(same.view(torch.int32), out.view(torch.int32))
    assert int(hip.size("moe_workspace_bytes", T, I, top_k)) >= int(oracle.size("moe_workspace_bytes", T, I, top_k))


@pytest.mark.parametrize("T", [1, 5, 19])
def test_experts_w8_more_than_eight_picks(hip, oracle, T):
    # engine/cpu/moe.cpp:460-476 takes any top_k.
    E, L, I, top_k = 16, 512, 256, 12
    gu, dn = random_stack(W_INT8, E, 2 * I, L, 91), random_stack(W_INT8, E, L, I, 92)
    latent, ids, weights = checks.make_routing(T, E, L, top_k, 93 + T)
    out = ops.experts_w8(hip, latent.cuda(), ids.cuda(), weights.cuda(), gu.to("cuda"), dn.to("cuda"), I, top_k)
    want = ops.experts_w8(oracle, latent, ids, weights, gu, dn, I, top_k)
    assert rel_l2(out, want) <= 2e-3
    checks.experts_close(out, ops.experts_reference(latent, ids, weights, gu.dense(), dn.dense()))


@pytest.mark.parametrize("M", [1, 8, 33, 64])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16(hip, oracle, M, y_dtype):
    N, K = 300, 1024
    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    y0 = torch.randn(M, N, generator=g).to(y_dtype)
    got = ops.gemm_bf16(hip, x.cuda(), w.cuda(), bias.cuda(), y=y0.clone().cuda(), alpha=0.5, beta=2.0)
    want = ops.gemm_bf16(oracle, x, w, bias, y=y0.clone(), alpha=0.5, beta=2.0)
    assert rel_l2(got, want) <= (4e-3 if y_dtype == torch.bfloat16 else 1e-5)
    # the same kernel as lx_gemm_w on a bf16 weight: the same bits
    same = ops.gemm_w(hip, x.cuda(), Weight(W_BF16, w).to("cuda"), MATH_BF16, bias=bias.cuda(), y=y0.clone().cuda(), alpha=0.5, beta=2.0)
    assert torch.equal(same.view(torch.int16 if y_dtype == torch.bfloat16 else torch.int32),
                       got.view(torch.int16 if y_dtype == torch.bfloat16 else torch.int32))
