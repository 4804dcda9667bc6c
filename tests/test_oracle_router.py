"""Pins the oracle's restatements of the calls either side of the experts (lx_spec_gemv_f32, lx_router_route,
lx_moe_summary, lx_moe_summary_history) and of the legacy product forms (lx_moe_experts_w8, lx_gemm_bf16): against
float64 closed forms, and bit for bit against the reference's CPU backend at its generic level where it was built."""

import pytest
import torch

import checks
import ops
from conftest import close, rel_l2
from dromos_amd.abi import W_INT8
from dromos_amd.formats import random_stack


def router_inputs(M, E, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    w = torch.randn(E, K, generator=g) / K**0.5
    bias = torch.randn(E, generator=g) * 0.1
    sel = torch.randn(E, generator=g) * 0.5
    return x, w, bias, sel


@pytest.mark.parametrize("M,N,K", [(1, 64, 2048), (8, 128, 1024), (3, 37, 130), (5, 1, 7)])
def test_spec_gemv_f32(oracle, M, N, K):
    x, w, bias, _ = router_inputs(M, N, K, M + N)
    y = ops.spec_gemv_f32(oracle, x, w, bias)
    want = x.double() @ w.double().T + bias.double()
    close(y, want, atol=2e-6 * want.abs().max().item() * K**0.5)
    assert ops.spec_gemv_f32(oracle, torch.zeros(9, K), w, bias, status=True) == 1  # M > 8
    assert ops.spec_gemv_f32(oracle, x, w, bias, M=0, status=True) == 0


def test_spec_gemv_f32_equals_the_reference_generic_level(oracle, ref):
    ref.lib.lx_set_arch_override(1)
    try:
        for M, N, K in [(1, 64, 2048), (8, 128, 1024), (3, 37, 130)]:
            x, w, bias, _ = router_inputs(M, N, K, K)
            a, b = ops.spec_gemv_f32(oracle, x, w, bias), ops.spec_gemv_f32(ref, x, w, bias)
            assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    finally:
        ref.lib.lx_set_arch_override(0)


def test_router_route_is_the_two_calls(oracle):
    x, w, bias, sel = router_inputs(6, 64, 512, 3)
    logits, ids, weights, entropy, confidence = ops.router_route(oracle, x, w, bias, sel, 8)
    want_logits = ops.spec_gemv_f32(oracle, x, w, bias)
    assert torch.equal(logits.view(torch.int32), want_logits.view(torch.int32))
    want = ops.route(oracle, want_logits, sel, 8)
    for u, v in zip((ids, weights, entropy, confidence), want):
        assert torch.equal(u, v)
    assert ops.router_route(oracle, torch.zeros(9, 512), w, bias, sel, 8, status=True) == 1


@pytest.mark.parametrize("T,E,R,top_k", [(1, 64, 128, 8), (7, 37, 50, 3), (64, 128, 256, 4)])
def test_summary(oracle, ref, T, E, R, top_k):
    g = torch.Generator().manual_seed(T + R)
    emb = torch.randn(E, R, generator=g).to(torch.bfloat16)
    _, ids, weights = checks.make_routing(T, E, 16, top_k, T)
    got = ops.moe_summary(oracle, ids, weights, emb)
    want = (weights.double().unsqueeze(-1) * emb.double()[ids.long()]).sum(1)
    close(got, want, atol=1e-6 * max(want.abs().max().item(), 1.0))
    hist0 = torch.randn(T, R, generator=g)
    h = hist0.clone()
    got_h = ops.moe_summary(oracle, ids, weights, emb, history=h, a=0.9, b=0.1)
    assert torch.equal(got_h, got)
    close(h, 0.9 * hist0.double() + 0.1 * want, atol=1e-6 * max(want.abs().max().item(), 1.0))
    # the reference's own backend: the same multiplies and adds in the same order
    assert torch.equal(ops.moe_summary(ref, ids, weights, emb).view(torch.int32), got.view(torch.int32))
    h2 = hist0.clone()
    ops.moe_summary(ref, ids, weights, emb, history=h2, a=0.9, b=0.1)
    assert torch.equal(h2.view(torch.int32), h.view(torch.int32))


@pytest.mark.parametrize("T", [1, 5, 19])
def test_experts_w8(oracle, ref, T):
    E, L, I, top_k = 12, 256, 128, 4
    gu, dn = random_stack(W_INT8, E, 2 * I, L, 81), random_stack(W_INT8, E, L, I, 82)
    latent, ids, weights = checks.make_routing(T, E, L, top_k, 83 + T)
    out = ops.experts_w8(oracle, latent, ids, weights, gu, dn, I, top_k)
    checks.experts_close(out, ops.experts_reference(latent, ids, weights, gu.dense(), dn.dense()))
    ref.lib.lx_set_arch_override(1)
    try:
        assert torch.equal(ops.experts_w8(ref, latent, ids, weights, gu, dn, I, top_k).view(torch.int32), out.view(torch.int32))
    finally:
        ref.lib.lx_set_arch_override(0)
    assert int(oracle.size("moe_workspace_bytes", T, I, top_k)) == int(ref.size("moe_workspace_bytes", T, I, top_k))


@pytest.mark.parametrize("M", [1, 8, 33])
def test_gemm_bf16(oracle, ref, M):
    N, K = 96, 512
    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    y0 = torch.randn(M, N, generator=g)
    got = ops.gemm_bf16(oracle, x, w, bias, y=y0.clone(), alpha=0.5, beta=2.0)
    want = 0.5 * (x.double() @ w.double().T + bias.double()) + 2.0 * y0.double()
    assert rel_l2(got, want) < 1e-5
    ref.lib.lx_set_arch_override(1)
    try:
        there = ops.gemm_bf16(ref, x, w, bias, y=y0.clone(), alpha=0.5, beta=2.0)
    finally:
        ref.lib.lx_set_arch_override(0)
    # M <= 8: the same f32 dot, bit for bit; more rows may take the reference's bf16 dot instructions
    if M <= 8:
        assert torch.equal(there.view(torch.int32), got.view(torch.int32))
    else:
        assert rel_l2(there, got) < 1e-5
