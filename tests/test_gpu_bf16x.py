"""GPU parity for LX_W_BF16X: the encoder writes the oracle's bytes, every round trip gives back every bit, and the
products on encoded weights equal the bf16 products on the original weights bit for bit (lx_gemv_bf16x against
lx_gemv_decode_bf16, lx_moe_experts_bf16x against lx_moe_experts_decode_bf16), through the C ABI."""

import ctypes

import pytest
import torch

import checks
import ops
from conftest import rel_l2
from dromos_amd.abi import W_BF16, W_BF16X
from dromos_amd.formats import Weight

pytestmark = pytest.mark.gpu

SHAPES = [(5, 512), (3, 1024), (4, 2048), (2, 4096), (7, 130), (3, 1), (2, 127), (2, 129), (1, 6144), (300, 1536), (1, 70000)]


def bits(t):
    return t.view(torch.int32)


@pytest.mark.parametrize("kind", ["trained", "wild", "spill"])
@pytest.mark.parametrize("rows,K", SHAPES)
def test_round_trip_and_the_oracles_bytes(hip, oracle, rows, K, kind):
    w, enc, counts = checks.bf16x_round_trip(hip, rows, K, rows * K, kind)
    theirs = ops.bf16x_encode(oracle, w.cpu())
    assert torch.equal(enc.cpu(), theirs)
    if kind == "spill":
        assert int(counts.max()) > checks.bf16x_geometry(K)[2] or K < 16


def test_codec_arguments(hip):
    w = checks.bf16x_weights(2, 256, 1).cuda()
    n = ops.bf16x_bytes(hip, w)
    out = torch.zeros(n + 8, dtype=torch.uint8, device="cuda")
    st = lambda *a: hip.status("bf16x_encode", *a)
    assert st(w, ctypes.c_int64(2), 256, out, ctypes.c_int64(n - 1)) == 1
    assert st(w, ctypes.c_int64(2), 256, out[1:], ctypes.c_int64(n)) == 1
    assert st(w, ctypes.c_int64(2), 0, out, ctypes.c_int64(n)) == 1
    assert st(w, ctypes.c_int64(0), 256, None, ctypes.c_int64(0)) == 0
    fn = hip.lib.lx_bf16x_bytes
    fn.restype = ctypes.c_int64
    assert fn(None, ctypes.c_int64(2), 256, None) == -1
    assert ops.bf16x_row_bytes(hip, 1 << 23) == -1


# Streamed shapes (K a multiple of 8) of every batch depth and split, and shapes only the element-wise kernel takes.
GEMV_SHAPES = [(4096, 4096), (14336, 4096), (4096, 14336), (256, 2048), (96, 512), (40, 1024), (1000, 6144), (33, 8), (64, 24576),
               (17, 130), (5, 7), (12, 1029)]


@pytest.mark.parametrize("kind", ["trained", "spill"])
@pytest.mark.parametrize("N,K", GEMV_SHAPES)
def test_gemv_equals_the_bf16_gemv_bit_for_bit(hip, oracle, N, K, kind):
    g = torch.Generator().manual_seed(N + K)
    w = checks.bf16x_weights(N, K, N ^ K, kind).cuda()
    enc = ops.bf16x_encode(hip, w)
    bias = torch.randn(N, generator=g).cuda()
    for M in (1, 2, 3, 5, 8):
        for dtype in (torch.bfloat16, torch.float32):
            x = torch.randn(M, K, generator=g).to(dtype).cuda()
            got = ops.gemv_bf16x(hip, x, enc, N, bias=bias, alpha=0.75)
            plain = ops.gemv_bf16x(hip, x, w, N, bias=bias, alpha=0.75, entry="gemv_decode_bf16")
            assert torch.equal(bits(got), bits(plain)), (M, dtype)
    # through lx_gemv_w, and against the oracle on the same encoding
    via_w = ops.gemv_w(hip, x, Weight(W_BF16X, enc), bias=bias, alpha=0.75, N=N, K=K)
    assert torch.equal(bits(via_w), bits(got))
    if N * K <= 1 << 24:
        want = ops.gemv_bf16x(oracle, x.cpu(), enc.cpu(), N, bias=bias.cpu(), alpha=0.75)
        assert rel_l2(got, want) <= 1e-5


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_gemv_follows_the_bf16_kernels_forced_split(hip, variant):
    # A K split forced for the bf16 GEMV is the encoded GEMV's too: the two keep equal bits under any variant table.
    lib = hip.lib
    g = torch.Generator().manual_seed(variant)
    try:
        for M, N, K in [(1, 300, 2048), (4, 512, 4096), (8, 96, 1024)]:
            w = checks.bf16x_weights(N, K, N + K, "trained").cuda()
            enc = ops.bf16x_encode(hip, w)
            x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
            lib.lx_tune_clear()
            default = ops.gemv_bf16x(hip, x, w, N, entry="gemv_decode_bf16")
            assert lib.lx_tune_force(b"gemv_w_bf16", M, N, K, variant) == 0
            got = ops.gemv_bf16x(hip, x, enc, N)
            plain = ops.gemv_bf16x(hip, x, w, N, entry="gemv_decode_bf16")
            assert torch.equal(bits(got), bits(plain)), (M, N, K)
            assert rel_l2(plain, default) <= 1e-5
    finally:
        lib.lx_tune_clear()


def test_gemv_arguments(hip):
    w = checks.bf16x_weights(16, 256, 3).cuda()
    enc = ops.bf16x_encode(hip, w)
    x = torch.zeros(2, 256, device="cuda")
    assert ops.gemv_bf16x(hip, x, enc[1:], 16, status=True) == 1  # not 8-byte aligned
    assert ops.gemv_bf16x(hip, torch.zeros(9, 256, device="cuda"), enc, 16, status=True) == 1
    y = torch.full((2, 16), 7.0, device="cuda")
    assert hip.status("gemv_bf16x", x, 0, 256, enc, None, 0, y, 0, 16, 0, 16, 256, 1.0, 0.0) == 0
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())


@pytest.mark.parametrize("T,E,L,I,top_k,kinds", [
    (1, 16, 1024, 512, 4, ("trained", "trained")),
    (1, 64, 2048, 1024, 8, ("spill", "trained")),
    (3, 16, 1024, 512, 4, ("trained", "spill")),
    (8, 8, 2048, 768, 8, ("trained", "trained")),
    (11, 6, 512, 256, 2, ("spill", "spill")),
    (5, 6, 130, 72, 3, ("trained", "spill")),  # rows the streaming kernels cannot take
])
def test_experts_equal_the_bf16_experts_bit_for_bit(hip, oracle, T, E, L, I, top_k, kinds):
    gu = checks.bf16x_weights(E * 2 * I, L, 1, kinds[0]).view(E, 2 * I, L).cuda()
    dn = checks.bf16x_weights(E * L, I, 2, kinds[1]).view(E, L, I).cuda()
    latent, ids, weights = (t.cuda() for t in checks.make_routing(T, E, L, top_k, T))
    gu_x, dn_x = ops.bf16x_encode(hip, gu), ops.bf16x_encode(hip, dn)
    got = ops.experts_bf16x(hip, latent, ids, weights, gu_x, dn_x, I, top_k)
    plain = ops.experts_bf16x(hip, latent, ids, weights, gu, dn, I, top_k, entry="moe_experts_decode_bf16")
    assert torch.equal(bits(got), bits(plain))
    want = ops.experts_bf16x(oracle, latent.cpu(), ids.cpu(), weights.cpu(), gu_x.cpu(), dn_x.cpu(), I, top_k)
    err = rel_l2(got, want)
    assert err <= 2e-3, err
    if T <= 8:
        # engine/cuda/kernels.h:598-610: a decode step's lx_moe_experts on the bf16 stacks gives the same bits
        legacy = ops.experts_bf16(hip, latent, ids, weights, gu, dn, I, top_k)
        assert torch.equal(bits(legacy), bits(got))
        via = ops.experts_decode(hip, latent, ids, weights, Weight(W_BF16X, gu_x), Weight(W_BF16X, dn_x), I, top_k)
        assert torch.equal(bits(via), bits(got))
        assert ops.experts_decode(hip, latent, ids, weights, Weight(W_BF16X, gu_x), Weight(W_BF16, dn), I, top_k, status=True) == 801


def test_experts_arguments(hip):
    E, L, I = 4, 256, 128
    gu = ops.bf16x_encode(hip, checks.bf16x_weights(E * 2 * I, L, 1).cuda())
    dn = ops.bf16x_encode(hip, checks.bf16x_weights(E * L, I, 2).cuda())
    latent, ids, weights = (t.cuda() for t in checks.make_routing(2, E, L, 2, 0))
    assert ops.experts_bf16x(hip, latent, ids, weights, gu[1:], dn, I, 2, status=True) == 1
    wide_ids = torch.zeros(2, 9, dtype=torch.int32, device="cuda")
    wide_w = torch.zeros(2, 9, device="cuda")
    assert ops.experts_bf16x(hip, latent, wide_ids, wide_w, gu, dn, I, 9, status=True) == 1
