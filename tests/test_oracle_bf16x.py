"""Pins the oracle's restatement of LX_W_BF16X (the codec, lx_gemv_bf16x, lx_moe_experts_bf16x): round trips over every
kind of exponent pattern read back by a numpy reading of the layout that shares no code with it, sizes by closed form,
a record built by hand, and byte for byte / bit for bit against the reference's CPU backend where it was built."""

import ctypes

import numpy as np
import pytest
import torch

import checks
import ops
from dromos_amd.abi import W_BF16, W_BF16X
from dromos_amd.formats import Weight

SHAPES = [(5, 512), (3, 1024), (4, 2048), (2, 4096), (7, 130), (3, 1), (2, 127), (2, 129), (1, 6144)]


@pytest.mark.parametrize("kind", ["trained", "wild", "spill"])
@pytest.mark.parametrize("rows,K", SHAPES)
def test_round_trip(oracle, rows, K, kind):
    checks.bf16x_round_trip(oracle, rows, K, rows * K, kind)


def test_geometry_known_answers(oracle):
    # The reference states the slot counts of its model's row lengths (engine/cuda/bf16x.cuh:27): 3 at K = 512, 2 at
    # 1024, 4 at 2048 and 4096.
    for K, slots in [(512, 3), (1024, 2), (2048, 4), (4096, 4)]:
        spans = K // 128
        rb = ops.bf16x_row_bytes(oracle, K)
        assert (rb - 192 * spans - spans) // 4 == slots and rb % 8 == 0
    assert ops.bf16x_row_bytes(oracle, 0) == -1 and ops.bf16x_row_bytes(oracle, 1 << 23) == -1
    assert ops.bf16x_row_bytes(oracle, (1 << 23) - 1) > 0


def test_a_record_built_by_hand(oracle):
    # K = 10: one span, header = roundup(4 * 2 + 1, 8) = 16 bytes, 3 slots, the top at byte 12.
    vals = torch.tensor([1.0, -2.0, 0.5, 3.0, 2.0**-20, 1.5, -0.75, 0.0, 2.0, 1.0], dtype=torch.bfloat16)
    enc = ops.bf16x_encode(oracle, vals.view(1, 10)).numpy()
    assert enc.size == 16 + 192
    bits = vals.view(torch.int16).numpy().astype(np.uint16)
    exps = (bits >> 7) & 0xFF
    top = int(exps.max())  # 128: the exponent of 2.0 and 3.0
    assert top == 128
    words = enc[:12].view(np.uint32)
    # 2^-20 (k = 4, exponent 107) and 0.0 (k = 7, exponent 0) lie more than 15 below the top: two exception words.
    assert list(words) == [(4 << 8) | 107, (7 << 8) | 0, 0xFFFFFFFF]
    assert enc[12] == top and list(enc[13:16]) == [0, 0, 0]
    want_sm = ((bits >> 8) & 0x80) | (bits & 0x7F)
    assert list(enc[16:26]) == list(want_sm) and not enc[26:16 + 128].any()
    codes = [top - int(e) for e in exps]
    codes[4] = codes[7] = 0
    nib = enc[16 + 128:16 + 192]
    # Word 0 holds values 0..7: byte b = value b (low) | value 4 + b (high); word 1 byte b = value 8 + b (low).
    assert list(nib[:4]) == [codes[b] | codes[4 + b] << 4 for b in range(4)]
    assert list(nib[4:8]) == [codes[8], codes[9], 0, 0] and not nib[8:].any()


def test_validation(oracle):
    w = checks.bf16x_weights(2, 256, 1)
    n = ops.bf16x_bytes(oracle, w)
    out = torch.zeros(n + 8, dtype=torch.uint8)
    st = lambda *a: oracle.status("bf16x_encode", *a)
    assert st(w, ctypes.c_int64(2), 256, out, ctypes.c_int64(n - 1)) == 1  # too small
    assert st(w, ctypes.c_int64(2), 256, out[1:], ctypes.c_int64(n)) == 1  # misaligned
    assert st(w, ctypes.c_int64(2), 0, out, ctypes.c_int64(n)) == 1
    assert st(w, ctypes.c_int64(0), 256, None, ctypes.c_int64(0)) == 0
    fn = oracle.lib.lx_bf16x_bytes
    fn.restype = ctypes.c_int64
    assert fn(None, ctypes.c_int64(2), 256, None) == -1
    assert fn(ctypes.c_void_p(w.data_ptr()), ctypes.c_int64(0), 256, None) == -1


@pytest.mark.parametrize("kind", ["trained", "wild", "spill"])
def test_bytes_equal_the_reference(oracle, ref, kind):
    for rows, K in SHAPES:
        w = checks.bf16x_weights(rows, K, K + rows, kind)
        a, b = ops.bf16x_encode(oracle, w), ops.bf16x_encode(ref, w)
        assert torch.equal(a, b)
        assert torch.equal(ops.bf16x_decode(ref, a, rows, K).view(torch.int16), w.view(torch.int16))


@pytest.mark.parametrize("M,N,K,kind", [(1, 48, 1024, "trained"), (8, 33, 2048, "spill"), (3, 17, 130, "trained"), (2, 5, 7, "spill")])
def test_gemv_is_the_bf16_gemv(oracle, ref, M, N, K, kind):
    g = torch.Generator().manual_seed(N)
    w = checks.bf16x_weights(N, K, N * K, kind)
    enc = ops.bf16x_encode(oracle, w)
    for x in (torch.randn(M, K, generator=g), torch.randn(M, K, generator=g).to(torch.bfloat16)):
        bias = torch.randn(N, generator=g)
        y0 = torch.randn(M, N, generator=g)
        got = ops.gemv_bf16x(oracle, x, enc, N, bias=bias, y=y0.clone(), alpha=0.5, beta=2.0)
        plain = ops.gemv_bf16x(oracle, x, w, N, bias=bias, y=y0.clone(), alpha=0.5, beta=2.0, entry="gemv_decode_bf16")
        assert torch.equal(got.view(torch.int32), plain.view(torch.int32))
        via_w = ops.gemv_w(oracle, x, Weight(W_BF16X, enc), bias=bias, y=y0.clone(), alpha=0.5, beta=2.0, N=N, K=K)
        assert torch.equal(via_w.view(torch.int32), plain.view(torch.int32))
        ref.lib.lx_set_arch_override(1)
        try:
            theirs = ops.gemv_bf16x(ref, x, enc, N, bias=bias, y=y0.clone(), alpha=0.5, beta=2.0)
        finally:
            ref.lib.lx_set_arch_override(0)
        assert torch.equal(got.view(torch.int32), theirs.view(torch.int32))
    assert ops.gemv_bf16x(oracle, x, enc[1:], N, status=True) == 1  # not 8-byte aligned
    assert ops.gemv_bf16x(oracle, torch.zeros(9, K), enc, N, status=True) == 1


@pytest.mark.parametrize("T,E,L,I,top_k", [(1, 8, 256, 128, 4), (5, 6, 130, 72, 3), (11, 4, 512, 256, 2)])
def test_experts_are_the_bf16_experts(oracle, ref, T, E, L, I, top_k):
    gu = checks.bf16x_weights(E * 2 * I, L, 1, "spill").view(E, 2 * I, L)
    dn = checks.bf16x_weights(E * L, I, 2, "trained").view(E, L, I)
    latent, ids, weights = checks.make_routing(T, E, L, top_k, T)
    gu_x, dn_x = ops.bf16x_encode(oracle, gu), ops.bf16x_encode(oracle, dn)
    got = ops.experts_bf16x(oracle, latent, ids, weights, gu_x, dn_x, I, top_k)
    plain = ops.experts_bf16x(oracle, latent, ids, weights, gu, dn, I, top_k, entry="moe_experts_decode_bf16")
    assert torch.equal(got.view(torch.int32), plain.view(torch.int32))
    want = ops.experts_reference(latent, ids, weights, gu.double(), dn.double())
    checks.experts_close(got, want)
    ref.lib.lx_set_arch_override(1)
    try:
        theirs = ops.experts_bf16x(ref, latent, ids, weights, gu_x, dn_x, I, top_k)
    finally:
        ref.lib.lx_set_arch_override(0)
    assert torch.equal(got.view(torch.int32), theirs.view(torch.int32))
    if T <= 8:
        via = ops.experts_decode(oracle, latent, ids, weights, Weight(W_BF16X, gu_x), Weight(W_BF16X, dn_x), I, top_k)
        assert torch.equal(via.view(torch.int32), got.view(torch.int32))
        assert ops.experts_decode(oracle, latent, ids, weights, Weight(W_BF16X, gu_x), Weight(W_BF16, dn), I, top_k, status=True) == 801
    assert ops.experts_bf16x(oracle, latent, ids.repeat(1, 5)[:, :9].contiguous(), weights.repeat(1, 5)[:, :9].contiguous(), gu_x, dn_x, I, 9, status=True) == 1
