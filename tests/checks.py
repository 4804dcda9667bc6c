"""Checks of a backend library against closed-form float64 statements of the ops, shared by the CPU tests
(run on the oracle, which pins it) and the GPU tests (run on the product). Shapes, edge cases and tolerances
follow the reference's kernel tests (tests/kernels/test_gemv_w.py, test_quant.py, test_moe.py,
test_moe_decode.py, test_moe_grouped.py of the reference)."""

import ctypes

import torch

import ops
from conftest import close, rel_l2
from dromos_amd.abi import FORMATS, W_BF16, W_FP8, W_INT8, W_NVFP4
from dromos_amd.formats import (Weight, alloc_quantized, quantize_reference, quantize_with, random_stack,
                                random_weight)

FMT_NAMES = list(FORMATS)


def dev(lx, t):
    return t.to(lx.device)


def check_product(got, want):
    """Half a bf16 ulp of the largest output for bf16 outputs, 2e-4 of it for f32 outputs
    (tests/kernels/test_gemv_w.py:64-68 of the reference), and the path's own 1e-2 relative L2 bound."""
    scale = want.abs().max().item()
    rel = 2.0**-8 if got.dtype == torch.bfloat16 else 2e-4
    close(got, want, atol=rel * scale + 1e-30)
    assert rel_l2(got, want) <= (1e-2 if got.dtype == torch.float32 else 2e-2)


# ---- quantisers ---------------------------------------------------------------------------------------------


def quantize_matches_rules(lx, fmt, rows, cols, seed, spread=4.0, zero_row=False, zero_block=False):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(rows, cols, generator=g) * torch.rand(rows, 1, generator=g) * spread
    if fmt == W_NVFP4:
        w = w * torch.rand(rows, cols // 16, generator=g).repeat_interleave(16, 1)
    w = w.to(torch.bfloat16)
    if zero_row and rows > 2:
        w[0] = 0.0
    if zero_block and fmt == W_NVFP4:
        w[:, :16] = 0.0
    got = quantize_with(lx, dev(lx, w), fmt)
    want = quantize_reference(w, fmt)
    assert torch.equal(got.data.cpu().view(torch.uint8), want.data.view(torch.uint8)), "quantised bytes differ"
    if fmt == W_NVFP4:
        assert got.glob == want.glob, "global differs from max|w| / 2688"
        assert torch.equal(got.scale.cpu(), want.scale), "block scales differ"
    else:
        assert torch.equal(got.scale.cpu(), want.scale), "row scales differ"
    return got


def quantize_w8_matches(lx, rows, cols, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(rows, cols, generator=g) * torch.rand(rows, 1, generator=g) * 4).to(torch.bfloat16)
    q = torch.empty(rows, cols, dtype=torch.int8, device=lx.device)
    scale = torch.empty(rows, dtype=torch.float32, device=lx.device)
    lx("quantize_w8", dev(lx, w), q, scale, ctypes.c_int64(rows), cols)
    want = quantize_reference(w, W_INT8)
    assert torch.equal(q.cpu(), want.data) and torch.equal(scale.cpu(), want.scale)


def int8_known_answers(lx):
    # ties to even (0.5 -> 0, 1.5 -> 2, 2.5 -> 2), the clamp, and a zero row keeping scale 1
    w = torch.zeros(3, 8)
    w[0] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, -127.0])
    w[1] = torch.tensor([254.0, 1.0, 3.0, 5.0, -1.0, -3.0, -5.0, -254.0])
    got = quantize_with(lx, dev(lx, w.to(torch.bfloat16)), W_INT8)
    assert got.scale.cpu().tolist() == [1.0, 2.0, 1.0]
    assert got.data.cpu()[0].tolist() == [127, 0, 2, 2, 0, -2, -2, -127]
    assert got.data.cpu()[1].tolist() == [127, 0, 2, 2, 0, -2, -2, -127]
    assert got.data.cpu()[2].tolist() == [0] * 8


def nvfp4_known_answers(lx):
    # The block with absmax 2688 makes the global 1; a block with absmax 12 gets scale 2 (0x40), so w / 2 lands
    # on the e2m1 midpoints, which go to the even code; -0.25 rounds to an unsigned zero
    # (tests/kernels/test_quant.py:107-126 of the reference).
    w = torch.zeros(2, 16)
    w[0, 0] = 2688.0
    w[1, 0] = 12.0
    ties = torch.tensor([0.5, 1.5, 2.5, 3.5, 5.0, 7.0, 10.0])
    w[1, 1:8] = ties
    w[1, 8:15] = -ties
    got = quantize_with(lx, dev(lx, w.to(torch.bfloat16)), W_NVFP4)
    assert got.glob == 1.0
    data = got.data.cpu()
    codes = torch.stack([data & 15, data >> 4], dim=-1).flatten(-2)
    assert codes[1, 1:8].tolist() == [0, 2, 2, 4, 4, 6, 6]
    assert codes[1, 8:15].tolist() == [0, 10, 10, 12, 12, 14, 14]
    assert got.scale.cpu()[1, 0].item() == 0x40 and codes[1, 0].item() == 7


def dequantize_is_exact(lx, fmt, N, K, seed):
    w = random_weight(fmt, N, K, seed)
    got = ops.dequantize(lx, w.to(lx.device), N, K)
    want = w.dense().float().to(torch.bfloat16)  # the product is exact in f32 for INT8 / FP8 scales? no: rounded once
    # element * rowfactor is one f32 multiply of exact operands, then one rounding to bf16: compute it that way.
    if fmt in (W_INT8, W_FP8):
        elem = w.dense() / w.scale.double().unsqueeze(-1)
        want = (elem.float() * w.scale.unsqueeze(-1)).to(torch.bfloat16)
    elif fmt == W_NVFP4:
        elem = w.dense() / w.glob
        want = (elem.float() * torch.tensor(w.glob, dtype=torch.float32)).to(torch.bfloat16)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16)), "dequantised bf16 bits differ"


# ---- GEMV -------------------------------------------------------------------------------------------------


def gemv_case(lx, fmt, M, N, K, seed, x_dtype=torch.float32, bias_dtype=None, y_dtype=torch.float32, alpha=1.0,
              beta=0.0, pad=0, entry="gemv_w"):
    g = torch.Generator().manual_seed(seed)
    w = random_weight(FORMATS[fmt] if isinstance(fmt, str) else fmt, N, K, seed + 1)
    x_buf = torch.randn(M, K + pad, generator=g).to(x_dtype)
    bias = None if bias_dtype is None else torch.randn(N, generator=g).to(bias_dtype)
    y0 = torch.randn(M, N + pad, generator=g).to(y_dtype)
    # With beta 0 the kernel must not read y: it starts as NaN.
    y = y0.clone() if beta != 0.0 else torch.full((M, N + pad), float("nan"), dtype=y_dtype)
    if pad and beta == 0.0:
        y[:, N:] = y0[:, N:]
    yd = dev(lx, y)
    ops.gemv_w(lx, dev(lx, x_buf), w.to(lx.device), None if bias is None else dev(lx, bias), yd, alpha, beta, M=M, N=N, K=K,
               ld_x=K + pad, ld_y=N + pad, entry=entry)
    want = ops.gemv_reference(x_buf[:, :K], w.dense(), bias, alpha, beta, y0[:, :N])
    got = yd.cpu()
    check_product(got[:, :N], want)
    if pad:
        assert torch.equal(got[:, N:].view(torch.uint8), y0[:, N:].contiguous().view(torch.uint8).reshape(M, -1)), "wrote past N"
    return got[:, :N]


def gemv_rows_do_not_depend_on_batch(lx, fmt, N, K, seed):
    w = random_weight(FORMATS[fmt], N, K, seed).to(lx.device)
    g = torch.Generator().manual_seed(seed + 1)
    x = dev(lx, torch.randn(8, K, generator=g).to(torch.bfloat16))
    alone = torch.cat([ops.gemv_w(lx, x[m : m + 1].contiguous(), w) for m in range(8)])
    for M in range(1, 9):
        y = ops.gemv_w(lx, x[:M].contiguous(), w)
        assert torch.equal(y.view(torch.int32), alone[:M].view(torch.int32)), f"M={M}: a row differs from the row alone"


def gemv_nvfp4_global_is_linear(lx):
    N, K, M = 64, 2048, 2
    g = torch.Generator().manual_seed(9)
    x = dev(lx, torch.randn(M, K, generator=g))
    w = random_weight(W_NVFP4, N, K, 4).to(lx.device)
    y1 = ops.gemv_w(lx, x, w)
    w.glob *= 2.0
    y2 = ops.gemv_w(lx, x, w)
    assert torch.equal(y2, 2.0 * y1)


# ---- activation quantiser ----------------------------------------------------------------------------------


def quantize_act_case(lx, math, M, K, seed, x_dtype=torch.float32, pad=0, x_pad=0):
    """Bytes, row scales and block scales equal the contract's rules; nothing is written past a row."""
    from dromos_amd.formats import quantize_act_reference

    g = torch.Generator().manual_seed(seed)
    x_buf = (torch.randn(M, K + x_pad, generator=g) * torch.rand(M, 1, generator=g) * 4).to(x_dtype)
    x_buf[0, :K] *= 1e-3  # a quiet row: small scales, subnormal e4m3 block scales for FP4
    if M > 2:
        x_buf[2, :K] = 0  # a zero row
    x = x_buf[:, :K]
    q, scale, bs = ops.quantize_act(lx, dev(lx, x_buf), math, pad=pad, K=K)
    want_q, want_scale, want_bs = quantize_act_reference(x, math)
    width = want_q.shape[1]
    q, scale = q.cpu(), scale.cpu()
    assert torch.equal(q[:, :width], want_q), f"quantised values differ at {(q[:, :width] != want_q).nonzero()[:4].tolist()}"
    assert torch.equal(scale.view(torch.int32), want_scale.float().view(torch.int32)), "per-row scales differ"
    assert bool((q[:, width:] == 0xAB).all()), "wrote past the row"
    if want_bs is not None:
        bs = bs.cpu()
        assert torch.equal(bs[:, : K // 16], want_bs), "block scales differ"
        assert bool((bs[:, K // 16 :] == 0xAB).all()), "wrote past the block scales"
    if M > 2:
        assert bool((q[2, :width] == 0).all()) and scale[2].item() == 1.0, "a zero row quantises to 0 with scale 1"
    return q, scale, bs


def quantize_act_fp4_extremes(lx):
    """Ties of the e2m1 rounding, saturation, and a block whose scale underflows to zero
    (the cases of tests/kernels/test_quant_act.py:59-72 of the reference)."""
    from dromos_amd.abi import MATH_FP4
    from dromos_amd.formats import quantize_act_reference

    M, K = 4, 64
    x = torch.zeros(M, K)
    x[0, :16] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, -0.25, -0.75, -2.5, -5.0, 0.1, 7.0, -7.0, 3.0])
    x[1, :16] = 1.0
    x[1, 16:32] = 1e-6
    x[2] = torch.linspace(-3, 3, K)
    q, scale, bs = ops.quantize_act(lx, dev(lx, x), MATH_FP4)
    want_q, want_scale, want_bs = quantize_act_reference(x, MATH_FP4)
    assert torch.equal(q.cpu(), want_q) and torch.equal(scale.cpu(), want_scale.float()) and torch.equal(bs.cpu(), want_bs)
    # Known answers, by hand: row 1's first block is all ones with the row's absmax 1: g = 1 / 2688,
    # s_b = e4m3(1 / (6 g)) = e4m3(448) = 0x7e, code = e2m1(1 * (1 / (448 / 2688))) = e2m1(6) = 7; its second block
    # underflows: scale byte 0 and zero codes; the all-zero row 3 has scale 1.
    assert bs[1, 0].item() == 0x7E and bool((q[1, :8].cpu() == 0x77).all())
    assert bs[1, 1].item() == 0 and bool((q[1, 8:16].cpu() == 0).all())
    assert scale[3].item() == 1.0 and bool((q[3].cpu() == 0).all())


# ---- routing ----------------------------------------------------------------------------------------------


def route_case(lx, T, E, top_k, seed, with_bias=True):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(T, E, generator=g) * 2).float()
    bias = (torch.randn(E, generator=g) * 0.5).float() if with_bias else None
    biased = logits if bias is None else logits + bias
    if top_k < E:
        desc = torch.sort(biased, dim=-1, descending=True).values[:, : top_k + 1]
        assert (desc[:, :-1] - desc[:, 1:]).min().item() > 1e-6, "near tie in the test logits, pick another seed"
    ids, weights, entropy, confidence = ops.route(lx, dev(lx, logits), None if bias is None else dev(lx, bias), top_k)
    want_ids, want_w, want_h, want_c = ops.route_reference(logits, bias, top_k)
    assert torch.equal(ids.cpu().long(), want_ids), "expert ids differ"
    close(weights, want_w, atol=1e-5)
    close(entropy, want_h, atol=1e-5)
    close(confidence, want_c, atol=1e-5)


def route_ties(lx):
    logits = torch.tensor([[0.5, 2.0, 2.0, -1.0, 2.0, 0.0, 1.0, 0.0]])
    ids, weights, entropy, confidence = ops.route(lx, dev(lx, logits), None, 3)
    assert ids.cpu().tolist() == [[1, 2, 4]]
    close(weights, torch.full((1, 3), 1.0 / 3.0), atol=1e-6)
    _, _, want_h, want_c = ops.route_reference(logits, None, 3)
    close(entropy, want_h, atol=1e-5)
    close(confidence, want_c, atol=1e-5)
    # the bias decides the picks, the unbiased logits the weights
    logits = torch.tensor([[1.0, 0.0, 0.5, -2.0, -3.0]])
    bias = torch.tensor([0.0, 1.0, 0.5, 0.0, 0.0])
    ids, weights, _, _ = ops.route(lx, dev(lx, logits), dev(lx, bias), 2)
    assert ids.cpu().tolist() == [[0, 1]]
    close(weights, torch.softmax(torch.tensor([[1.0, 0.0]]), -1), atol=1e-6)


def awkward_logits(E, top_k, T=48):
    """Logits and a bias where floats are awkward for a pick order: many equal values, signed zeros (equal: the lower
    index goes first), denormals (distinct from zero), infinities and NaNs (never picked while anything else can be),
    rows of one value, a row with fewer rankable values than picks."""
    g = torch.Generator().manual_seed(E * 31 + top_k)
    pool = torch.tensor([0.0, -0.0, 1e-40, -1e-40, 1.0, 1.0, -1.0, 2.5, float("inf"), float("-inf"), float("nan"), -float("nan"), 3e-39])
    logits = pool[torch.randint(0, len(pool), (T, E), generator=g)].contiguous()
    logits[0] = 0.0
    logits[1] = float("-inf")
    logits[2] = float("nan")
    logits[3, : E // 2] = -0.0
    logits[4] = torch.where(torch.arange(E) % 2 == 0, torch.tensor(-0.0), torch.tensor(0.0))
    logits[5, top_k - 1:] = float("nan")
    bias = pool[torch.randint(0, 8, (E,), generator=g)].contiguous()
    return logits, bias


def same_routes(a, w, E):
    """Two lx_moe_route results: the same ids; the same weights on every row whose picks all exist. A row with fewer
    rankable logits than picks gets the id E for the rest, and its weights are not compared: the reference's softmax
    then reads the element behind the row (engine/cpu/moe.cpp:383-395), which is nobody's contract."""
    assert torch.equal(a[0].cpu(), w[0].cpu())
    whole = (a[0].cpu() < E).all(-1)
    x, y = a[1].cpu()[whole], w[1].cpu()[whole]
    both = torch.isnan(x) & torch.isnan(y)
    close(torch.where(both, 0.0, x), torch.where(both, 0.0, y), atol=1e-5)


# ---- experts ------------------------------------------------------------------------------------------------


def make_routing(T, E, L, top_k, seed, pool=None):
    g = torch.Generator().manual_seed(seed)
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16)
    if pool is None:
        ids = torch.rand(T, E, generator=g).argsort(-1)[:, :top_k]
    else:
        ids = pool[torch.rand(T, len(pool), generator=g).argsort(-1)[:, :top_k]]
    weights = torch.softmax(torch.randn(T, top_k, generator=g), -1)
    return latent.contiguous(), ids.to(torch.int32).contiguous(), weights.contiguous()


def experts_close(out, want, tol=1e-3):
    scale = want.abs().max().item()
    close(out, want, atol=tol * scale, rtol=tol)
    assert rel_l2(out, want) <= 1e-2


def decode_case(lx, gu_fmt, dn_fmt, T, E, L, I, top_k, seed, pool=None):
    gu = random_stack(FORMATS[gu_fmt], E, 2 * I, L, seed + 1)
    dn = random_stack(FORMATS[dn_fmt], E, L, I, seed + 2)
    latent, ids, weights = make_routing(T, E, L, top_k, seed, pool)
    out = ops.experts_decode(lx, dev(lx, latent), dev(lx, ids), dev(lx, weights), gu.to(lx.device), dn.to(lx.device), I, top_k)
    want = ops.experts_reference(latent, ids, weights, gu.dense(), dn.dense())
    experts_close(out, want)
    return out


def grouped_case(lx, fmt, T, L, I, E, top_k, seed, skew=False, tol=2e-3):
    g = torch.Generator().manual_seed(seed)
    gu = quantize_reference_stack(torch.randn(E, 2 * I, L, generator=g) / L**0.5, FORMATS[fmt])
    dn = quantize_reference_stack(torch.randn(E, L, I, generator=g) / I**0.5, FORMATS[fmt])
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16)
    noise = torch.rand(T, E, generator=g)
    if skew:
        hot = torch.randperm(E, generator=g)[: max(top_k, 3)]
        noise[:, hot] += 10.0 * (torch.rand(T, 1, generator=g) < 0.9)
    ids = noise.argsort(-1, descending=True)[:, :top_k].to(torch.int32).contiguous()
    weights = torch.softmax(torch.randn(T, top_k, generator=g), -1).contiguous()
    out = ops.experts_grouped(lx, dev(lx, latent), dev(lx, ids), dev(lx, weights), gu.to(lx.device), dn.to(lx.device), I, E, top_k)
    want = ops.experts_reference(latent, ids, weights, gu.dense(), dn.dense())
    close(out, want, atol=tol * want.abs().max().item())
    assert rel_l2(out, want) <= 1e-2
    return out


def quantize_reference_stack(w, fmt):
    """[E, N, K] float -> a stack in `fmt`; NVFP4 experts are quantised one by one, each with its own global."""
    wb = w.to(torch.bfloat16)
    if fmt != W_NVFP4:
        return quantize_reference(wb, fmt)
    parts = [quantize_reference(wb[e], fmt) for e in range(wb.shape[0])]
    eg = torch.tensor([p.glob for p in parts], dtype=torch.float32)
    return Weight(fmt, torch.stack([p.data for p in parts]), torch.stack([p.scale for p in parts]), parts[0].glob, eg)


# ---- lossless bf16 (LX_W_BF16X) ----------------------------------------------------------------------------------


def bf16x_weights(rows, K, seed, kind="trained"):
    """bf16 [rows, K] whose exponents exercise the format.
    trained: N(0, 0.02) with a sprinkle of values many binades down (a few exceptions a row, within the slots);
    wild:    every bit pattern is possible (infinities, NaNs, denormals, both zeros), exponents spread over all 256;
    spill:   rows where most values lie far below a few large ones (more exceptions than slots: spill records),
             mixed with rows that have none."""
    g = torch.Generator().manual_seed(seed)
    if kind == "wild":
        return torch.randint(-32768, 32768, (rows, K), generator=g, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    w = (torch.randn(rows, K, generator=g) * 0.02).to(torch.bfloat16)
    if kind == "trained":
        tiny = torch.rand(rows, K, generator=g) < 2.0 / K
        w[tiny] = (w[tiny].float() * 2.0**-40).to(torch.bfloat16)
        w[torch.rand(rows, K, generator=g) < 1.0 / K] = 0.0
        return w
    assert kind == "spill"
    small = torch.rand(rows, K, generator=g) < 0.3
    w[small] = (w[small].float() * 2.0**-30).to(torch.bfloat16)
    w[1::3] = (torch.randn(K, generator=g) * 0.02).to(torch.bfloat16)  # rows without exceptions in between
    return w


def bf16x_geometry(K):
    spans = (K + 127) // 128
    header = (4 * (2 + K // 2048) + spans + 7) // 8 * 8
    return spans, header, (header - spans) // 4, header + 192 * spans


def bf16x_round_trip(lx, rows, K, seed, kind):
    """encode -> the library's decode and the numpy reading of the layout both give back every bit; the size is the
    closed form plus spill records; nothing is written past it."""
    w = dev(lx, bf16x_weights(rows, K, seed, kind))
    enc = ops.bf16x_encode(lx, w, slack=64)
    _, _, slots, rb = bf16x_geometry(K)
    assert ops.bf16x_row_bytes(lx, K) == rb
    # Exceptions a row: values more than 15 binades under the largest exponent of their span of 128.
    e = ((w.cpu().view(torch.int16).int() >> 7) & 0xFF)
    pad = (-K) % 128
    span_e = torch.nn.functional.pad(e, (0, pad), value=0).view(rows, -1, 128)
    inside = torch.nn.functional.pad(torch.ones_like(e, dtype=torch.bool), (0, pad), value=False).view(rows, -1, 128)
    counts = (((span_e.max(-1, keepdim=True).values - span_e) > 15) & inside).sum((-1, -2))
    spill = sum((4 * (int(n) + 2) + 7) // 8 * 8 for n in counts if n > slots)
    assert enc.numel() - 64 == rows * rb + spill
    assert bool((enc[-64:] == 0xEE).all())
    back = ops.bf16x_decode(lx, enc, rows, K)
    assert torch.equal(back.view(torch.int16).cpu(), w.view(torch.int16).cpu())
    assert torch.equal(ops.bf16x_decode_reference(enc[:-64], rows, K).view(torch.int16), w.view(torch.int16).cpu())
    return w, enc[:-64], counts
