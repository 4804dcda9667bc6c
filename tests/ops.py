"""Calls into a backend library (an abi.Kernels), shared by the CPU and GPU tests: each function allocates
the outputs on the library's device, calls one lx_* entry point and returns the result."""

import ctypes

import torch

from dromos_amd.abi import DTYPE, F32, MATH_BF16
from dromos_amd.formats import Weight


def gemv_w(lx, x, w, bias=None, y=None, alpha=1.0, beta=0.0, M=None, N=None, K=None, ld_x=None, ld_y=None,
           y_dtype=torch.float32, entry="gemv_w", status=False):
    M = x.shape[0] if M is None else M
    K = x.shape[1] if K is None else K
    N = w.data.shape[-2] if N is None else N
    if y is None:
        y = torch.full((M, N), float("nan"), dtype=y_dtype, device=lx.device)
    lw = w.lx()
    args = (x, DTYPE[x.dtype], ld_x if ld_x is not None else x.shape[1], ctypes.pointer(lw), bias,
            DTYPE[bias.dtype] if bias is not None else F32, y, DTYPE[y.dtype], ld_y if ld_y is not None else y.shape[1],
            M, N, K, float(alpha), float(beta))
    if status:
        return lx.status(entry, *args)
    lx(entry, *args)
    return y


def gemm_w(lx, x, w, math=MATH_BF16, bias=None, y=None, alpha=1.0, beta=0.0, y_dtype=torch.float32, status=False,
           ld_x=None, ld_y=None, N=None):
    M, K = x.shape[0], w_cols(w)
    N = w.data.shape[-2] if N is None else N
    if y is None:
        y = torch.full((M, N), float("nan"), dtype=y_dtype, device=lx.device)
    nbytes = max(int(lx.size("gemm_workspace_bytes", M, K, math)), 256)
    ws = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=lx.device)
    lw = w.lx()
    args = (x, DTYPE[x.dtype], ld_x if ld_x is not None else x.shape[1], ctypes.pointer(lw), math, bias,
            DTYPE[bias.dtype] if bias is not None else F32, y, DTYPE[y.dtype], ld_y if ld_y is not None else y.shape[1],
            M, N, K, float(alpha), float(beta), ws)
    if status:
        return lx.status("gemm_w", *args)
    lx("gemm_w", *args)
    return y


def w_cols(w):
    from dromos_amd.abi import W_NVFP4

    return w.data.shape[-1] * 2 if w.fmt == W_NVFP4 else w.data.shape[-1]


def gemm_skinny(lx, x, w, bias=None, y=None, alpha=1.0, beta=0.0, y_dtype=torch.float32, status=False):
    M, K = x.shape
    N = w.data.shape[-2]
    if y is None:
        y = torch.full((M, N), float("nan"), dtype=y_dtype, device=lx.device)
    lw = w.lx()
    args = (x, DTYPE[x.dtype], K, ctypes.pointer(lw), bias, DTYPE[bias.dtype] if bias is not None else F32, y,
            DTYPE[y.dtype], N, M, N, K, float(alpha), float(beta))
    if status:
        return lx.status("gemm_skinny", *args)
    lx("gemm_skinny", *args)
    return y


def dequantize(lx, w, N, K):
    out = torch.empty(N, K, dtype=torch.bfloat16, device=lx.device)
    lw = w.lx()
    lx("dequantize_weight", ctypes.pointer(lw), out, ctypes.c_int64(N), K)
    return out


def quantize_act(lx, x, math, pad=0, status=False, K=None):
    """lx_quantize_act on the first K columns of x [M, ld_x]; returns (q bytes [M, ld_q], scale [M], block scales
    [M, ld_bs] or None). pad > 0 widens the output rows, filled with 0xAB, to show nothing is written past a row."""
    from dromos_amd.abi import MATH_FP4

    M = x.shape[0]
    K = x.shape[1] if K is None else K
    ld_q = (K // 2 if math == MATH_FP4 else K) + pad
    q = torch.full((M, ld_q), 0xAB, dtype=torch.uint8, device=lx.device)
    scale = torch.full((M,), float("nan"), dtype=torch.float32, device=lx.device)
    ld_bs = K // 16 + pad if math == MATH_FP4 else 0
    bs = torch.full((M, max(ld_bs, 1)), 0xAB, dtype=torch.uint8, device=lx.device) if math == MATH_FP4 else None
    args = (x, DTYPE[x.dtype], x.shape[1], math, q, ld_q, scale, bs, ld_bs, M, K)
    if status:
        return lx.status("quantize_act", *args)
    lx("quantize_act", *args)
    return q, scale, bs


def route(lx, logits, bias, top_k):
    T, E = logits.shape
    ids = torch.full((T, top_k), -1, dtype=torch.int32, device=lx.device)
    weights = torch.full((T, top_k), float("nan"), dtype=torch.float32, device=lx.device)
    entropy = torch.full((T,), float("nan"), dtype=torch.float32, device=lx.device)
    confidence = torch.full((T,), float("nan"), dtype=torch.float32, device=lx.device)
    lx("moe_route", logits, bias, ids, weights, entropy, confidence, T, E, top_k)
    return ids, weights, entropy, confidence


def experts_decode(lx, latent, ids, weights, gu, dn, I, top_k, status=False):
    T, L = latent.shape
    nbytes = int(lx.size("moe_decode_workspace_bytes", T, I, top_k))
    assert nbytes >= 2 * T * top_k * I
    ws = torch.full((max(nbytes, 1),), 0xFF, dtype=torch.uint8, device=lx.device)  # garbage: NaN bf16
    out = torch.full((T, L), float("nan"), device=lx.device)
    g, d = gu.lx(), dn.lx()
    args = (latent, ids, weights, ctypes.pointer(g), ctypes.pointer(d), out, ws, T, L, I, top_k)
    if status:
        return lx.status("moe_experts_decode", *args)
    lx("moe_experts_decode", *args)
    return out


def experts_grouped(lx, latent, ids, weights, gu, dn, I, E, top_k, math=MATH_BF16, status=False):
    T, L = latent.shape
    fn = lx.lib.lx_moe_grouped_workspace_bytes
    fn.restype = ctypes.c_int64
    nbytes = int(fn(T, L, I, E, top_k, math))
    ws = torch.full((max(nbytes, 1),), 0xFF, dtype=torch.uint8, device=lx.device)
    out = torch.full((T, L), float("nan"), device=lx.device)
    g, d = gu.lx(), dn.lx()
    args = (latent, ids, weights, ctypes.pointer(g), ctypes.pointer(d), math, out, ws, T, L, I, E, top_k)
    if status:
        return lx.status("moe_experts_grouped", *args)
    lx("moe_experts_grouped", *args)
    return out


def experts_bf16(lx, latent, ids, weights, gate_up, down, I, top_k):
    T, L = latent.shape
    out = torch.full((T, L), float("nan"), device=lx.device)
    lx("moe_experts", latent, ids, weights, gate_up, down, out, T, L, I, top_k)
    return out


# ---- float64 statements of what the ops compute, from closed forms only ----------------------------------


def gemv_reference(x, dense, bias, alpha, beta, y0):
    out = x.double().cpu() @ dense.double().T
    if bias is not None:
        out = out + bias.double().cpu()
    out = alpha * out
    if beta != 0.0:
        out = out + beta * y0.double().cpu()
    return out


def route_reference(logits, bias, top_k):
    """Selection on f32 biased logits (one IEEE add), stable descending order; weights and statistics in float64."""
    logits = logits.cpu()
    biased = logits.float() if bias is None else logits.float() + bias.cpu().float()
    ids = torch.sort(-biased, dim=-1, stable=True).indices[:, :top_k]
    wide = logits.double()
    weights = torch.softmax(torch.gather(wide, -1, ids), dim=-1)
    p = torch.softmax(wide, dim=-1)
    entropy = -(p * torch.log(p.clamp_min(1e-9))).sum(-1)
    return ids, weights, entropy, p.max(-1).values


def experts_reference(latent, ids, weights, gu_dense, dn_dense):
    """float64 experts on dense stacks gu [E, 2I, L], dn [E, L, I]; the intermediate is rounded to bf16."""
    import torch.nn.functional as F

    I = gu_dense.shape[1] // 2
    x = latent.double().cpu()
    ids, weights = ids.cpu(), weights.cpu()
    out = torch.zeros(x.shape[0], x.shape[1], dtype=torch.float64)
    for t in range(ids.shape[0]):
        for k in range(ids.shape[1]):
            e = int(ids[t, k])
            g, u = gu_dense[e, :I] @ x[t], gu_dense[e, I:] @ x[t]
            mid = (F.silu(g) * u).to(torch.bfloat16).double()
            out[t] += weights[t, k].double() * (dn_dense[e] @ mid)
    return out


# ---- the calls either side of the experts, and the legacy product forms ----------------------------------------


def spec_gemv_f32(lx, x, w, bias=None, M=None, status=False):
    M = x.shape[0] if M is None else M
    N, K = w.shape
    y = torch.full((max(M, 1), N), float("nan"), device=lx.device)
    args = (x, x.shape[1], w, bias, y, N, M, N, K)
    if status:
        return lx.status("spec_gemv_f32", *args)
    lx("spec_gemv_f32", *args)
    return y[:M]


def gemm_f32(lx, x, w, bias=None, pad=0, status=False):
    """lx_gemm_f32 with `pad` unused columns behind the rows of x and y."""
    M, K = x.shape
    N = w.shape[0]
    xb = torch.zeros(M, K + pad, device=lx.device)
    xb[:, :K] = x
    y = torch.full((max(M, 1), N + pad), float("nan"), device=lx.device)
    args = (xb, K + pad, w, bias, y, N + pad, M, N, K)
    if status:
        return lx.status("gemm_f32", *args)
    lx("gemm_f32", *args)
    return y[:M]


def router_route(lx, x, w, bias, selection_bias, top_k, status=False):
    M, K = x.shape
    E = w.shape[0]
    logits = torch.full((M, E), float("nan"), device=lx.device)
    ids = torch.full((M, top_k), -1, dtype=torch.int32, device=lx.device)
    weights = torch.full((M, top_k), float("nan"), device=lx.device)
    entropy = torch.full((M,), float("nan"), device=lx.device)
    confidence = torch.full((M,), float("nan"), device=lx.device)
    ticket = torch.zeros(1, dtype=torch.int32, device=lx.device)
    args = (x, K, w, bias, logits, selection_bias, ids, weights, entropy, confidence, ticket, M, E, K, top_k)
    if status:
        return lx.status("router_route", *args)
    lx("router_route", *args)
    assert ticket.item() == 0
    return logits, ids, weights, entropy, confidence


def moe_summary(lx, ids, weights, emb, history=None, a=0.0, b=0.0):
    T, top_k = ids.shape
    R = emb.shape[1]
    out = torch.full((T, R), float("nan"), device=lx.device)
    if history is None:
        lx("moe_summary", ids, weights, emb, out, T, R, top_k)
    else:
        lx("moe_summary_history", ids, weights, emb, out, history, float(a), float(b), T, R, top_k)
    return out


def experts_w8(lx, latent, ids, weights, gu, dn, I, top_k, status=False):
    T, L = latent.shape
    nbytes = int(lx.size("moe_workspace_bytes", T, I, top_k))
    ws = torch.full((max(nbytes, 1),), 0xFF, dtype=torch.uint8, device=lx.device)
    out = torch.full((T, L), float("nan"), device=lx.device)
    args = (latent, ids, weights, gu.data, gu.scale, dn.data, dn.scale, out, ws, T, L, I, top_k)
    if status:
        return lx.status("moe_experts_w8", *args)
    lx("moe_experts_w8", *args)
    return out


def gemm_bf16(lx, x, w, bias=None, y=None, alpha=1.0, beta=0.0, y_dtype=torch.float32):
    M, K = x.shape
    N = w.shape[0]
    if y is None:
        y = torch.full((M, N), float("nan"), dtype=y_dtype, device=lx.device)
    lx("gemm_bf16", x, K, w, bias, y, DTYPE[y.dtype], N, M, N, K, float(alpha), float(beta))
    return y


# ---- lossless bf16 (LX_W_BF16X) ----------------------------------------------------------------------------------


def bf16x_row_bytes(lx, K):
    fn = lx.lib.lx_bf16x_row_bytes
    fn.restype = ctypes.c_int64
    return int(fn(ctypes.c_int(K)))


def bf16x_bytes(lx, w):
    """lx_bf16x_bytes of bf16 rows w [rows, K] (a stack is flattened to rows)."""
    K = w.shape[-1]
    rows = w.numel() // K
    fn = lx.lib.lx_bf16x_bytes
    fn.restype = ctypes.c_int64
    return int(fn(ctypes.c_void_p(w.data_ptr()), ctypes.c_int64(rows), ctypes.c_int(K), lx.stream))


def bf16x_encode(lx, w, slack=0):
    """The encoding of bf16 w [..., K] as a uint8 tensor of exactly lx_bf16x_bytes (+ slack bytes of 0xEE, to show
    nothing is written past the end)."""
    w = w.contiguous()
    K = w.shape[-1]
    rows = w.numel() // K
    n = bf16x_bytes(lx, w)
    assert n >= rows * bf16x_row_bytes(lx, K)
    out = torch.full((n + slack,), 0xEE, dtype=torch.uint8, device=lx.device)
    assert out.data_ptr() % 8 == 0
    lx("bf16x_encode", w, ctypes.c_int64(rows), K, out, ctypes.c_int64(n))
    return out


def bf16x_decode(lx, data, rows, K):
    w = torch.full((rows, K), -1, dtype=torch.int16, device=lx.device).view(torch.bfloat16)
    lx("bf16x_decode", data, ctypes.c_int64(rows), K, w)
    return w


def gemv_bf16x(lx, x, data, N, bias=None, y=None, alpha=1.0, beta=0.0, y_dtype=torch.float32, entry="gemv_bf16x", status=False):
    """lx_gemv_bf16x (or lx_gemv_decode_bf16 with `data` the plain bf16 weights)."""
    M, K = x.shape
    if y is None:
        y = torch.full((M, N), float("nan"), dtype=y_dtype, device=lx.device)
    args = (x, DTYPE[x.dtype], K, data, bias, DTYPE[bias.dtype] if bias is not None else F32, y, DTYPE[y.dtype], N, M, N, K,
            float(alpha), float(beta))
    if status:
        return lx.status(entry, *args)
    lx(entry, *args)
    return y


def experts_bf16x(lx, latent, ids, weights, gate_up, down, I, top_k, entry="moe_experts_bf16x", status=False):
    """lx_moe_experts_bf16x on encoded stacks (or lx_moe_experts_decode_bf16 on plain bf16 stacks)."""
    T, L = latent.shape
    nbytes = int(lx.size("moe_bf16x_workspace_bytes", T, I, top_k))
    ws = torch.full((max(nbytes, 1),), 0xFF, dtype=torch.uint8, device=lx.device)
    out = torch.full((T, L), float("nan"), device=lx.device)
    args = (latent, ids, weights, gate_up, down, out, ws, T, L, I, top_k)
    if status:
        return lx.status(entry, *args)
    lx(entry, *args)
    return out


def bf16x_decode_reference(data, rows, K):
    """The layout read back with numpy alone (no library): bf16 bits [rows, K] as uint16. Written from the format's
    description: S exception words, a top exponent per span of 128, 192-byte spans of 128 sign|mantissa bytes and 64
    bytes of 4-bit codes."""
    import numpy as np

    buf = data.cpu().numpy()
    spans = (K + 127) // 128
    header = (4 * (2 + K // 2048) + spans + 7) // 8 * 8
    slots = (header - spans) // 4
    rb = header + 192 * spans
    out = np.zeros((rows, K), dtype=np.uint16)
    for r in range(rows):
        rec = buf[r * rb:(r + 1) * rb]
        tops = rec[4 * slots:4 * slots + spans].astype(np.int32)
        body = rec[header:].reshape(spans, 192)
        sm = body[:, :128].astype(np.uint16)
        pairs = body[:, 128:].reshape(spans, 16, 4)
        codes = np.concatenate([pairs & 15, pairs >> 4], axis=2).reshape(spans, 128).astype(np.int32)
        e = ((tops[:, None] - codes) & 0xFF).astype(np.uint16)
        bits = ((sm & 0x80) << 8) | (e << 7) | (sm & 0x7F)
        row = bits.reshape(-1)[:K].copy()
        words = rec[:4 * slots].view(np.uint32)
        if words[0] != 0xFFFFFFFF and words[0] & 0x80000000:
            at = r * rb + int(words[0] & 0x7FFFFFFF) * 8
            n = int(buf[at:at + 4].view(np.uint32)[0])
            words = buf[at + 4:at + 4 + 4 * n].view(np.uint32)
        for word in words:
            if word == 0xFFFFFFFF:
                break
            k = int(word >> 8)
            row[k] = (row[k] & 0x807F) | ((int(word) & 0xFF) << 7)
        out[r] = row
    return torch.from_numpy(out.view(np.int16)).view(torch.bfloat16)
