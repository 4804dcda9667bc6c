"""The seeded cases behind the golden vectors in this folder.

Every case builds its inputs from torch's CPU generator (the same bits on any machine of this image; each
fixture also stores a checksum of its inputs, which the tests check first) and names the backend calls whose
outputs were recorded. ``run_case(lx, name)`` performs the calls on any library that speaks the lx_* ABI and
returns {output name: CPU tensor}; make_golden.py runs it on the reference's CPU backend, the tests on the
oracle and on the GPU library.
"""

import torch

import ops
from dromos_amd.abi import W_BF16, W_FP8, W_INT8, W_NVFP4
from dromos_amd.formats import Weight, master_weight, quantize_reference, quantize_with, random_stack, random_weight

FORMATS = {"bf16": W_BF16, "int8": W_INT8, "fp8": W_FP8, "nvfp4": W_NVFP4}


def _bits(t):
    """Any tensor -> integer view of its bytes, for exact comparison and storage."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float32,):
        return t.view(torch.int32)
    if t.dtype in (torch.bfloat16,):
        return t.view(torch.int16)
    return t


def checksum(tensors):
    """Order-sensitive 64-bit checksum of a list of tensors' bytes."""
    h = 1469598103934665603
    for t in tensors:
        b = _bits(t).flatten().to(torch.int64)
        w = torch.arange(1, b.numel() + 1, dtype=torch.int64)
        h = (h * 1099511628211 + int(((b * w) % 1000003).sum())) % (1 << 61)
    return h


def _quant_master():
    g = torch.Generator().manual_seed(4101)
    w = master_weight(24, 96, g)
    w[3] = 0  # a zero row: scale 1, zero codes
    w[5, 16:32] = 0  # a zero NVFP4 block
    w[7, :8] = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, -3.5]).to(torch.bfloat16) * 0.01  # near ties
    return w


def quantize(lx, fmt):
    w = _quant_master().to(lx.device)
    q = quantize_with(lx, w, FORMATS[fmt])
    out = {"data": q.data, "scale": q.scale}
    if fmt == "nvfp4":
        out["global"] = torch.tensor([q.glob], dtype=torch.float32)
    out["dequantized"] = ops.dequantize(lx, q, 24, 96)
    return [w], out


def quantize_act(lx, math, x_dtype):
    g = torch.Generator().manual_seed(4150 + math)
    x = (torch.randn(9, 160, generator=g) * torch.rand(9, 1, generator=g) * 4).to(x_dtype)
    x[0] *= 1e-3  # subnormal block scales
    x[2] = 0  # a zero row
    q, scale, bs = ops.quantize_act(lx, x.to(lx.device), math)
    out = {"data": q, "scale": scale}
    if bs is not None:
        out["block_scale"] = bs
    return [x], out


def gemv(lx, fmt, x_dtype, y_dtype):
    M, N, K = 3, 40, 352
    g = torch.Generator().manual_seed(4200 + FORMATS[fmt])
    x = torch.randn(M, K, generator=g).to(x_dtype)
    w = random_weight(FORMATS[fmt], N, K, 4300 + FORMATS[fmt])
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g).to(y_dtype)
    y = ops.gemv_w(lx, x.to(lx.device), w.to(lx.device), bias.to(lx.device), y0.clone().to(lx.device), alpha=0.75, beta=0.5)
    return [x, w.data, bias, y0], {"y": y}


def gemm(lx, fmt):
    M, N, K = 12, 48, 320
    g = torch.Generator().manual_seed(4400 + FORMATS[fmt])
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = random_weight(FORMATS[fmt], N, K, 4500 + FORMATS[fmt])
    bias = torch.randn(N, generator=g)
    y = ops.gemm_w(lx, x.to(lx.device), w.to(lx.device), bias=bias.to(lx.device), alpha=1.5)
    return [x, w.data, bias], {"y": y}


def gemm_math(lx, fmt, math):
    M, N, K = 12, 48, 320
    g = torch.Generator().manual_seed(4550 + math)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = random_weight(FORMATS[fmt], N, K, 4560 + math)
    bias = torch.randn(N, generator=g)
    y = ops.gemm_w(lx, x.to(lx.device), w.to(lx.device), math=math, bias=bias.to(lx.device), alpha=1.5)
    return [x, w.data, bias], {"y_exact" if math == 1 else "y": y}


def route(lx):
    T, E, top_k = 5, 64, 8
    g = torch.Generator().manual_seed(4600)
    logits = (torch.randn(T, E, generator=g) * 2).float()
    logits[1, 10] = logits[1, 3]  # a tie: the lower index wins
    bias = (torch.randn(E, generator=g) * 0.5).float()
    bias[10] = bias[3]
    ids, weights, entropy, confidence = ops.route(lx, logits.to(lx.device), bias.to(lx.device), top_k)
    return [logits, bias], {"ids": ids, "weights": weights, "entropy": entropy, "confidence": confidence}


def _expert_inputs(fmt, T):
    E, L, I, top_k = 6, 128, 64, 2
    g = torch.Generator().manual_seed(4700 + T)
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:top_k] for _ in range(T)]).to(torch.int32)
    weights = torch.softmax(torch.randn(T, top_k, generator=g), -1).float()
    gu = random_stack(FORMATS[fmt], E, 2 * I, L, 48)
    dn = random_stack(FORMATS[fmt], E, L, I, 49)
    return E, L, I, top_k, latent, ids, weights, gu, dn


def experts_decode(lx, fmt):
    E, L, I, top_k, latent, ids, weights, gu, dn = _expert_inputs(fmt, 3)
    d = lx.device
    out = ops.experts_decode(lx, latent.to(d), ids.to(d), weights.to(d), gu.to(d), dn.to(d), I, top_k)
    return [latent, ids, weights, gu.data, dn.data], {"out": out}


def experts_grouped(lx, fmt, math=0):
    E, L, I, top_k, latent, ids, weights, gu, dn = _expert_inputs(fmt, 12)
    d = lx.device
    out = ops.experts_grouped(lx, latent.to(d), ids.to(d), weights.to(d), gu.to(d), dn.to(d), I, E, top_k, math=math)
    return [latent, ids, weights, gu.data, dn.data], {"out": out}


def experts_w8(lx):
    E, L, I, top_k, latent, ids, weights, gu, dn = _expert_inputs("int8", 11)
    d = lx.device
    out = ops.experts_w8(lx, latent.to(d), ids.to(d), weights.to(d), gu.to(d), dn.to(d), I, top_k)
    return [latent, ids, weights, gu.data, dn.data], {"out": out}


def router(lx):
    M, E, K, top_k = 5, 48, 200, 6
    g = torch.Generator().manual_seed(4800)
    x = torch.randn(M, K, generator=g)
    w = torch.randn(E, K, generator=g) / K**0.5
    bias = torch.randn(E, generator=g) * 0.1
    d = lx.device
    logits = ops.spec_gemv_f32(lx, x.to(d), w.to(d), bias.to(d))
    ids, weights, _, _ = ops.route(lx, logits, None, top_k)
    emb = torch.randn(E, 40, generator=g).to(torch.bfloat16)
    hist = torch.randn(M, 40, generator=g).to(d)
    summary = ops.moe_summary(lx, ids, weights, emb.to(d), history=hist, a=0.75, b=0.25)
    return [x, w, bias, emb], {"logits": logits, "ids": ids, "summary": summary, "history": hist}


def gemm_bf16(lx):
    M, N, K = 12, 48, 320
    g = torch.Generator().manual_seed(4900)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    d = lx.device
    return [x, w, bias], {"y": ops.gemm_bf16(lx, x.to(d), w.to(d), bias.to(d), alpha=1.5)}


def experts_bf16(lx):
    E, L, I, top_k, latent, ids, weights, gu, dn = _expert_inputs("bf16", 4)
    d = lx.device
    out = ops.experts_bf16(lx, latent.to(d), ids.to(d), weights.to(d), gu.data.to(d), dn.data.to(d), I, top_k)
    return [latent, ids, weights, gu.data, dn.data], {"out": out}


def _bf16x_rows(rows, K, seed):
    """Trained-looking bf16 rows with a few values far down (exceptions within the header slots), one row with many
    (a spill record), and a partial last span."""
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(rows, K, generator=g) * 0.02).to(torch.bfloat16)
    tiny = torch.rand(rows, K, generator=g) < 3.0 / K
    w[tiny] = (w[tiny].float() * 2.0**-40).to(torch.bfloat16)
    w[2, ::5] = (w[2, ::5].float() * 2.0**-25).to(torch.bfloat16)
    w[4, 7] = 0.0
    return w


def bf16x_codec(lx):
    w = _bf16x_rows(9, 1160, 5000)
    enc = ops.bf16x_encode(lx, w.to(lx.device))
    back = ops.bf16x_decode(lx, enc, 9, 1160)
    return [w], {"data": enc, "dequantized": back}


def bf16x_gemv(lx):
    N, K, M = 40, 1160, 3
    w = _bf16x_rows(N, K, 5100)
    g = torch.Generator().manual_seed(5101)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    bias = torch.randn(N, generator=g)
    d = lx.device
    enc = ops.bf16x_encode(lx, w.to(d))
    return [w, x, bias], {"y": ops.gemv_bf16x(lx, x.to(d), enc, N, bias=bias.to(d), alpha=0.5)}


def bf16x_experts(lx):
    E, L, I, top_k, T = 5, 136, 72, 2, 10
    gu = _bf16x_rows(E * 2 * I, L, 5200).view(E, 2 * I, L)
    dn = _bf16x_rows(E * L, I, 5201).view(E, L, I)
    g = torch.Generator().manual_seed(5202)
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:top_k] for _ in range(T)]).to(torch.int32)
    weights = torch.softmax(torch.randn(T, top_k, generator=g), -1).float()
    d = lx.device
    out = ops.experts_bf16x(lx, latent.to(d), ids.to(d), weights.to(d), ops.bf16x_encode(lx, gu.to(d)), ops.bf16x_encode(lx, dn.to(d)), I, top_k)
    return [latent, ids, weights, gu, dn], {"out": out}


CASES = {}
for _f in ("int8", "fp8", "nvfp4"):
    CASES[f"quantize_{_f}"] = (quantize, (_f,))
for _f in FORMATS:
    CASES[f"gemv_{_f}_bf16x_f32y"] = (gemv, (_f, torch.bfloat16, torch.float32))
    CASES[f"gemm_{_f}"] = (gemm, (_f,))
    CASES[f"experts_decode_{_f}"] = (experts_decode, (_f,))
    CASES[f"experts_grouped_{_f}"] = (experts_grouped, (_f,))
CASES["gemv_int8_f32x_bf16y"] = (gemv, ("int8", torch.float32, torch.bfloat16))
CASES["gemv_bf16_f32x_f32y"] = (gemv, ("bf16", torch.float32, torch.float32))
for _m, _n in ((1, "int8"), (2, "fp8"), (3, "fp4")):
    CASES[f"quantize_act_{_n}_bf16"] = (quantize_act, (_m, torch.bfloat16))
CASES["quantize_act_fp8_f32"] = (quantize_act, (2, torch.float32))
CASES["gemm_int8_int8math"] = (gemm_math, ("int8", 1))
CASES["gemm_fp8_fp8math"] = (gemm_math, ("fp8", 2))
CASES["gemm_nvfp4_fp8math"] = (gemm_math, ("nvfp4", 2))
CASES["gemm_nvfp4_fp4math"] = (gemm_math, ("nvfp4", 3))
for _f, _m, _n in (("int8", 1, "int8"), ("fp8", 2, "fp8"), ("nvfp4", 2, "fp8"), ("nvfp4", 3, "fp4")):
    CASES[f"experts_grouped_{_f}_{_n}math"] = (experts_grouped, (_f, _m))
CASES["experts_w8"] = (experts_w8, ())
CASES["router"] = (router, ())
CASES["gemm_bf16"] = (gemm_bf16, ())
CASES["route"] = (route, ())
CASES["experts_bf16"] = (experts_bf16, ())
CASES["bf16x_codec"] = (bf16x_codec, ())
CASES["bf16x_gemv"] = (bf16x_gemv, ())
CASES["bf16x_experts"] = (bf16x_experts, ())

# Outputs whose bits every backend must reproduce (codec and index work); the rest are f32 sums whose last
# bits depend on the summation order (the reference's own differ between its ISA levels).
EXACT = {"data", "scale", "global", "dequantized", "ids", "block_scale", "y_exact"}  # y_exact: the INT8 math's exact sums


def run_case(lx, name):
    fn, args = CASES[name]
    inputs, outputs = fn(lx, *args)
    lx.sync()
    return checksum(inputs), {k: _bits(v) for k, v in outputs.items() if v is not None}
