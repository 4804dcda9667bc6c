"""Weights in the four stored formats (include/dromos_hip.h, lx_weight) for the harness, tests and bench.

A ``Weight`` owns the tensors of one [N, K] matrix or one [E, N, K] stack, builds the ``lx_weight`` struct
that names them, and can state the exact values its bytes stand for (``dense()``, float64, from closed
forms only: no library under test is involved). ``quantize_reference`` restates the quantisation rules of
engine/cuda/kernels.h:248-251,513-518 in torch with IEEE divisions, as a second, independent derivation of
the bytes the quantisers must produce (the reference's own tests do the same: tests/kernels/wformats.py:69-129).
"""

import torch

from .abi import W_BF16, W_FP8, W_INT8, W_NVFP4, LxWeight

E2M1_GRID = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def e4m3_table():
    """The 256 e4m3fn values by the format's definition (bias 7, subnormals m * 2^-9), float64.
    Codes 0x7f / 0xff are NaN."""
    vals = []
    for b in range(256):
        e, m = (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            v = float("nan")
        elif e == 0:
            v = m * 2.0**-9
        else:
            v = (1.0 + m / 8.0) * 2.0 ** (e - 7)
        vals.append(-v if b & 0x80 else v)
    return torch.tensor(vals, dtype=torch.float64)


def e2m1_table():
    """The 16 e2m1 values (bit 3 is the sign), float64."""
    return torch.tensor([(-1.0 if c & 8 else 1.0) * E2M1_GRID[c & 7] for c in range(16)], dtype=torch.float64)


def unpack_codes(packed):
    """[..., K/2] bytes -> [..., K] 4-bit codes; the low nibble is the even k."""
    lo, hi = packed & 15, packed >> 4
    return torch.stack((lo, hi), dim=-1).flatten(-2)


class Weight:
    def __init__(self, fmt, data, scale=None, glob=1.0, expert_global=None):
        self.fmt = fmt
        self.data = data.contiguous()
        self.scale = None if scale is None else scale.contiguous()
        self.glob = float(glob)
        self.expert_global = expert_global

    def lx(self):
        """The lx_weight struct; keep the returned object (and this Weight) alive while a call uses it."""
        return LxWeight(
            type=self.fmt,
            data=self.data.data_ptr(),
            scale=None if self.scale is None else self.scale.data_ptr(),
            global_=self.glob,
            expert_global=None if self.expert_global is None else self.expert_global.data_ptr(),
        )

    def to(self, device):
        return Weight(
            self.fmt,
            self.data.to(device),
            None if self.scale is None else self.scale.to(device),
            self.glob,
            None if self.expert_global is None else self.expert_global.to(device),
        )

    def expert(self, e):
        """Expert e of a stack as its own [N, K] weight, with its own global when the stack carries them."""
        glob = self.glob if self.expert_global is None else float(self.expert_global[e].item())
        return Weight(self.fmt, self.data[e], None if self.scale is None else self.scale[e], glob)

    def nbytes(self):
        n = self.data.numel() * self.data.element_size()
        if self.scale is not None:
            n += self.scale.numel() * self.scale.element_size()
        return n

    def dense(self):
        """The exact values [..., N, K] as float64 (row factors applied), from the stored bytes."""
        data = self.data.cpu()
        if self.fmt == W_BF16:
            return data.double()
        if self.fmt == W_INT8:
            return data.double() * self.scale.cpu().double().unsqueeze(-1)
        if self.fmt == W_FP8:
            return e4m3_table()[data.long()] * self.scale.cpu().double().unsqueeze(-1)
        codes = unpack_codes(data)
        vals = e2m1_table()[codes.long()]
        block = e4m3_table()[self.scale.cpu().long()].repeat_interleave(16, dim=-1)
        if self.expert_global is not None:
            g = self.expert_global.cpu().double().view(-1, *([1] * (vals.dim() - 1)))
        else:
            g = self.glob
        return vals * block * g


def random_weight(fmt, N, K, seed, device="cpu", glob=0.0371):
    """Random stored bytes in format `fmt` (every valid code can appear), as the reference's tests draw them
    (tests/kernels/formats.py:68-94)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    if fmt == W_BF16:
        w = (torch.randn(N, K, generator=g) * 0.5).to(torch.bfloat16)
        return Weight(fmt, w.to(device))
    if fmt == W_INT8:
        q = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
        scale = (torch.rand(N, generator=g) * 0.02 + 0.001).float()
        return Weight(fmt, q.to(device), scale.to(device))
    if fmt == W_FP8:
        b = (torch.randn(N, K, generator=g) * 3.0).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
        scale = (torch.rand(N, generator=g) * 0.02 + 0.001).float()
        return Weight(fmt, b.to(device), scale.to(device))
    if fmt == W_NVFP4:
        assert K % 16 == 0
        codes = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.int32).to(torch.uint8)
        blocks = (torch.rand(N, K // 16, generator=g) * 2.0).to(torch.float8_e4m3fn).view(torch.uint8)
        return Weight(fmt, codes.to(device), blocks.to(device), glob=glob)
    raise ValueError(fmt)


def random_stack(fmt, E, N, K, seed, device="cpu"):
    """An [E, N, K] stack of random weights; an NVFP4 stack gets a distinct global per expert."""
    parts = [random_weight(fmt, N, K, seed * 1000 + e, "cpu", glob=0.01 + 0.004 * e) for e in range(E)]
    data = torch.stack([p.data for p in parts])
    scale = None if parts[0].scale is None else torch.stack([p.scale for p in parts])
    eg = None
    if fmt == W_NVFP4:
        eg = torch.tensor([p.glob for p in parts], dtype=torch.float32)
    return Weight(fmt, data, scale, parts[0].glob, eg).to(device)


def master_weight(N, K, generator, std=0.02):
    """A bf16 master matrix ~ N(0, std) drawn from a CPU generator (bit-reproducible on any machine)."""
    return (torch.randn(N, K, generator=generator) * std).to(torch.bfloat16)


# ---- the quantisation rules, restated in torch ---------------------------------------------------------


def _div(a, b):
    """IEEE f32 division of tensors (a scalar divisor would be turned into a reciprocal multiply)."""
    a = a if isinstance(a, torch.Tensor) else torch.full_like(b, a)
    b = b if isinstance(b, torch.Tensor) else torch.full_like(a, b)
    return a / b.expand_as(a)


def e4m3_bytes(v):
    """f32 -> e4m3fn bytes, nearest even, saturating at 448."""
    return v.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)


def e2m1_codes(v):
    """f32 -> nearest e2m1 code, ties to the even code, saturating at 6, zero unsigned."""
    a = v.abs()
    idx = torch.zeros_like(a, dtype=torch.int32)
    # thresholds between codes i and i + 1: a strict ">" when the even neighbour is below, ">=" when above
    for thr, strict in ((0.25, True), (0.75, False), (1.25, True), (1.75, False), (2.5, True), (3.5, False), (5.0, True)):
        idx = idx + ((a > thr) if strict else (a >= thr)).int()
    sign = ((v < 0) & (idx > 0)).int() * 8
    return (idx | sign).to(torch.uint8)


def quantize_reference(w, fmt):
    """bf16 [N, K] (or [E, N, K] for INT8 / FP8) -> Weight by the contract's rules (engine/cuda/kernels.h:248-251,
    513-518): per-row absmax scales /127 or /448; NVFP4 global = max|w| / 2688, block scale =
    e4m3(absmax_b / (6 * global)), code = e2m1(w / (e4m3 value * global)), zero where the block scale is zero."""
    wf = w.float()
    if fmt == W_BF16:
        return Weight(W_BF16, w.to(torch.bfloat16))
    if fmt in (W_INT8, W_FP8):
        qmax = 127.0 if fmt == W_INT8 else 448.0
        amax = wf.abs().amax(-1)
        scale = torch.where(amax > 0, _div(amax, qmax), torch.ones_like(amax))
        v = _div(wf, scale.unsqueeze(-1))
        q = torch.round(v).clamp(-127, 127).to(torch.int8) if fmt == W_INT8 else e4m3_bytes(v)
        return Weight(fmt, q, scale)
    K = wf.shape[-1]
    assert wf.dim() == 2 and K % 16 == 0
    amax = wf.abs().max().reshape(1)
    glob = _div(amax, 2688.0)
    blocks = wf.reshape(wf.shape[0], K // 16, 16)
    bmax = blocks.abs().amax(-1)
    s8 = e4m3_bytes(_div(bmax, (6.0 * glob)))
    eff = (s8.view(torch.float8_e4m3fn).float() * glob).unsqueeze(-1)
    live = eff > 0
    ratio = _div(blocks, torch.where(live, eff, torch.ones_like(eff)))
    codes = torch.where(live, e2m1_codes(ratio).int(), 0).to(torch.uint8).reshape(wf.shape)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).contiguous()
    return Weight(W_NVFP4, packed, s8, glob.item())


def quantize_act_reference(x, math):
    """Per-token activation quantisation by the contract's rules (engine/cuda/kernels.h:479-493), restated in torch
    with IEEE f32 operations: INT8 q = rne(x * (127 / a)), FP8 q = e4m3(x * (448 / a)), FP4 g = a / 2688,
    s_b = e4m3(a_b / (6 g)), code = e2m1(x * (1 / (s_b g))). Returns (q bytes, scale f32 [M], block scales or None).
    The reference's own tests derive the same three tensors this way (tests/kernels/wformats.py)."""
    xf = x.float().cpu()
    a = xf.abs().amax(-1)
    live = a > 0
    safe = torch.where(live, a, torch.ones_like(a))
    if math in (1, 2):
        qmax = 127.0 if math == 1 else 448.0
        inv = torch.where(live, _div(qmax, safe), torch.zeros_like(a))
        v = xf * inv.unsqueeze(-1)
        q = torch.round(v).clamp(-127, 127).to(torch.int8).view(torch.uint8) if math == 1 else e4m3_bytes(v)
        return q, torch.where(live, _div(safe, qmax), torch.ones_like(a)), None
    M, K = xf.shape
    assert K % 16 == 0
    g = torch.where(live, _div(safe, 2688.0), torch.ones_like(a))
    blocks = xf.reshape(M, K // 16, 16)
    bmax = blocks.abs().amax(-1)
    s8 = e4m3_bytes(_div(bmax, (6.0 * g).unsqueeze(-1)))
    d = s8.view(torch.float8_e4m3fn).float() * g.unsqueeze(-1)
    on = d > 0
    r = torch.where(on, _div(1.0, torch.where(on, d, torch.ones_like(d))), torch.zeros_like(d))
    codes = torch.where(on.unsqueeze(-1), e2m1_codes(blocks * r.unsqueeze(-1)).int(), 0).to(torch.uint8).reshape(M, K)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).contiguous()
    return packed, g, s8


def alloc_quantized(fmt, N, K, device):
    """Empty buffers of the right sizes for lx_quantize_weight to fill."""
    if fmt == W_INT8:
        return Weight(fmt, torch.empty(N, K, dtype=torch.int8, device=device), torch.empty(N, dtype=torch.float32, device=device))
    if fmt == W_FP8:
        return Weight(fmt, torch.empty(N, K, dtype=torch.uint8, device=device), torch.empty(N, dtype=torch.float32, device=device))
    if fmt == W_NVFP4:
        return Weight(fmt, torch.empty(N, K // 2, dtype=torch.uint8, device=device),
                      torch.empty(N, K // 16, dtype=torch.uint8, device=device))
    raise ValueError(fmt)


def quantize_with(lx, w_bf16, fmt):
    """Quantises bf16 [N, K] with the backend library `lx` (lx_quantize_weight); returns the Weight."""
    import ctypes

    if fmt == W_BF16:
        return Weight(W_BF16, w_bf16)
    N, K = w_bf16.shape
    out = alloc_quantized(fmt, N, K, w_bf16.device)
    s = out.lx()
    lx("quantize_weight", w_bf16, ctypes.pointer(s), ctypes.c_int64(N), K)
    out.glob = float(s.global_)
    return out
