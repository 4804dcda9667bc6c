"""GPU parity: lx_moe_experts_grouped (BF16 math on the matrix cores) and lx_moe_experts through the C ABI, against
float64 with the bf16-rounded intermediate at the reference tests' shapes (tests/kernels/test_moe_grouped.py:63-70 of
the reference), against the CPU oracle at the headline decode shape, and the bitwise invariants (token rows that do not
depend on the batch, identical bits from run to run out of a garbage-filled workspace)."""

import pytest
import torch

import checks
import ops
from conftest import close, rel_l2
from dromos_amd.abi import FORMATS, MATH_BF16, MATH_FP4, MATH_FP8, MATH_INT8, W_BF16
from dromos_amd.formats import Weight

pytestmark = pytest.mark.gpu
FMT = checks.FMT_NAMES
SHAPES = [(5, 256, 256, 8, 2), (37, 512, 256, 16, 3), (200, 1024, 512, 128, 4), (96, 1024, 768, 192, 4)]


@pytest.mark.parametrize("T,L,I,E,top_k", SHAPES)
@pytest.mark.parametrize("fmt", FMT)
def test_grouped(hip, fmt, T, L, I, E, top_k):
    checks.grouped_case(hip, fmt, T, L, I, E, top_k, seed=T * 31 + E)


@pytest.mark.parametrize("T", [16, 1024])
@pytest.mark.parametrize("fmt", ["bf16", "int8"])
def test_grouped_skewed(hip, fmt, T):
    # Most tokens on a few experts: tiles of every height next to empty experts, several tiles per expert.
    checks.grouped_case(hip, fmt, T, 1024, 512, 128, 4, seed=T + 1, skew=True)


def test_grouped_odd_shapes_take_the_plain_kernels(hip):
    # L or I that cannot be read 16 bytes at a time.
    checks.grouped_case(hip, "bf16", 19, 72, 36, 6, 2, seed=3)
    checks.grouped_case(hip, "int8", 11, 48, 40, 5, 3, seed=4)


def make(fmt, T, L, I, E, top_k, seed):
    g = torch.Generator().manual_seed(seed)
    gu = checks.quantize_reference_stack(torch.randn(E, 2 * I, L, generator=g) / L**0.5, FORMATS[fmt]).to("cuda")
    dn = checks.quantize_reference_stack(torch.randn(E, L, I, generator=g) / I**0.5, FORMATS[fmt]).to("cuda")
    latent, ids, weights = checks.make_routing(T, E, L, top_k, seed + 1)
    return latent.cuda(), ids.cuda(), weights.cuda(), gu, dn


def test_nvfp4_block_scales_read_either_way_give_the_same_bits(hip):
    # Block scales are read eight bytes at a time where every row's lie eight-byte aligned and rows are whole load
    # steps (128 values), two bytes at a time otherwise: the same stacks two bytes off, and rows of 2.25 and 1.25 steps.
    L, I, E, top_k = 1024, 512, 16, 4
    latent, ids, weights, gu, dn = make("nvfp4", 40, L, I, E, top_k, 5)
    want = ops.experts_grouped(hip, latent, ids, weights, gu, dn, I, E, top_k)

    def shifted(w):
        flat = torch.zeros(w.scale.numel() * w.scale.element_size() + 8, dtype=torch.uint8, device="cuda")
        view = flat[2 : 2 + w.scale.numel() * w.scale.element_size()].view(w.scale.dtype).view(w.scale.shape)
        view.copy_(w.scale)
        assert view.data_ptr() % 8 == 2
        return Weight(w.fmt, w.data, view, w.glob, w.expert_global)

    got = ops.experts_grouped(hip, latent, ids, weights, shifted(gu), shifted(dn), I, E, top_k)
    assert torch.equal(got, want)
    checks.grouped_case(hip, "nvfp4", 23, 288, 160, 8, 2, seed=9)


@pytest.mark.parametrize("fmt", FMT)
def test_rows_do_not_depend_on_the_batch(hip, fmt):
    L, I, E, top_k = 1024, 512, 32, 4
    latent, ids, weights, gu, dn = make(fmt, 40, L, I, E, top_k, 77)
    full = ops.experts_grouped(hip, latent, ids, weights, gu, dn, I, E, top_k)
    for t in (0, 3, 17, 39):
        alone = ops.experts_grouped(hip, latent[t : t + 1].contiguous(), ids[t : t + 1].contiguous(),
                                    weights[t : t + 1].contiguous(), gu, dn, I, E, top_k)
        assert torch.equal(alone[0], full[t]), f"token {t} alone differs from the token in a batch of 40"
    for T in range(1, 9):
        out = ops.experts_grouped(hip, latent[:T].contiguous(), ids[:T].contiguous(), weights[:T].contiguous(), gu, dn, I, E, top_k)
        assert torch.equal(out, full[:T]), f"T={T}"


@pytest.mark.parametrize("fmt", ["bf16", "nvfp4"])
@pytest.mark.parametrize("skew", [False, True])
def test_repeats_bit_for_bit(hip, fmt, skew):
    T, L, I, E, top_k = 1024, 1024, 512, 128, 8
    g = torch.Generator().manual_seed(91)
    latent, ids, weights, gu, dn = make(fmt, T, L, I, E, top_k, 91)
    if skew:
        noise = torch.rand(T, E, generator=g)
        hot = torch.randperm(E, generator=g)[:8]
        noise[:, hot] += 10.0 * (torch.rand(T, 1, generator=g) < 0.9)
        ids = noise.argsort(-1, descending=True)[:, :top_k].to(torch.int32).contiguous().cuda()
    first = ops.experts_grouped(hip, latent, ids, weights, gu, dn, I, E, top_k)
    for _ in range(3):
        assert torch.equal(ops.experts_grouped(hip, latent, ids, weights, gu, dn, I, E, top_k), first)


def test_empty_invalid_and_other_maths(hip):
    latent, ids, weights, gu, dn = make("bf16", 4, 256, 256, 8, 2, 1)
    assert ops.experts_grouped(hip, latent[:0], ids[:0], weights[:0], gu, dn, 256, 8, 2, status=True) == 0
    import ctypes

    fn = hip.lib.lx_moe_grouped_workspace_bytes
    fn.restype = ctypes.c_int64
    assert fn(0, 256, 256, 8, 2, 0) == 0 and fn(4, 256, 256, 8, 2, 0) >= 2 * 4 * 2 * 256
    for math in (MATH_INT8, MATH_FP8, MATH_FP4):
        assert ops.experts_grouped(hip, latent, ids, weights, gu, dn, 256, 8, 2, math=math, status=True) == 801
    assert ops.experts_grouped(hip, latent, ids, weights, gu, dn, 256, 0, 2, status=True) == 1


@pytest.mark.parametrize("T", [1, 7, 300])
def test_moe_experts_bf16_entry(hip, T):
    E, L, I, top_k = 128, 1024, 512, 4
    g = torch.Generator().manual_seed(E * 1000 + T)
    gate_up = (torch.randn(E, 2 * I, L, generator=g) / L**0.5).to(torch.bfloat16)
    down = (torch.randn(E, L, I, generator=g) / I**0.5).to(torch.bfloat16)
    latent, ids, weights = checks.make_routing(T, E, L, top_k, T)
    out = ops.experts_bf16(hip, latent.cuda(), ids.cuda(), weights.cuda(), gate_up.cuda(), down.cuda(), I, top_k)
    want = ops.experts_reference(latent, ids, weights, gate_up.double(), down.double())
    close(out, want, atol=1e-3 * want.abs().max().item(), rtol=1e-3)


@pytest.mark.parametrize("T", [32, 64])
def test_baseline_config_against_the_oracle(hip, oracle, T):
    E, L, I, top_k = 64, 2048, 1024, 8
    g = torch.Generator().manual_seed(3000 + T)
    gu = Weight(W_BF16, (torch.randn(E, 2 * I, L, generator=g) * 0.02).to(torch.bfloat16))
    dn = Weight(W_BF16, (torch.randn(E, L, I, generator=g) * 0.02).to(torch.bfloat16))
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    ids, weights, _, _ = ops.route(hip, logits.cuda(), None, top_k)
    ids_o, weights_o, _, _ = ops.route(oracle, logits, None, top_k)
    assert torch.equal(ids.cpu(), ids_o)
    out = ops.experts_grouped(hip, latent.cuda(), ids, weights, gu.to("cuda"), dn.to("cuda"), I, E, top_k)
    want = ops.experts_grouped(oracle, latent, ids_o, weights_o, gu, dn, I, E, top_k)
    err = rel_l2(out.cpu(), want)
    assert err <= 1e-2 and err <= 2e-3, err


# ---- the quantised maths: latent rows quantised per token, the intermediate per pair, both by lx_quantize_act's rule --

GROUPED_MATHS = [("int8", MATH_INT8), ("fp8", MATH_FP8), ("nvfp4", MATH_FP8), ("nvfp4", MATH_FP4)]


@pytest.mark.parametrize("fmt,math", GROUPED_MATHS)
@pytest.mark.parametrize("T,L,I,E,top_k", [(5, 256, 256, 8, 2), (37, 512, 256, 16, 3), (96, 1024, 768, 64, 4)])
def test_grouped_under_a_math_against_the_oracle(hip, oracle, fmt, math, T, L, I, E, top_k):
    g = torch.Generator().manual_seed(T * 31 + E + math)
    gu = checks.quantize_reference_stack(torch.randn(E, 2 * I, L, generator=g) / L**0.5, FORMATS[fmt])
    dn = checks.quantize_reference_stack(torch.randn(E, L, I, generator=g) / I**0.5, FORMATS[fmt])
    latent, ids, weights = checks.make_routing(T, E, L, top_k, T + 1)
    want = ops.experts_grouped(oracle, latent, ids, weights, gu, dn, I, E, top_k, math=math)
    got = ops.experts_grouped(hip, latent.cuda(), ids.cuda(), weights.cuda(), gu.to("cuda"), dn.to("cuda"), I, E, top_k, math=math)
    # The device's exp and f32 sums differ from the oracle's in last bits; where that moves a bf16 intermediate value it
    # can move its quantised code too (the coarser the math, the further): a tolerance, not bits.
    err = rel_l2(got, want)
    assert err <= 1e-2 and err <= (1e-2 if math == MATH_FP4 else 3e-3), err


@pytest.mark.parametrize("fmt,math", GROUPED_MATHS)
def test_grouped_under_a_math_rows_do_not_depend_on_the_batch(hip, fmt, math):
    L, I, E, top_k = 1024, 512, 32, 4
    latent, ids, weights, gu, dn = make(fmt, 40, L, I, E, top_k, 77)
    full = ops.experts_grouped(hip, latent, ids, weights, gu, dn, I, E, top_k, math=math)
    assert torch.equal(ops.experts_grouped(hip, latent, ids, weights, gu, dn, I, E, top_k, math=math), full)
    for t in (0, 17, 39):
        alone = ops.experts_grouped(hip, latent[t : t + 1].contiguous(), ids[t : t + 1].contiguous(),
                                    weights[t : t + 1].contiguous(), gu, dn, I, E, top_k, math=math)
        assert torch.equal(alone[0], full[t]), f"token {t} alone differs from the token in a batch of 40"


def test_grouped_maths_and_formats_that_do_not_pair(hip):
    from dromos_amd.formats import random_stack

    T, E, L, I, top_k = 2, 4, 64, 32, 2
    latent, ids, weights = (t.cuda() for t in checks.make_routing(T, E, L, top_k, 1))
    for fmt, math, want in [("int8", 2, 801), ("fp8", 1, 801), ("bf16", 3, 801), ("nvfp4", 1, 801), ("fp8", 3, 801), ("nvfp4", 3, 0),
                            ("int8", 1, 0), ("fp8", 2, 0), ("nvfp4", 2, 0), ("bf16", 7, 1)]:
        gu, dn = random_stack(FORMATS[fmt], E, 2 * I, L, 3).to("cuda"), random_stack(FORMATS[fmt], E, L, I, 4).to("cuda")
        assert ops.experts_grouped(hip, latent, ids, weights, gu, dn, I, E, top_k, math=math, status=True) == want, (fmt, math)
