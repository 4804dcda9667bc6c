"""Pins the oracle's routing and routed experts: routing against a stable sort of the f32 biased logits and
float64 softmax statistics (ids exact), tie cases from the reference's tests, the experts against float64 with the
bf16-rounded intermediate, and both against the reference's CPU backend where it was built."""

import pytest
import torch

import checks
import ops
from conftest import close, rel_l2
from dromos_amd.abi import FORMATS
from dromos_amd.formats import random_stack

FMT = checks.FMT_NAMES


@pytest.mark.parametrize("E,T,top_k", [(128, 1, 4), (128, 7, 4), (192, 300, 4), (64, 8, 8), (5, 3, 2), (37, 7, 3), (7, 2, 7), (64, 1, 1)])
def test_route(oracle, E, T, top_k):
    checks.route_case(oracle, T, E, top_k, seed=E * 1000 + T)


def test_route_without_bias_and_ties(oracle):
    checks.route_case(oracle, 33, 128, 4, seed=7, with_bias=False)
    checks.route_ties(oracle)


@pytest.mark.parametrize("E,top_k", [(64, 8), (40, 8), (128, 8), (200, 6), (256, 64), (512, 8)])
def test_route_on_awkward_values_equals_the_reference_backend(oracle, ref, E, top_k):
    logits, bias = checks.awkward_logits(E, top_k)
    for b in (None, bias):
        checks.same_routes(ops.route(oracle, logits, b, top_k), ops.route(ref, logits, b, top_k), E)


def test_route_equals_the_reference_backend(oracle, ref):
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(64, 128, generator=g) * 2
    bias = torch.randn(128, generator=g) * 0.5
    a, b = ops.route(oracle, logits, bias, 8), ops.route(ref, logits, bias, 8)
    for u, v in zip(a, b):
        assert torch.equal(u, v)  # same libm, same order: bit for bit


@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("T", [1, 4, 8])
def test_decode_experts(oracle, fmt, T):
    checks.decode_case(oracle, fmt, fmt, T, 16, 256, 128, 4, seed=T * 13)


@pytest.mark.parametrize("T,E,L,I,top_k", [(1, 1, 16, 16, 1), (3, 5, 48, 32, 2), (5, 9, 64, 48, 3), (8, 8, 32, 64, 8)])
@pytest.mark.parametrize("fmt", FMT)
def test_decode_experts_odd_shapes(oracle, fmt, T, E, L, I, top_k):
    checks.decode_case(oracle, fmt, fmt, T, E, L, I, top_k, seed=T + E)


def test_decode_experts_mixed_formats_and_repeats(oracle):
    checks.decode_case(oracle, "nvfp4", "fp8", 4, 16, 256, 128, 4, seed=23)
    checks.decode_case(oracle, "int8", "bf16", 4, 16, 256, 128, 4, seed=24)
    pool = torch.tensor([3, 9, 17, 21, 40, 55])
    checks.decode_case(oracle, "nvfp4", "nvfp4", 8, 64, 256, 128, 4, seed=33, pool=pool)


def test_decode_rejects_more_than_eight_tokens(oracle):
    gu, dn = random_stack(0, 8, 64, 32, 1), random_stack(0, 8, 32, 32, 2)
    latent, ids, weights = checks.make_routing(9, 8, 32, 2, 3)
    assert ops.experts_decode(oracle, latent, ids, weights, gu, dn, 32, 2, status=True) != 0


@pytest.mark.parametrize("fmt", FMT)
def test_grouped_experts(oracle, fmt):
    checks.grouped_case(oracle, fmt, 37, 128, 64, 16, 3, seed=31)


@pytest.mark.parametrize("fmt", FMT)
def test_experts_equal_the_reference_generic_level(oracle, ref, fmt):
    # Same grouping, same f32 sums (generic level), same libm exp in silu: every output bit agrees.
    ref.lib.lx_set_arch_override(1)
    try:
        T, E, L, I, top_k = 6, 12, 256, 128, 4
        gu, dn = random_stack(FORMATS[fmt], E, 2 * I, L, 71), random_stack(FORMATS[fmt], E, L, I, 72)
        latent, ids, weights = checks.make_routing(T, E, L, top_k, 73)
        a = ops.experts_decode(oracle, latent, ids, weights, gu, dn, I, top_k)
        b = ops.experts_decode(ref, latent, ids, weights, gu, dn, I, top_k)
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
        a = ops.experts_grouped(oracle, latent, ids, weights, gu, dn, I, E, top_k)
        b = ops.experts_grouped(ref, latent, ids, weights, gu, dn, I, E, top_k)
        assert rel_l2(a, b) < 1e-5  # the reference's BF16 math may take its bf16 dot instructions
    finally:
        ref.lib.lx_set_arch_override(0)


GROUPED_MATHS = [("int8", 1), ("fp8", 2), ("nvfp4", 2), ("nvfp4", 3), ("bf16", 0)]


def grouped_math_reference(latent, ids, weights, gu, dn, math):
    """The routed experts under a quantised math from closed forms, in float64: per pair, the token's latent row
    quantised by the per-row rule, gate and up as scale products of exact dots, SwiGLU, the bf16 intermediate quantised
    again per row, down, and the weighted sum."""
    import torch.nn.functional as F

    from dromos_amd.formats import e2m1_table, e4m3_table, quantize_act_reference, unpack_codes

    def values(rows):
        if math == 0:
            return rows.double(), torch.ones(rows.shape[0], dtype=torch.float64)
        q, xs, bs = quantize_act_reference(rows, math)
        if math == 1:
            return q.view(torch.int8).double(), xs.double()
        if math == 2:
            return e4m3_table()[q.long()], xs.double()
        return e2m1_table()[unpack_codes(q).long()] * e4m3_table()[bs.long()].repeat_interleave(16, dim=-1), xs.double()

    I = gu.data.shape[1] // 2
    gd, dd = gu.dense(), dn.dense()
    xv, xs = values(latent)
    out = torch.zeros(latent.shape, dtype=torch.float64)
    for t in range(ids.shape[0]):
        for k in range(ids.shape[1]):
            e = int(ids[t, k])
            g, u = xs[t] * (gd[e, :I] @ xv[t]), xs[t] * (gd[e, I:] @ xv[t])
            mid = (F.silu(g) * u).to(torch.bfloat16)
            mv, ms = values(mid.unsqueeze(0))
            out[t] += weights[t, k].double() * ms[0] * (dd[e] @ mv[0])
    return out


@pytest.mark.parametrize("fmt,math", GROUPED_MATHS)
def test_grouped_experts_under_a_math(oracle, fmt, math):
    T, E, L, I, top_k = 9, 8, 128, 64, 3
    g = torch.Generator().manual_seed(5 + math)
    gu = checks.quantize_reference_stack(torch.randn(E, 2 * I, L, generator=g) / L**0.5, FORMATS[fmt])
    dn = checks.quantize_reference_stack(torch.randn(E, L, I, generator=g) / I**0.5, FORMATS[fmt])
    latent, ids, weights = checks.make_routing(T, E, L, top_k, 6)
    out = ops.experts_grouped(oracle, latent, ids, weights, gu, dn, I, E, top_k, math=math)
    want = grouped_math_reference(latent, ids, weights, gu, dn, math)
    # The intermediate is rounded to bf16 and quantised again: a last-bit difference in a sum can move one of its
    # values by a code, so the comparison with float64 is a tolerance, not bits.
    close(out, want, atol=(2e-2 if math == 3 else 5e-3) * want.abs().max().item())
    assert rel_l2(out, want) <= (3e-2 if math == 3 else 1e-2)


@pytest.mark.parametrize("fmt,math", GROUPED_MATHS)
def test_grouped_experts_under_a_math_equal_the_reference_generic_level(oracle, ref, fmt, math):
    ref.lib.lx_set_arch_override(1)
    try:
        T, E, L, I, top_k = 7, 12, 256, 128, 4
        gu, dn = random_stack(FORMATS[fmt], E, 2 * I, L, 71), random_stack(FORMATS[fmt], E, L, I, 72)
        latent, ids, weights = checks.make_routing(T, E, L, top_k, 73)
        a = ops.experts_grouped(oracle, latent, ids, weights, gu, dn, I, E, top_k, math=math)
        b = ops.experts_grouped(ref, latent, ids, weights, gu, dn, I, E, top_k, math=math)
        if math == 0:
            assert rel_l2(a, b) < 1e-5  # the reference's BF16 math may take its bf16 dot instructions
        else:
            assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    finally:
        ref.lib.lx_set_arch_override(0)


def test_grouped_maths_and_formats_that_do_not_pair(oracle):
    T, E, L, I, top_k = 2, 4, 64, 32, 2
    latent, ids, weights = checks.make_routing(T, E, L, top_k, 1)
    for fmt, math, want in [("int8", 2, 801), ("fp8", 1, 801), ("bf16", 3, 801), ("nvfp4", 1, 801), ("fp8", 3, 801), ("nvfp4", 3, 0),
                            ("int8", 1, 0), ("fp8", 2, 0), ("nvfp4", 2, 0), ("bf16", 7, 1)]:
        gu, dn = random_stack(FORMATS[fmt], E, 2 * I, L, 3), random_stack(FORMATS[fmt], E, L, I, 4)
        assert ops.experts_grouped(oracle, latent, ids, weights, gu, dn, I, E, top_k, math=math, status=True) == want, (fmt, math)
