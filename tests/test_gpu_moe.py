"""GPU parity: routing and the decode experts through the C ABI, against float64 statements, the reference
tests' edge cases, and the CPU oracle on the same seeded inputs."""

import pytest
import torch

import checks
import ops
from conftest import close, rel_l2
from dromos_amd.abi import FORMATS, W_BF16, W_NVFP4
from dromos_amd.formats import random_stack

pytestmark = pytest.mark.gpu
FMT = checks.FMT_NAMES


@pytest.mark.parametrize("E,T,top_k", [(128, 1, 4), (128, 7, 4), (128, 300, 4), (192, 1, 4), (192, 300, 4), (64, 64, 8), (128, 32, 8),
                                       (5, 3, 2), (37, 7, 3), (7, 2, 7), (64, 1, 1), (1024, 9, 8)])
def test_route(hip, E, T, top_k):
    checks.route_case(hip, T, E, top_k, seed=E * 1000 + T)


def test_route_without_bias_and_ties(hip):
    checks.route_case(hip, 33, 128, 4, seed=7, with_bias=False)
    checks.route_ties(hip)


def test_route_matches_the_oracle(hip, oracle):
    g = torch.Generator().manual_seed(3064)
    logits = torch.randn(64, 64, generator=g)
    a, b = ops.route(hip, logits.cuda(), None, 8), ops.route(oracle, logits, None, 8)
    assert torch.equal(a[0].cpu(), b[0])
    for u, v in zip(a[1:], b[1:]):
        close(u, v, atol=1e-5)



@pytest.mark.parametrize("E,top_k", [(64, 8), (40, 8), (128, 8), (200, 6), (256, 64), (512, 8)])
def test_route_picks_on_awkward_values_match_the_oracle(hip, oracle, E, top_k):
    logits, bias = checks.awkward_logits(E, top_k)
    for b in (None, bias):
        checks.same_routes(ops.route(hip, logits.cuda(), None if b is None else b.cuda(), top_k), ops.route(oracle, logits, b, top_k), E)


def test_route_empty_and_invalid(hip):
    logits = torch.zeros(2, 8, device="cuda")
    ids = torch.zeros(2, 2, dtype=torch.int32, device="cuda")
    w = torch.zeros(2, 2, device="cuda")
    h = torch.zeros(2, device="cuda")
    assert hip.status("moe_route", logits, None, ids, w, h, h, 0, 8, 2) == 0
    assert hip.status("moe_route", logits, None, ids, w, h, h, 2, 8, 9) == 1  # top_k > E
    assert hip.status("moe_route", logits, None, ids, w, h, h, 2, 8, 0) == 1


@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("T", [1, 2, 4, 8])
def test_decode_metis_shapes(hip, T, fmt):
    checks.decode_case(hip, fmt, fmt, T, 32, 1024, 512, 4, seed=T * 13)


@pytest.mark.parametrize("T,E,L,I,top_k", [(1, 1, 16, 16, 1), (3, 5, 48, 32, 2), (5, 9, 64, 48, 3), (8, 8, 32, 64, 8), (2, 6, 1024, 16, 4)])
@pytest.mark.parametrize("fmt", FMT)
def test_decode_odd_shapes(hip, T, E, L, I, top_k, fmt):
    checks.decode_case(hip, fmt, fmt, T, E, L, I, top_k, seed=T + E)


@pytest.mark.parametrize("gu_fmt,dn_fmt", [("nvfp4", "fp8"), ("fp8", "nvfp4"), ("int8", "bf16"), ("bf16", "nvfp4")])
def test_decode_mixed_formats(hip, gu_fmt, dn_fmt):
    checks.decode_case(hip, gu_fmt, dn_fmt, 4, 16, 1024, 512, 4, seed=23)


def test_decode_repeated_experts(hip):
    pool = torch.randperm(128, generator=torch.Generator().manual_seed(1))[:6]
    checks.decode_case(hip, "nvfp4", "nvfp4", 8, 128, 1024, 512, 4, seed=33, pool=pool)


def test_decode_expert_repeated_within_a_token(hip):
    # Not what routing produces, but the contract allows it: a group larger than the token count.
    T, E, L, I, top_k = 2, 4, 256, 128, 8
    gu, dn = random_stack(FORMATS["int8"], E, 2 * I, L, 5), random_stack(FORMATS["int8"], E, L, I, 6)
    latent, _, weights = checks.make_routing(T, E, L, top_k, 7)
    ids = torch.tensor([[1, 1, 1, 2, 1, 1, 3, 1], [1, 1, 1, 1, 1, 1, 1, 1]], dtype=torch.int32)
    out = ops.experts_decode(hip, latent.cuda(), ids.cuda(), weights.cuda(), gu.to("cuda"), dn.to("cuda"), I, top_k)
    checks.experts_close(out, ops.experts_reference(latent, ids, weights, gu.dense(), dn.dense()))


@pytest.mark.parametrize("fmt", FMT)
def test_decode_deterministic_and_token_independent(hip, fmt):
    T, E, L, I, top_k = 8, 128, 1024, 512, 4
    gu, dn = random_stack(FORMATS[fmt], E, 2 * I, L, 41).to("cuda"), random_stack(FORMATS[fmt], E, L, I, 42).to("cuda")
    latent, ids, weights = (t.cuda() for t in checks.make_routing(T, E, L, top_k, 43))
    first = ops.experts_decode(hip, latent, ids, weights, gu, dn, I, top_k)
    assert torch.equal(first, ops.experts_decode(hip, latent, ids, weights, gu, dn, I, top_k))
    alone = torch.cat([ops.experts_decode(hip, latent[t : t + 1].contiguous(), ids[t : t + 1].contiguous(),
                                          weights[t : t + 1].contiguous(), gu, dn, I, top_k) for t in range(T)])
    for n in range(1, T + 1):
        out = ops.experts_decode(hip, latent[:n].contiguous(), ids[:n].contiguous(), weights[:n].contiguous(), gu, dn, I, top_k)
        assert torch.equal(out, alone[:n]), f"a token of a T={n} batch differs from the token alone"


def test_decode_rejects_more_than_eight_tokens(hip):
    gu, dn = random_stack(W_BF16, 8, 64, 32, 1).to("cuda"), random_stack(W_BF16, 8, 32, 32, 2).to("cuda")
    latent, ids, weights = (t.cuda() for t in checks.make_routing(9, 8, 32, 2, 3))
    assert ops.experts_decode(hip, latent, ids, weights, gu, dn, 32, 2, status=True) != 0
    assert ops.experts_decode(hip, latent[:0], ids[:0], weights[:0], gu, dn, 32, 2, status=True) == 0


def test_decode_global_is_per_expert(hip):
    T, E, L, I = 1, 4, 1024, 512
    gu, dn = random_stack(W_NVFP4, E, 2 * I, L, 61).to("cuda"), random_stack(W_NVFP4, E, L, I, 62).to("cuda")
    latent, _, _ = checks.make_routing(T, E, L, 2, 63)
    ids = torch.tensor([[1, 3]], dtype=torch.int32, device="cuda")
    weights = torch.tensor([[1.0, 0.0]], device="cuda")
    base = ops.experts_decode(hip, latent.cuda(), ids, weights, gu, dn, I, 2)
    dn.expert_global[3] *= 2.0
    assert torch.equal(ops.experts_decode(hip, latent.cuda(), ids, weights, gu, dn, I, 2), base)
    dn.expert_global[1] *= 2.0
    assert torch.equal(ops.experts_decode(hip, latent.cuda(), ids, weights, gu, dn, I, 2), base * 2.0)


@pytest.mark.parametrize("T", [1, 8])
def test_decode_baseline_config_against_the_oracle(hip, oracle, T):
    # 64 experts of gate/up 2048 -> 1024 and down 1024 -> 2048 in bf16 ~ N(0, 0.02), top-8 routing from
    # softmax over logits ~ N(0, 1): routed on the GPU, experts on the GPU, against the oracle end to end.
    E, L, I, top_k = 64, 2048, 1024, 8
    g = torch.Generator().manual_seed(3000 + T)
    gate_up = (torch.randn(E, 2 * I, L, generator=g) * 0.02).to(torch.bfloat16)
    down = (torch.randn(E, L, I, generator=g) * 0.02).to(torch.bfloat16)
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    ids, weights, _, _ = ops.route(hip, logits.cuda(), None, top_k)
    ids_o, weights_o, _, _ = ops.route(oracle, logits, None, top_k)
    assert torch.equal(ids.cpu(), ids_o)
    from dromos_amd.formats import Weight

    gu, dn = Weight(W_BF16, gate_up), Weight(W_BF16, down)
    out = ops.experts_decode(hip, latent.cuda(), ids, weights, gu.to("cuda"), dn.to("cuda"), I, top_k)
    want = ops.experts_decode(oracle, latent, ids_o, weights_o, gu, dn, I, top_k)
    assert rel_l2(out.cpu(), want) <= 1e-2
    assert rel_l2(out.cpu(), want) <= 2e-3
