"""GPU: lx_moe_experts_noalloc, the form of lx_moe_experts for callers that cannot allocate (its workspace is a fixed
array in device memory), through the C ABI against lx_moe_experts on the same inputs: the same kernels, so the same
bits. Two calls in a row share the array, the second with a smaller input; a shape beyond the array is refused."""

import pytest
import torch

import checks
import ops

pytestmark = pytest.mark.gpu


def call(hip, entry, latent, ids, weights, gate_up, down, I, top_k):
    T, L = latent.shape
    out = torch.full((T, L), float("nan"), device="cuda")
    hip(entry, latent, ids, weights, gate_up, down, out, T, L, I, top_k)
    return out


def test_noalloc_entry_equals_the_allocating_one(hip):
    E, L, I, top_k = 64, 1024, 512, 4
    g = torch.Generator().manual_seed(77)
    gate_up = (torch.randn(E, 2 * I, L, generator=g) / L**0.5).to(torch.bfloat16).cuda()
    down = (torch.randn(E, L, I, generator=g) / I**0.5).to(torch.bfloat16).cuda()
    for T in (48, 5):  # the second call finds the first one's tables and rows in the array
        latent, ids, weights = (t.cuda() for t in checks.make_routing(T, E, L, top_k, 100 + T))
        want = call(hip, "moe_experts", latent, ids, weights, gate_up, down, I, top_k)
        got = call(hip, "moe_experts_noalloc", latent, ids, weights, gate_up, down, I, top_k)
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), f"T={T}: differs from lx_moe_experts"
        ref = ops.experts_reference(latent.cpu(), ids.cpu(), weights.cpu(), gate_up.cpu().double(), down.cpu().double())
        checks.experts_close(got, ref)


def test_noalloc_entry_refuses_what_the_array_cannot_hold(hip):
    # 4096 pairs of 4096 f32 outputs alone are 64 MiB: beyond the 8 MiB array. Nothing is launched.
    T, L, I, top_k = 1024, 4096, 512, 4
    x = torch.zeros(8, device="cuda")
    out = torch.full((8,), 7.0, device="cuda")
    assert hip.status("moe_experts_noalloc", x, x, x, x, x, out, T, L, I, top_k) == 1
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())
    assert hip.status("moe_experts_noalloc", x, x, x, x, x, out, 0, L, I, top_k) == 0
