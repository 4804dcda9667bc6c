"""Synthetic model folders in the three on-disk layouts the loader reads (engine/core/checkpoint.cpp:1-32): bf16;
compressed-tensors FP8 (F8_E4M3 weights, an F32 weight_scale per row); GPTQ NVFP4 (U8 nibble pairs, an e4m3 weight_scale
per 16 values, an F32 weight_scale_2 per expert, the dense projections FP8). The quantised bytes come from the
quantisation rules restated in torch (dromos_amd.formats.quantize_reference), not from the library under test."""

import hashlib
import json
from pathlib import Path

import torch
from safetensors.torch import save_file

from dromos_amd.abi import W_FP8, W_NVFP4
from dromos_amd.formats import quantize_reference

V, H, L, I, E = 96, 128, 64, 48, 3  # vocabulary, hidden, latent, expert intermediate, experts


def masters(seed=11, wide=False):
    """bf16 masters of a toy model: name -> tensor. Projections and plain tensors alike. `wide` adds a second layer
    that carries every other projection name the loader's recipe knows (engine/core/checkpoint.cpp:99-116)."""
    g = torch.Generator().manual_seed(seed)
    r = lambda *shape: (torch.randn(*shape, generator=g) * 0.05).to(torch.bfloat16)  # noqa: E731
    m = _toy(r, g)
    if wide:
        m.update({
            "layers.1.norm.weight": r(H),
            "layers.1.mixer.qkv.weight": r(3 * H, H),
            "layers.1.mixer.out.weight": r(H, H),
            "layers.1.mixer.pass_lora_down.weight": r(16, H),
            "layers.1.mixer.pass_lora_up.weight": r(3 * H, 16),
            "layers.1.moe.latent_down.weight": r(L, H),
            "layers.1.moe.latent_up.weight": r(H, L),
            "layers.1.moe.shared_expert.gate_up.weight": r(2 * 64, H),
            "layers.1.moe.shared_expert.down.weight": r(H, 64),
            "layers.1.moe.router.weight": torch.randn(E, H, generator=g),
            "layers.1.moe.router.bias": torch.randn(E, generator=g),
            "layers.1.moe.local_experts.gate_up.weight": r(E, 2 * I, L),
            "layers.1.moe.local_experts.down.weight": r(E, L, I),
            "layers.1.depth_memory.query.weight": r(H, H),
            "layers.1.depth_memory.state_write.weight": r(H, H),
            "layers.1.depth_memory.output.weight": r(H, H),
            "layers.1.depth_memory.route_projection.weight": r(32, H),
            "layers.1.depth_memory.key.weight": r(H, H),
            "layers.1.depth_memory.value.weight": r(H, H),
            "layers.1.depth_memory.metadata_write.weight": r(H, 32),
        })
    return m


def _toy(r, g):
    return {
        "embedding.weight": r(V, H),
        "layers.0.norm.weight": r(H),
        "layers.0.mixer.qkv.weight": r(3 * H, H),
        "layers.0.mixer.out.weight": r(H, H),
        "layers.0.mixer.impl.mixer.in_proj.weight": r(2 * H, H),
        "layers.0.mixer.impl.mixer.out_proj.weight": r(H, H),
        "layers.0.moe.latent_down.weight": r(L, H),
        "layers.0.moe.latent_up.weight": r(H, L),
        "layers.0.moe.router.weight": torch.randn(E, H, generator=g),  # f32, plain
        "layers.0.moe.local_experts.gate_up.weight": r(E, 2 * I, L),
        "layers.0.moe.local_experts.down.weight": r(E, L, I),
        "layers.0.depth_memory.key.weight": r(H, H),
        "final_norm.bias": torch.randn(H, generator=g),
    }


PROJECTIONS = ["layers.0.mixer.qkv", "layers.0.mixer.out", "layers.0.mixer.impl.mixer.in_proj", "layers.0.mixer.impl.mixer.out_proj",
               "layers.0.moe.latent_down", "layers.0.moe.latent_up", "layers.0.moe.local_experts.gate_up",
               "layers.0.moe.local_experts.down", "layers.0.depth_memory.key"]
PLAIN = ["embedding.weight", "layers.0.norm.weight", "layers.0.moe.router.weight", "final_norm.bias"]
_NOT_PROJECTIONS = ("norm.weight", "router.weight", "router.bias", "final_norm.bias", "embedding.weight")


def projections(wide=False):
    """The projection keys (names without ".weight") of the toy model, or of its wide form."""
    if not wide:
        return list(PROJECTIONS)
    return [n[: -len(".weight")] for n in masters(wide=True) if not n.endswith(_NOT_PROJECTIONS)]


def plain(wide=False):
    return [n for n in masters(wide=wide) if n.endswith(_NOT_PROJECTIONS)]


def _fp8(w):
    """(F8_E4M3 data, F32 scale per row) of a bf16 matrix or stack."""
    rows = w.reshape(-1, w.shape[-1])
    q = quantize_reference(rows, W_FP8)
    return q.data.view(torch.float8_e4m3fn).reshape(w.shape), q.scale.reshape(w.shape[:-1]).contiguous()


def _nvfp4(w):
    """(U8 data, e4m3 block scales, F32 global per expert or scalar) of a bf16 matrix or stack."""
    stack = w.dim() == 3
    datas, scales, globals_ = [], [], []
    for m in (w if stack else [w]):
        q = quantize_reference(m, W_NVFP4)
        datas.append(q.data), scales.append(q.scale.view(torch.float8_e4m3fn)), globals_.append(q.glob)
    if stack:
        return torch.stack(datas), torch.stack(scales), torch.tensor(globals_, dtype=torch.float32)
    return datas[0], scales[0], torch.tensor(globals_[0], dtype=torch.float32)


def tensors_of(layout, seed=11, wide=False):
    """name -> tensor as the folder of that layout stores it ("bf16", "fp8", "nvfp4"): which projections the published
    FP8 and NVFP4 folders quantise is told by tests/unit/checkpoint_test.cpp:137-176 of the reference."""
    m = masters(seed, wide)
    every = projections(wide)
    if layout == "bf16":
        return m
    out = {}
    fp8_parts = ("mixer.qkv", "mixer.out", "mixer.impl.mixer.in_proj", "local_experts.gate_up", "local_experts.down")
    for name, w in m.items():
        key = name[: -len(".weight")] if name.endswith(".weight") else name
        if layout == "fp8" and key.endswith(fp8_parts):
            out[name], out[key + ".weight_scale"] = _fp8(w)
        elif layout == "nvfp4" and "local_experts." in key:
            out[name], out[key + ".weight_scale"], out[key + ".weight_scale_2"] = _nvfp4(w)
        elif layout == "nvfp4" and (key in every or key == "embedding") and not key.endswith(
                ("out_proj", "latent_up", "pass_lora_down", "pass_lora_up", "metadata_write")):
            out[name], out[key + ".weight_scale"] = _fp8(w)  # the dense projections and the tied head are FP8 there
        else:
            out[name] = w
    return out


def write(directory, layout, seed=11, shards=1, wide=False):
    directory = Path(directory)
    directory.mkdir(parents=True, exist_ok=True)
    tensors = {k: v.contiguous() for k, v in tensors_of(layout, seed, wide).items()}
    if shards == 1:
        save_file(tensors, str(directory / "model.safetensors"))
        return tensors
    names = sorted(tensors)
    weight_map = {}
    for s in range(shards):
        part = {n: tensors[n] for n in names[s::shards]}
        fname = f"model-{s + 1:05d}-of-{shards:05d}.safetensors"
        save_file(part, str(directory / fname))
        weight_map.update({n: fname for n in part})
    (directory / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": weight_map}))
    return tensors


def digest(tensors):
    """One SHA-256 over a folder's tensors in name order (name, dtype, shape, bytes): tells whether two folders are the
    same data, whatever wrote them."""
    h = hashlib.sha256()
    for name in sorted(tensors):
        t = tensors[name].contiguous()
        h.update(f"{name}|{t.dtype}|{tuple(t.shape)}|".encode())
        h.update(t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    return h.hexdigest()
