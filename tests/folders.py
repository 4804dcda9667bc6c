"""Synthetic model folders in the three on-disk layouts the loader reads (engine/core/checkpoint.cpp:1-32): bf16;
compressed-tensors FP8 (F8_E4M3 weights, an F32 weight_scale per row); GPTQ NVFP4 (U8 nibble pairs, an e4m3 weight_scale
per 16 values, an F32 weight_scale_2 per expert, the dense projections FP8). The quantised bytes come from the
quantisation rules restated in torch (dromos_amd.formats.quantize_reference), not from the library under test."""

import json
from pathlib import Path

import torch
from safetensors.torch import save_file

from dromos_amd.abi import W_FP8, W_NVFP4
from dromos_amd.formats import quantize_reference

V, H, L, I, E = 96, 128, 64, 48, 3  # vocabulary, hidden, latent, expert intermediate, experts


def masters(seed=11):
    """bf16 masters of a toy model: name -> tensor. Projections and plain tensors alike."""
    g = torch.Generator().manual_seed(seed)
    r = lambda *shape: (torch.randn(*shape, generator=g) * 0.05).to(torch.bfloat16)  # noqa: E731
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


def tensors_of(layout, seed=11):
    """name -> tensor as the folder of that layout stores it ("bf16", "fp8", "nvfp4")."""
    m = masters(seed)
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
        elif layout == "nvfp4" and (key in PROJECTIONS or key == "embedding") and not key.endswith(("out_proj", "latent_up")):
            out[name], out[key + ".weight_scale"] = _fp8(w)  # the dense projections and the tied head are FP8 there
        else:
            out[name] = w
    return out


def write(directory, layout, seed=11, shards=1):
    directory = Path(directory)
    directory.mkdir(parents=True, exist_ok=True)
    tensors = {k: v.contiguous() for k, v in tensors_of(layout, seed).items()}
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
