"""GPU tests of the model-folder loader (lx_ckpt_*): folders in the bf16, compressed-tensors FP8 and GPTQ NVFP4 layouts
loaded for every target, first against the fixture that records what the reference's own loader made of the same
folders (tests/golden/ckpt_reference.json), then rule by rule: a projection held in the file's format has the file's bytes; a converted one has the bytes the
library's own quantiser gives the same bf16 values (the quantisers are pinned bit for bit elsewhere), the lossless target
the bytes of lx_bf16x_encode; the products on the loaded weights run."""

import ctypes
import hashlib
import json
import struct
from pathlib import Path

import pytest
import torch

import folders
import ops
from conftest import rel_l2
from dromos_amd.abi import W_BF16, W_BF16X, W_FP8, W_INT8, W_NVFP4
from dromos_amd.checkpoint import ModelWeights, projection_format
from dromos_amd.formats import Weight, quantize_with

pytestmark = pytest.mark.gpu
STORED = {"bf16": W_BF16, "fp8": W_FP8, "nvfp4": W_NVFP4}


def device_bytes(ptr, n):
    """n bytes at a device address, as a CPU uint8 tensor (copied with lx_rt_copy)."""
    import dromos_amd.abi as abi

    out = torch.empty(n, dtype=torch.uint8, device="cuda")
    lib = ctypes.CDLL(str(abi.hip_library_path()))
    assert lib.lx_rt_copy(ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(ptr), ctypes.c_int64(n), 2, None) == 0  # device to device
    torch.cuda.synchronize()
    return out.cpu()


def stored_as_weight(tensors, key):
    """The file's tensors of a projection as a Weight of the file's format (CPU), and that format."""
    w = tensors[key + ".weight"]
    if w.dtype == torch.bfloat16:
        return Weight(W_BF16, w), W_BF16
    if w.dtype == torch.float8_e4m3fn:
        return Weight(W_FP8, w.view(torch.uint8), tensors[key + ".weight_scale"]), W_FP8
    g = tensors[key + ".weight_scale_2"]
    return Weight(W_NVFP4, w, tensors[key + ".weight_scale"].view(torch.uint8), float(g.flatten()[0]), g if g.dim() else None), W_NVFP4


def as_bf16(hip, w, fmt):
    """bf16 values of a stored projection, expert by expert, by the library's dequantiser."""
    if fmt == W_BF16:
        return w.data.cuda()
    data = w.data.cuda()
    lead = data.shape[:-2]
    rows = data.reshape(-1, *data.shape[-2:])
    scales = w.scale.cuda().reshape(rows.shape[0], *w.scale.shape[len(lead):])
    outs = []
    for e in range(rows.shape[0]):
        glob = w.glob if w.expert_global is None else float(w.expert_global[e])
        K = rows.shape[-1] * (2 if fmt == W_NVFP4 else 1)
        outs.append(ops.dequantize(hip, Weight(fmt, rows[e], scales[e], glob), rows.shape[-2], K))
    return torch.stack(outs).reshape(*lead, *outs[0].shape)


GOLDEN = json.loads((Path(__file__).parent / "golden" / "ckpt_reference.json").read_text())
TARGET_OF = {"bf16": W_BF16, "int8": W_INT8, "fp8": W_FP8, "nvfp4": W_NVFP4, "bf16x": W_BF16X}


def sha_of_device(ptr, n):
    return hashlib.sha256(device_bytes(ptr, n).numpy().tobytes()).hexdigest() if n else None


@pytest.mark.parametrize("case", sorted(GOLDEN["cases"]))
def test_the_reference_loaders_formats_and_bytes(hip, tmp_path, case):
    """Against what the reference's own loader (engine/core/checkpoint.cpp, ModelWeights::load, compiled from its sources
    and run over its CPU backend) made of the same folders: every projection's format, shape, data, scale and global
    bytes, the plain tensors, what skip_experts leaves readable, and the refusals' words."""
    want = GOLDEN["cases"][case]
    layout, _, rest = case.partition("->")
    target, skip = TARGET_OF[rest.split()[0]], rest.endswith("skip_experts")
    tensors = folders.write(tmp_path, layout, seed=GOLDEN["seed"], shards=1, wide=GOLDEN["wide"])
    assert folders.digest(tensors) == GOLDEN["inputs"][layout], "this folder is not the one the fixture was made from"
    assert ModelWeights.stored_format(hip, tmp_path) == want["stored"]
    if "error" in want:
        with pytest.raises(RuntimeError) as err:
            ModelWeights.load(hip, tmp_path, target, skip)
        assert str(err.value) == want["error"]
        return
    mw = ModelWeights.load(hip, tmp_path, target, skip)
    assert mw.format() == want["format"]
    assert sorted(mw.projection_names()) == sorted(want["projections"])
    for name, p in want["projections"].items():
        w, shape = mw.projection(name), mw.projection_shape(name)
        assert w is not None and w.type == p["type"] == mw.projection_format(name), name
        assert (shape.E, shape.N, shape.K, int(shape.stack)) == (p["E"], p["N"], p["K"], p["stack"]), name
        assert list(mw.expert_bytes(name)) == p["expert_bytes"], name
        assert sha_of_device(w.data, p["data_bytes"]) == p["data"], name
        assert (w.scale is None) == (p["scale"] is None), name
        if p["scale"]:
            assert sha_of_device(w.scale, p["scale_bytes"]) == p["scale"], name
        assert struct.unpack("<I", struct.pack("<f", w.global_))[0] == p["global_bits"], name
        assert (w.expert_global is None) == (p["globals"] is None), name
        if p["globals"]:
            assert sha_of_device(w.expert_global, 4 * p["E"]) == p["globals"], name
    for name, t in want["plain"].items():
        view = mw.find(name)
        assert view is not None and view.dtype == t["dtype"] and list(view.shape) == t["shape"], name
        n = (2 if t["dtype"] == 1 else 4) * int(torch.tensor(t["shape"]).prod())
        assert sha_of_device(view.data, n) == t["bytes"], name
    for name, p in want["skipped"].items():
        shape = mw.projection_shape(name)
        assert (mw.projection(name) is not None) == bool(p["held"]), name
        assert (shape.E, shape.N, shape.K, int(shape.stack)) == (p["E"], p["N"], p["K"], p["stack"]), name
        assert list(mw.expert_bytes(name)) == p["expert_bytes"], name
    assert mw.device_bytes() == want["device_bytes"]


@pytest.mark.parametrize("layout", ["bf16", "fp8", "nvfp4"])
@pytest.mark.parametrize("target", [W_BF16, W_INT8, W_FP8, W_NVFP4, W_BF16X])
def test_every_layout_for_every_target(hip, tmp_path, layout, target):
    tensors = folders.write(tmp_path, layout, shards=2 if target == W_INT8 else 1)
    if target == W_NVFP4 and layout != "nvfp4":
        # engine/core/checkpoint.cpp:186-197 with no model family known (the loader here reads no config.json)
        said = "NVFP4 from " + ("an FP8" if layout == "fp8" else "a BF16") + " checkpoint is refused: round-to-nearest conversion fails its KL. No NVFP4 checkpoint of this model is published yet."
        with pytest.raises(RuntimeError) as err:
            ModelWeights.load(hip, tmp_path, target)
        assert str(err.value) == said
        return
    mw = ModelWeights.load(hip, tmp_path, target)
    assert mw.format() == target
    assert sorted(mw.projection_names()) == sorted(folders.PROJECTIONS + ["lm_head"])
    own = target == STORED[layout]
    for key in folders.PROJECTIONS:
        w, src = stored_as_weight(tensors, key)
        want_fmt = src if own else projection_format(hip, target, key)
        lw = mw.projection(key)
        shape = mw.projection_shape(key)
        assert lw.type == want_fmt == mw.projection_format(key), key
        full = tensors[key + ".weight"].shape
        assert (shape.E, shape.N) == ((full[0], full[1]) if len(full) == 3 else (1, full[0])) and shape.stack == (len(full) == 3)
        rows = shape.E * shape.N
        if want_fmt == src:
            got = device_bytes(lw.data, w.data.numel() * w.data.element_size())
            assert torch.equal(got, w.data.contiguous().view(torch.uint8).flatten()), key
            if w.scale is not None:
                assert torch.equal(device_bytes(lw.scale, w.scale.numel() * w.scale.element_size()), w.scale.contiguous().view(torch.uint8).flatten())
            continue
        bf16 = as_bf16(hip, w, src).reshape(rows, shape.K)
        if want_fmt == W_BF16:
            assert torch.equal(device_bytes(lw.data, rows * shape.K * 2), bf16.cpu().view(torch.uint8).flatten()), key
        elif want_fmt == W_BF16X:
            enc = ops.bf16x_encode(hip, bf16)
            assert torch.equal(device_bytes(lw.data, enc.numel()), enc.cpu()), key
        else:
            for e in range(shape.E):
                q = quantize_with(hip, bf16[e * shape.N:(e + 1) * shape.N].contiguous(), want_fmt)
                part = mw.projection_expert(key, e)
                assert torch.equal(device_bytes(part.data, q.data.numel() * q.data.element_size()), q.data.cpu().view(torch.uint8).flatten()), (key, e)
                assert torch.equal(device_bytes(part.scale, q.scale.numel() * q.scale.element_size()), q.scale.cpu().view(torch.uint8).flatten()), (key, e)
    # plain tensors, as they are; the gather table is bf16 whatever the folder holds
    for name in folders.PLAIN:
        view = mw.find(name)
        assert view is not None, name
        t = tensors[name]
        if name == "embedding.weight" and t.dtype != torch.bfloat16:
            w, src = stored_as_weight(tensors, "embedding")
            t = as_bf16(hip, w, src).cpu()
        assert view.shape == tuple(t.shape) and view.dtype == (1 if t.dtype == torch.bfloat16 else 0)
        assert torch.equal(device_bytes(view.data, t.numel() * t.element_size()), t.contiguous().view(torch.uint8).flatten()), name
    assert mw.find("layers.0.mixer.qkv.weight") is None and mw.find("layers.0.mixer.qkv.weight_scale") is None
    # the tied head: from the recipe (or the folder's own format), on the gather table's values
    head = mw.projection("lm_head")
    w, src = stored_as_weight(tensors, "embedding")
    head_fmt = src if own else projection_format(hip, target, "embedding")
    assert head.type == head_fmt
    if head_fmt == W_BF16:
        assert head.data == mw.find("embedding.weight").data
    assert mw.peak_device_bytes() >= mw.device_bytes() > 0
    if own and tensors["embedding.weight"].dtype == torch.bfloat16:  # nothing is converted: no scratch was taken
        assert mw.peak_device_bytes() == mw.device_bytes()
    mw.close()


@pytest.mark.parametrize("layout,target", [("bf16", W_INT8), ("fp8", W_FP8), ("nvfp4", W_NVFP4), ("bf16", W_BF16X), ("fp8", W_BF16X)])
def test_products_on_loaded_weights(hip, oracle, tmp_path, layout, target):
    tensors = folders.write(tmp_path, layout)
    mw = ModelWeights.load(hip, tmp_path, target)
    g = torch.Generator().manual_seed(3)
    # a dense projection through lx_gemv_w
    key = "layers.0.mixer.qkv"
    shape = mw.projection_shape(key)
    x = torch.randn(2, shape.K, generator=g).to(torch.bfloat16).cuda()
    y = torch.full((2, shape.N), float("nan"), device="cuda")
    lw = mw.projection(key)
    hip("gemv_w", x, 1, shape.K, ctypes.pointer(lw), None, 0, y, 0, shape.N, 2, shape.N, shape.K, 1.0, 0.0)
    w, src = stored_as_weight(tensors, key)
    want = x.double().cpu() @ as_bf16(hip, w, src).double().cpu().T
    assert rel_l2(y, want) <= (2e-2 if lw.type in (W_INT8, W_FP8) else 1e-5)
    # the routed experts through lx_moe_experts_decode, and an expert of the stack on its own
    gu, dn = mw.projection("layers.0.moe.local_experts.gate_up"), mw.projection("layers.0.moe.local_experts.down")
    T, top_k = 3, 2
    latent = torch.randn(T, folders.L, generator=g).to(torch.bfloat16).cuda()
    ids = torch.tensor([[0, 2], [1, 0], [2, 1]], dtype=torch.int32, device="cuda")
    weights = torch.softmax(torch.randn(T, top_k, generator=g), -1).cuda()
    ws = torch.empty(int(hip.size("moe_decode_workspace_bytes", T, folders.I, top_k)), dtype=torch.uint8, device="cuda")
    out = torch.full((T, folders.L), float("nan"), device="cuda")
    hip("moe_experts_decode", latent, ids, weights, ctypes.pointer(gu), ctypes.pointer(dn), out, ws, T, folders.L, folders.I, top_k)
    gw, gsrc = stored_as_weight(tensors, "layers.0.moe.local_experts.gate_up")
    dw, dsrc = stored_as_weight(tensors, "layers.0.moe.local_experts.down")
    want = ops.experts_reference(latent.cpu(), ids.cpu(), weights.cpu(), as_bf16(hip, gw, gsrc).double().cpu(), as_bf16(hip, dw, dsrc).double().cpu())
    assert rel_l2(out, want) <= (5e-2 if gu.type in (W_INT8, W_FP8, W_NVFP4) else 2e-3)
    data, scale = mw.expert_bytes("layers.0.moe.local_experts.down")
    one = mw.projection_expert("layers.0.moe.local_experts.down", 1)
    assert one.data == dn.data + data and (not dn.scale or one.scale == dn.scale + scale)
    with pytest.raises(RuntimeError, match="out of range"):
        mw.projection_expert("layers.0.moe.local_experts.down", folders.E)
    mw.close()


def test_skip_experts_and_layout_refusals(hip, tmp_path):
    folders.write(tmp_path / "a", "fp8")
    full = ModelWeights.load(hip, tmp_path / "a", W_FP8)
    lean = ModelWeights.load(hip, tmp_path / "a", W_FP8, skip_experts=True)
    assert lean.projection("layers.0.moe.local_experts.gate_up") is None
    assert lean.projection_shape("layers.0.moe.local_experts.gate_up") == full.projection_shape("layers.0.moe.local_experts.gate_up")
    assert lean.expert_bytes("layers.0.moe.local_experts.down") == full.expert_bytes("layers.0.moe.local_experts.down")
    assert lean.projection_format("layers.0.moe.local_experts.down") == W_FP8
    # the stacks' bytes in the file are exactly what stays off the device (tests/unit/checkpoint_test.cpp:248-284)
    stacks = sum(t.numel() * t.element_size() for name, t in folders.tensors_of("fp8").items() if ".local_experts." in name)
    assert lean.device_bytes() == full.device_bytes() - stacks
    with pytest.raises(RuntimeError, match="skip_experts"):
        lean.projection_expert("layers.0.moe.local_experts.down", 0)
    # a quantised projection without its scale, a scale of the wrong size, an NVFP4 stack without its globals
    from safetensors.torch import save_file

    t = folders.tensors_of("fp8")
    del t["layers.0.mixer.qkv.weight_scale"]
    (tmp_path / "b").mkdir()
    save_file({k: v.contiguous() for k, v in t.items()}, str(tmp_path / "b" / "model.safetensors"))
    with pytest.raises(RuntimeError, match="has no weight_scale"):
        ModelWeights.load(hip, tmp_path / "b", W_FP8)
    t = folders.tensors_of("fp8")
    t["layers.0.mixer.qkv.weight_scale"] = t["layers.0.mixer.qkv.weight_scale"][:-1]
    (tmp_path / "c").mkdir()
    save_file({k: v.contiguous() for k, v in t.items()}, str(tmp_path / "c" / "model.safetensors"))
    with pytest.raises(RuntimeError, match="one f32 scale per row"):
        ModelWeights.load(hip, tmp_path / "c", W_FP8)
    t = folders.tensors_of("nvfp4")
    del t["layers.0.moe.local_experts.down.weight_scale_2"]
    (tmp_path / "d").mkdir()
    save_file({k: v.contiguous() for k, v in t.items()}, str(tmp_path / "d" / "model.safetensors"))
    with pytest.raises(RuntimeError, match="weight_scale_2"):
        ModelWeights.load(hip, tmp_path / "d", W_NVFP4)
    t = folders.tensors_of("bf16")
    del t["embedding.weight"]
    (tmp_path / "e").mkdir()
    save_file({k: v.contiguous() for k, v in t.items()}, str(tmp_path / "e" / "model.safetensors"))
    with pytest.raises(RuntimeError, match="no embedding.weight"):
        ModelWeights.load(hip, tmp_path / "e", W_BF16)
