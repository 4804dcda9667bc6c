"""Host logic of the model-folder loader (lx_ckpt_*): the recipe, what a folder holds, and the safetensors reader's
refusals. No device call is made here (the library is only loaded)."""

import json
import struct

import pytest

import folders
from dromos_amd.abi import Kernels, W_BF16, W_BF16X, W_FP8, W_INT8, W_NVFP4, hip_library_path
from dromos_amd.checkpoint import ModelWeights, projection_format


@pytest.fixture(scope="module")
def lib():
    path = hip_library_path()
    if not path.exists():
        pytest.fail(f"{path} is not built: run `python -m dromos_amd.build`")
    return Kernels(path, "cpu")


def test_recipe_known_answers(lib):
    # engine/core/checkpoint.cpp:15-27 in words, and recipe() at :124-166.
    wide = ["layers.3.mixer.impl.mixer.out_proj", "layers.3.mixer.pass_lora_down", "layers.3.mixer.pass_lora_up", "layers.3.depth_memory.metadata_write"]
    for target in (W_BF16, W_INT8, W_FP8, W_NVFP4, W_BF16X):
        for key in wide:
            assert projection_format(lib, target, key) == W_BF16, (target, key)
        for key in ("layers.1.depth_memory.key", "layers.1.depth_memory.value"):
            assert projection_format(lib, target, key) == (W_FP8 if target == W_NVFP4 else W_BF16)
    assert [projection_format(lib, t, "embedding") for t in (W_BF16, W_INT8, W_FP8, W_NVFP4, W_BF16X)] == [W_BF16, W_INT8, W_BF16, W_FP8, W_BF16X]
    experts = ["layers.0.moe.local_experts.gate_up", "layers.0.moe.local_experts.down"]
    fp8_dense = ["layers.0.mixer.impl.mixer.in_proj", "layers.0.mixer.qkv", "layers.0.mixer.out"]
    other = ["layers.0.moe.latent_down", "layers.0.moe.latent_up", "layers.0.moe.shared_expert.gate_up", "layers.0.depth_memory.query"]
    for key in experts + fp8_dense + other:
        assert projection_format(lib, W_BF16, key) == W_BF16
        assert projection_format(lib, W_INT8, key) == W_INT8
        assert projection_format(lib, W_BF16X, key) == W_BF16X
    for key in experts + fp8_dense:
        assert projection_format(lib, W_FP8, key) == W_FP8
    for key in other:
        assert projection_format(lib, W_FP8, key) == W_BF16
    for key in experts:
        assert projection_format(lib, W_NVFP4, key) == W_NVFP4
    assert projection_format(lib, W_NVFP4, "layers.0.moe.latent_up") == W_BF16
    for key in fp8_dense + ["layers.0.moe.latent_down", "layers.0.moe.shared_expert.gate_up"]:
        assert projection_format(lib, W_NVFP4, key) == W_FP8
    # the ".weight" suffix is optional; a component must match whole ("xmixer.qkv" is not "mixer.qkv")
    assert projection_format(lib, W_FP8, "layers.0.mixer.qkv.weight") == W_FP8
    assert projection_format(lib, W_FP8, "layers.0.xmixer.qkv") == W_BF16


@pytest.mark.parametrize("layout,fmt", [("bf16", W_BF16), ("fp8", W_FP8), ("nvfp4", W_NVFP4)])
@pytest.mark.parametrize("shards", [1, 3])
def test_stored_format(lib, tmp_path, layout, fmt, shards):
    folders.write(tmp_path, layout, shards=shards)
    assert ModelWeights.stored_format(lib, tmp_path) == fmt


def test_reader_refusals(lib, tmp_path):
    with pytest.raises(RuntimeError, match="cannot open"):
        ModelWeights.stored_format(lib, tmp_path / "nowhere")
    d = tmp_path / "short"
    d.mkdir()
    (d / "model.safetensors").write_bytes(b"abc")
    with pytest.raises(RuntimeError, match="too short"):
        ModelWeights.stored_format(lib, d)

    def folder(name, header, payload=b"\0" * 64, length=None):
        f = tmp_path / name
        f.mkdir()
        body = json.dumps(header).encode() if not isinstance(header, bytes) else header
        (f / "model.safetensors").write_bytes(struct.pack("<Q", len(body) if length is None else length) + body + payload)
        return f

    with pytest.raises(RuntimeError, match="longer than the file"):
        ModelWeights.stored_format(lib, folder("long", {}, length=1 << 40))
    with pytest.raises(RuntimeError, match="not valid JSON"):
        ModelWeights.stored_format(lib, folder("json", b'{"a": [1, 2'))
    with pytest.raises(RuntimeError, match="outside the file"):
        ModelWeights.stored_format(lib, folder("outside", {"a": {"dtype": "F32", "shape": [64], "data_offsets": [0, 256]}}))
    with pytest.raises(RuntimeError, match="shape says otherwise"):
        ModelWeights.stored_format(lib, folder("bytes", {"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}))
    with pytest.raises(RuntimeError, match="unknown dtype"):
        ModelWeights.stored_format(lib, folder("dtype", {"a": {"dtype": "F4", "shape": [8], "data_offsets": [0, 8]}}))
    with pytest.raises(RuntimeError, match="lacks dtype"):
        ModelWeights.stored_format(lib, folder("lacks", {"a": {"dtype": "F32", "shape": [2]}}))
    # nesting the reader would have to recurse through: refused with a reason, in the header and in the index
    for i, opener in enumerate((b"[", b"{\"a\":", b"[{\"a\":")):
        with pytest.raises(RuntimeError, match="nested more than 64 deep"):
            ModelWeights.stored_format(lib, folder(f"deep{i}", b'{"a": ' + opener * 100000))
    deep = tmp_path / "deep_index"
    folders.write(deep, "bf16", shards=2)
    (deep / "model.safetensors.index.json").write_bytes(b'{"weight_map": ' + b"[" * 100000)
    with pytest.raises(RuntimeError, match="nested more than 64 deep"):
        ModelWeights.stored_format(lib, deep)
    sixty = b'{"__metadata__": ' + b"[" * 62 + b"]" * 62 + b', "a.weight": {"dtype": "BF16", "shape": [2, 2], "data_offsets": [0, 8]}}'
    assert ModelWeights.stored_format(lib, folder("sixty", sixty)) == W_BF16  # 63 levels are read
    # a header past the format's 100 MB limit (a sparse file: only the length is real)
    big = tmp_path / "big"
    big.mkdir()
    with open(big / "model.safetensors", "wb") as f:
        f.write(struct.pack("<Q", 100_000_001) + b"{")
        f.truncate(8 + 100_000_001 + 64)
    with pytest.raises(RuntimeError, match="longer than 100 MB"):
        ModelWeights.stored_format(lib, big)
    # metadata is skipped, escapes in names are read
    ok = folder("ok", {"__metadata__": {"format": "pt"}, "a\\u0041.weight": {"dtype": "BF16", "shape": [2, 2], "data_offsets": [0, 8]}})
    assert ModelWeights.stored_format(lib, ok) == W_BF16
    # an index that sends a tensor to the wrong shard
    folders.write(tmp_path / "sharded", "bf16", shards=2)
    idx = tmp_path / "sharded" / "model.safetensors.index.json"
    doc = json.loads(idx.read_text())
    names = sorted(doc["weight_map"])
    doc["weight_map"][names[0]] = doc["weight_map"][names[1]]
    idx.write_text(json.dumps(doc))
    with pytest.raises(RuntimeError, match="does not hold it"):
        ModelWeights.stored_format(lib, tmp_path / "sharded")
    idx.write_text(json.dumps({"metadata": {}}))
    with pytest.raises(RuntimeError, match="weight_map"):
        ModelWeights.stored_format(lib, tmp_path / "sharded")


def test_damaged_files_are_refused_or_read_never_worse(lib, tmp_path):
    """Random damage to the headers, the index and the file sizes of a one-file and a three-shard folder: every answer is
    a format or a refusal with a reason (a reader that trusted a length or an offset would fault instead)."""
    import random

    rnd = random.Random(20)
    folders.write(tmp_path / "one", "fp8", shards=1)
    folders.write(tmp_path / "three", "nvfp4", shards=3)
    good = {(d, f.name): f.read_bytes() for d in ("one", "three") for f in (tmp_path / d).iterdir()}
    refused = 0
    for _ in range(400):
        key = rnd.choice(sorted(good))
        data = bytearray(good[key])
        span = 8 + struct.unpack("<Q", data[:8])[0] if key[1].endswith(".safetensors") else len(data)
        kind = rnd.randrange(5)
        if kind == 0:
            for _ in range(rnd.randrange(1, 6)):
                data[rnd.randrange(span)] = rnd.randrange(256)
        elif kind == 1:
            del data[rnd.randrange(len(data)):]
        elif kind == 2 and key[1].endswith(".safetensors"):
            data[:8] = struct.pack("<Q", rnd.choice([0, 1, 7, 1 << 63, (1 << 64) - 1, len(data), len(data) - 8, rnd.randrange(1 << 40)]))
        elif kind == 3:
            at = rnd.randrange(span)
            del data[at:at + rnd.randrange(1, 40)]
        else:
            digits = [i for i in range(8, span) if 48 <= data[i] <= 57]
            at = rnd.choice(digits)
            data[at:at + 1] = rnd.choice([b"99999999999999999999", b"-1", b"1e99", b"0.5", b""])
        path = tmp_path / key[0] / key[1]
        path.write_bytes(bytes(data))
        try:
            assert ModelWeights.stored_format(lib, tmp_path / key[0]) in (W_BF16, W_FP8, W_NVFP4)
        except RuntimeError as e:
            assert str(e)
            refused += 1
        path.write_bytes(good[key])
    assert refused > 300
