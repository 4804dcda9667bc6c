"""The C-ABI library loads and exports exactly what include/dromos_hip.h declares (no compute calls: this runs
without a GPU)."""

import ctypes
import re
from pathlib import Path

import pytest

from dromos_amd.abi import LxWeight, hip_library_path, parse_header

ROOT = Path(__file__).resolve().parent.parent
REFERENCE = Path("/root/reference/engine/cuda")


def signatures(text):
    """{symbol: (result type, [parameter types])} of a header's LX_API prototypes, types as token strings
    (`const void *`, `lx_dtype`, `int64_t`), parameter names dropped."""
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    out = {}
    for m in re.finditer(r"LX_API\s+([\w\s\*]+?)\s*(lx_\w+)\s*\(([^;{]*)\)\s*;", text):
        norm = lambda t: " ".join(t.replace("*", " * ").split())
        params = []
        body = " ".join(m.group(3).split())
        if body and body != "void":
            for piece in body.split(","):
                piece = piece.strip()
                name = re.search(r"(\w+)\s*$", piece).group(1)
                params.append(norm(piece[: piece.rfind(name)]))
        out[m.group(2)] = (norm(m.group(1)), params)
    return out


def declared_symbols():
    text = (ROOT / "include" / "dromos_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"LX_API\s+[\w\s\*]+?\b(lx_\w+)\s*\(", text)))


def test_header_declares_the_hot_path():
    names = declared_symbols()
    for must in ("lx_gemv", "lx_gemv_w", "lx_gemv_decode_bf16", "lx_gemm_w", "lx_gemm_skinny", "lx_gemm_workspace_bytes",
                 "lx_quantize_w8", "lx_quantize_weight", "lx_dequantize_weight", "lx_moe_route", "lx_moe_experts",
                 "lx_moe_experts_decode", "lx_moe_decode_workspace_bytes", "lx_moe_experts_decode_bf16",
                 "lx_moe_bf16x_workspace_bytes", "lx_moe_experts_grouped", "lx_moe_grouped_workspace_bytes",
                 "lx_bf16x_row_bytes", "lx_bf16x_bytes", "lx_bf16x_encode", "lx_bf16x_decode", "lx_gemv_bf16x",
                 "lx_moe_experts_bf16x", "lx_ckpt_load", "lx_ckpt_projection", "lx_ckpt_projection_format", "lx_ckpt_stored_format",
                 "lx_ckpt_expert", "lx_ckpt_tensor", "lx_ckpt_free", "lx_rt_backend", "lx_rt_device_count", "lx_arch", "lx_tune_variants", "lx_bandwidth_probe"):
        assert must in names, must


def test_library_exports_every_declared_symbol():
    path = hip_library_path()
    if not path.exists():
        pytest.fail(f"{path} is not built: run `python -m dromos_amd.build`")
    lib = ctypes.CDLL(str(path))
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, f"declared in include/dromos_hip.h but not exported: {missing}"


def test_backend_identity_and_sizes():
    lib = ctypes.CDLL(str(hip_library_path()))
    assert lib.lx_rt_backend() == 1  # LX_BACKEND_HIP
    # lx_weight is {int, ptr, ptr, float, ptr}: 40 bytes on LP64, as the engine's struct
    assert ctypes.sizeof(LxWeight) == 40
    lib.lx_moe_decode_workspace_bytes.restype = ctypes.c_int64
    assert lib.lx_moe_decode_workspace_bytes(8, 512, 4) >= 2 * 8 * 4 * 512
    assert lib.lx_moe_decode_workspace_bytes(0, 512, 4) == 0
    lib.lx_gemm_workspace_bytes.restype = ctypes.c_int64
    assert lib.lx_gemm_workspace_bytes(0, 128, 0) == 0
    assert lib.lx_tune_variants(b"gemv_w_bf16") > 0 and lib.lx_tune_variants(b"nothing") == 0
    lib.lx_tune_variant_name.restype = ctypes.c_char_p
    assert lib.lx_tune_variant_name(b"gemv_w_int8", 1).decode().startswith("s2")
    lib.lx_rt_error_string.restype = ctypes.c_char_p
    assert lib.lx_rt_error_string(801) == b"operation not supported"


def test_the_binding_reads_every_prototype():
    names = declared_symbols()
    table = parse_header((ROOT / "include" / "dromos_hip.h").read_text())
    assert sorted(table) == names
    result, params = table["lx_gemm_w"]
    assert result is ctypes.c_int and [n for n, _ in params][-2:] == ["workspace", "stream"]
    assert table["lx_gemm_workspace_bytes"][0] is ctypes.c_int64
    assert table["lx_tune_variant_name"][0] is ctypes.c_char_p


@pytest.mark.skipif(not REFERENCE.exists(), reason="the reference's headers are not on this machine")
def test_shared_prototypes_equal_the_reference_headers():
    # Every symbol this library shares with the engine's backends has the engine's exact prototype: same result type,
    # same parameter types in the same order (engine/cuda/kernels.h, engine/cuda/tunable.h).
    ours = signatures((ROOT / "include" / "dromos_hip.h").read_text())
    theirs = {}
    for header in ("kernels.h", "tunable.h"):
        theirs.update(signatures((REFERENCE / header).read_text()))
    shared = sorted(set(ours) & set(theirs))
    assert len(shared) >= 60, shared
    different = {n: (ours[n], theirs[n]) for n in shared if ours[n] != theirs[n]}
    assert not different, different
    for must in ("lx_gemv_w", "lx_gemm_w", "lx_gemm_skinny", "lx_moe_route", "lx_moe_experts_decode", "lx_moe_experts_grouped",
                 "lx_quantize_weight", "lx_tune_set", "lx_rt_stream_create"):
        assert must in shared, must


def test_tune_key_and_runnable():
    # engine/cuda/tunable.cu:180-185: the name, "@w<weight>m<math>" when either is not 0, "@e<experts>" when not 1.
    class Problem(ctypes.Structure):
        _fields_ = [(n, ctypes.c_int) for n in ("M", "N", "K", "experts", "weight", "math")]

    lib = ctypes.CDLL(str(hip_library_path()))
    out = ctypes.create_string_buffer(64)
    for fields, want in (((1, 2, 3, 1, 0, 0), b"gemm_w"), ((1, 2, 3, 1, 2, 0), b"gemm_w@w2m0"), ((1, 2, 3, 64, 3, 1), b"gemm_w@w3m1@e64"),
                         ((1, 2, 3, 8, 0, 0), b"gemm_w@e8")):
        p = Problem(*fields)
        assert lib.lx_tune_key(b"gemm_w", ctypes.byref(p), out, 64) == len(want) and out.value == want
    p = Problem(1, 2, 3, 64, 3, 1)
    small = ctypes.create_string_buffer(8)
    assert lib.lx_tune_key(b"gemm_w", ctypes.byref(p), small, 8) == len(b"gemm_w@w3m1@e64") and small.value == b"gemm_w@"
    for fmt in ("bf16", "int8", "fp8", "nvfp4"):
        assert lib.lx_tune_runnable(f"gemm_w_{fmt}".encode()) == 1 and lib.lx_tune_runnable(f"gemv_w_{fmt}".encode()) == 1
    assert lib.lx_tune_runnable(b"attention") == 0
