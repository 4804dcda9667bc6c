"""The C-ABI library loads and exports exactly what include/dromos_hip.h declares (no compute calls: this runs
without a GPU)."""

import ctypes
import re
from pathlib import Path

import pytest

from dromos_amd.abi import LxWeight, hip_library_path

ROOT = Path(__file__).resolve().parent.parent


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
