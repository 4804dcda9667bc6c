"""ctypes harness for a backend library of the lx_* C ABI (include/dromos_hip.h).

Mirrors how the reference's kernel tests drive a backend (tests/kernels/conftest.py:79-121 and
tests/kernels/formats.py:17-24 of the reference): tensors are passed as raw pointers, Python ints as C ints,
floats as C floats, the current stream is appended as the last argument, a non-zero status is an error, and
the call is followed by a synchronisation. The same class drives the GPU library (device tensors), this
repository's CPU oracle and the reference's CPU backend (host tensors).
"""

import ctypes
import os
from pathlib import Path

import torch

F32, BF16 = 0, 1
DTYPE = {torch.float32: F32, torch.bfloat16: BF16}
W_BF16, W_INT8, W_FP8, W_NVFP4, W_BF16X = 0, 1, 2, 3, 4
MATH_BF16, MATH_INT8, MATH_FP8, MATH_FP4 = 0, 1, 2, 3
NOT_SUPPORTED = 801
FORMATS = {"bf16": W_BF16, "int8": W_INT8, "fp8": W_FP8, "nvfp4": W_NVFP4}

ROOT = Path(__file__).resolve().parent.parent


class LxWeight(ctypes.Structure):
    """lx_weight (include/dromos_hip.h): {type, data, scale, global, expert_global}."""

    _fields_ = [
        ("type", ctypes.c_int),
        ("data", ctypes.c_void_p),
        ("scale", ctypes.c_void_p),
        ("global_", ctypes.c_float),
        ("expert_global", ctypes.c_void_p),
    ]


def hip_library_path():
    return Path(os.environ.get("LX_KERNELS") or ROOT / "dromos_amd" / "lib" / "libdromos_hip.so")


class Kernels:
    """One backend library. ``device`` is where its tensors live: "cuda" for the GPU library, "cpu" for the
    CPU checkers."""

    def __init__(self, path, device):
        path = Path(path)
        if not path.exists():
            raise FileNotFoundError(f"backend library {path} is not built (python -m dromos_amd.build)")
        self.path = path
        self.device = device
        self.lib = ctypes.CDLL(str(path))
        for name in ("lx_gemm_workspace_bytes", "lx_moe_decode_workspace_bytes", "lx_moe_grouped_workspace_bytes",
                     "lx_moe_bf16x_workspace_bytes"):
            if hasattr(self.lib, name):
                getattr(self.lib, name).restype = ctypes.c_int64

    @property
    def stream(self):
        if self.device == "cpu":
            return ctypes.c_void_p(None)
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def sync(self):
        if self.device == "cpu":
            assert self.lib.lx_rt_stream_sync(None) == 0
        else:
            torch.cuda.synchronize()

    def status(self, name, *args, stream=True):
        """Calls lx_<name> and returns its status unchecked."""
        fn = getattr(self.lib, "lx_" + name)
        fn.restype = ctypes.c_int
        conv = []
        for a in args:
            if isinstance(a, torch.Tensor):
                assert a.device.type == self.device and a.is_contiguous(), f"kernels take contiguous {self.device} tensors"
                conv.append(ctypes.c_void_p(a.data_ptr()))
            elif isinstance(a, bool):
                conv.append(ctypes.c_int(int(a)))
            elif isinstance(a, int):
                conv.append(ctypes.c_int64(a) if abs(a) >= 2**31 else ctypes.c_int(a))
            elif isinstance(a, float):
                conv.append(ctypes.c_float(a))
            elif a is None:
                conv.append(ctypes.c_void_p(None))
            else:
                conv.append(a)
        if stream:
            conv.append(self.stream)
        return fn(*conv)

    def __call__(self, name, *args):
        status = self.status(name, *args)
        assert status == 0, f"lx_{name} returned status {status}"
        self.sync()

    def size(self, name, *args):
        """An int64-returning size query such as moe_decode_workspace_bytes."""
        fn = getattr(self.lib, "lx_" + name)
        fn.restype = ctypes.c_int64
        return fn(*[ctypes.c_int(a) for a in args])


def load_hip():
    """The GPU library. Raises when it is not built: there is no fallback path."""
    return Kernels(hip_library_path(), "cuda")
