"""Python binding of the lx_* C ABI, made from the header that declares it (include/dromos_hip.h).

Every prototype in the header becomes a ctypes signature (argument and result types), so a call converts its
Python arguments by the C declaration instead of by guessing from the Python value: a pointer parameter takes a
tensor (its data pointer), an address, a ctypes pointer or None; `int64_t` parameters take 64 bits, `int` and enum
parameters 32; `float` parameters a C float. The trailing `void* stream` of a call may be left out: the current
stream is supplied. The same binding drives the GPU library (device tensors), this repository's CPU oracle and
the reference's CPU backend (host tensors), which export the same ABI; a symbol a library lacks raises
AttributeError when it is first used. The reference's own tests drive a backend through ctypes too
(tests/kernels/conftest.py:79-121, tests/kernels/formats.py:17-24 of the reference).
"""

import ctypes
import os
import re
from pathlib import Path

import torch

F32, BF16 = 0, 1
DTYPE = {torch.float32: F32, torch.bfloat16: BF16}
W_BF16, W_INT8, W_FP8, W_NVFP4, W_BF16X = 0, 1, 2, 3, 4
MATH_BF16, MATH_INT8, MATH_FP8, MATH_FP4 = 0, 1, 2, 3
NOT_SUPPORTED = 801
FORMATS = {"bf16": W_BF16, "int8": W_INT8, "fp8": W_FP8, "nvfp4": W_NVFP4}

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "dromos_hip.h"


class LxWeight(ctypes.Structure):
    """lx_weight (include/dromos_hip.h): {type, data, scale, global, expert_global}."""

    _fields_ = [
        ("type", ctypes.c_int),
        ("data", ctypes.c_void_p),
        ("scale", ctypes.c_void_p),
        ("global_", ctypes.c_float),
        ("expert_global", ctypes.c_void_p),
    ]


_SCALARS = {"int": ctypes.c_int, "unsigned": ctypes.c_uint, "int64_t": ctypes.c_int64, "uint64_t": ctypes.c_uint64,
            "size_t": ctypes.c_size_t, "float": ctypes.c_float, "double": ctypes.c_double}
_PROTOTYPE = re.compile(r"LX_API\s+(?P<result>[\w\s\*]+?)\s*(?P<name>lx_\w+)\s*\((?P<params>[^;{]*)\)\s*;")


def _ctype(decl):
    """The ctypes type of a C parameter or result type as the header spells it."""
    words = decl.replace("const", " ").replace("*", " * ").split()
    if "*" in words:
        return ctypes.c_char_p if words == ["char", "*"] and "const" in decl else ctypes.c_void_p
    if words == ["void"]:
        return None
    if len(words) == 1 and words[0] in _SCALARS:
        return _SCALARS[words[0]]
    if len(words) == 1 and words[0].startswith("lx_"):  # the ABI's enums
        return ctypes.c_int
    raise ValueError(f"no ctypes type for '{decl}'")


def parse_header(text):
    """{name: (result ctype, [(parameter name, ctype), ...])} for every LX_API prototype of a header."""
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    table = {}
    for m in _PROTOTYPE.finditer(text):
        params = []
        body = " ".join(m.group("params").split())
        if body and body != "void":
            for piece in body.split(","):
                piece = piece.strip()
                name = re.search(r"(\w+)\s*$", piece).group(1)
                params.append((name, _ctype(piece[: piece.rfind(name)])))
        table[m.group("name")] = (_ctype(m.group("result")), params)
    return table


_TABLE = None


def prototypes():
    global _TABLE
    if _TABLE is None:
        _TABLE = parse_header(HEADER.read_text())
    return _TABLE


def hip_library_path():
    return Path(os.environ.get("LX_KERNELS") or ROOT / "dromos_amd" / "lib" / "libdromos_hip.so")


class Kernels:
    """One backend library. ``device`` is where its tensors live: "cuda" for the GPU library, "cpu" for the
    CPU checkers. ``lib`` is the ctypes library with the header's signatures applied to every symbol it has."""

    def __init__(self, path, device):
        path = Path(path)
        if not path.exists():
            raise FileNotFoundError(f"backend library {path} is not built (python -m dromos_amd.build)")
        self.path, self.device = path, device
        self.lib = ctypes.CDLL(str(path))
        self._params = {}
        for name, (result, params) in prototypes().items():
            try:
                fn = getattr(self.lib, name)
            except AttributeError:
                continue  # the CPU checkers export the product path only
            fn.restype = result
            fn.argtypes = [t for _, t in params]
            self._params[name] = params
        if device == "cuda" and "lx_rt_stream_reserve" in self._params and torch.cuda.is_available():
            # The harness issues on streams the library did not make (torch's): give the one it uses by default what
            # lx_rt_stream_create gives a stream.
            self.reserve_stream(None)

    def _stream(self):
        return None if self.device == "cpu" else torch.cuda.current_stream().cuda_stream

    @property
    def stream(self):
        return ctypes.c_void_p(self._stream())

    def reserve_stream(self, stream):
        status = self.lib.lx_rt_stream_reserve(stream)
        assert status == 0, f"lx_rt_stream_reserve returned status {status}"

    def sync(self):
        if self.device == "cpu":
            assert self.lib.lx_rt_stream_sync(None) == 0
        else:
            torch.cuda.synchronize()

    def _lower(self, value):
        if isinstance(value, torch.Tensor):
            if value.device.type != self.device or not value.is_contiguous():
                raise ValueError(f"kernels take contiguous {self.device} tensors, not {value.device} / strides {value.stride()}")
            return value.data_ptr()
        return int(value) if isinstance(value, bool) else value

    def status(self, name, *args, stream=True):
        """Calls lx_<name> and returns what it returns (a status, for most). With ``stream`` the call's last
        parameter, when it is the stream and was left out, is the current stream."""
        symbol = "lx_" + name
        fn = getattr(self.lib, symbol)
        lowered = [self._lower(a) for a in args]
        params = self._params.get(symbol)
        if params is None:  # not in the header: ctypes' own conversions, the stream behind the arguments
            if stream:
                lowered.append(self.stream)
            return fn(*lowered)
        if stream and len(lowered) == len(params) - 1 and params[-1][0] == "stream":
            lowered.append(self._stream())
        if len(lowered) != len(params):
            raise TypeError(f"{symbol} takes {len(params)} arguments ({', '.join(n for n, _ in params)}), got {len(lowered)}")
        return fn(*lowered)

    def __call__(self, name, *args):
        status = self.status(name, *args)
        assert status == 0, f"lx_{name} returned status {status}"
        self.sync()

    def size(self, name, *args):
        """A size query such as moe_decode_workspace_bytes (no stream parameter)."""
        return self.status(name, *args, stream=False)


def load_hip():
    """The GPU library. Raises when it is not built: there is no fallback path."""
    return Kernels(hip_library_path(), "cuda")
