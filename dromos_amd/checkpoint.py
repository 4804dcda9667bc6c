"""Host-side mirror of the reference's loader interface (engine/core/checkpoint.h:24-101) over the lx_ckpt_* C ABI:
the same names (projection_format, ModelWeights.stored_format / load / projection / projection_names /
projection_shape / projection_expert / expert_bytes / find / format / device_bytes / peak_device_bytes) and the same
errors (a refused load raises RuntimeError with the loader's message)."""

import ctypes
from collections import namedtuple

from .abi import LxWeight

Shape = namedtuple("Shape", "E N K stack")
WeightView = namedtuple("WeightView", "data dtype shape")


def _lib(lx):
    lib = lx.lib
    if not getattr(lib, "_ckpt_typed", False):
        lib.lx_ckpt_error.restype = ctypes.c_char_p
        lib.lx_ckpt_projection.restype = ctypes.POINTER(LxWeight)
        lib.lx_ckpt_projection.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        lib.lx_ckpt_name.restype = ctypes.c_char_p
        lib.lx_ckpt_name.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.lx_ckpt_count.argtypes = [ctypes.c_void_p]
        lib.lx_ckpt_free.argtypes = [ctypes.c_void_p]
        lib.lx_ckpt_tensor.restype = ctypes.c_void_p
        lib.lx_ckpt_tensor.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                       ctypes.POINTER(ctypes.c_int64), ctypes.c_int]
        lib.lx_ckpt_device_bytes.restype = ctypes.c_int64
        lib.lx_ckpt_device_bytes.argtypes = [ctypes.c_void_p]
        lib.lx_ckpt_peak_device_bytes.restype = ctypes.c_int64
        lib.lx_ckpt_peak_device_bytes.argtypes = [ctypes.c_void_p]
        lib.lx_ckpt_target.argtypes = [ctypes.c_void_p]
        lib.lx_ckpt_format_of.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        lib.lx_ckpt_shape.argtypes = [ctypes.c_void_p, ctypes.c_char_p] + [ctypes.POINTER(ctypes.c_int64)] * 3 + [ctypes.POINTER(ctypes.c_int)]
        lib.lx_ckpt_expert.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int64, ctypes.POINTER(LxWeight)]
        lib.lx_ckpt_expert_bytes.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]
        lib.lx_ckpt_load.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
        lib.lx_ckpt_stored_format.argtypes = [ctypes.c_char_p]
        lib.lx_ckpt_projection_format.argtypes = [ctypes.c_int, ctypes.c_char_p]
        lib._ckpt_typed = True
    return lib


def _error(lib):
    return RuntimeError(lib.lx_ckpt_error().decode("utf-8", "replace"))  # a damaged file's names may not be text


def projection_format(lx, target, projection):
    """The loader's recipe: the format `projection` is held in for `target`."""
    return _lib(lx).lx_ckpt_projection_format(int(target), projection.encode())


class ModelWeights:
    def __init__(self, lx, handle):
        self._lx, self._lib, self._h = lx, _lib(lx), handle

    @staticmethod
    def stored_format(lx, directory):
        lib = _lib(lx)
        fmt = lib.lx_ckpt_stored_format(str(directory).encode())
        if fmt < 0:
            raise _error(lib)
        return fmt

    @staticmethod
    def load(lx, directory, target=0, skip_experts=False):
        lib = _lib(lx)
        handle = ctypes.c_void_p()
        if lib.lx_ckpt_load(str(directory).encode(), int(target), int(skip_experts), ctypes.byref(handle)) != 0:
            raise _error(lib)
        return ModelWeights(lx, handle)

    def close(self):
        if self._h:
            self._lib.lx_ckpt_free(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def projection(self, name):
        p = self._lib.lx_ckpt_projection(self._h, name.encode())
        return p.contents if p else None

    def projection_names(self):
        return [self._lib.lx_ckpt_name(self._h, i).decode() for i in range(self._lib.lx_ckpt_count(self._h))]

    def projection_shape(self, name):
        E, N, K, stack = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int()
        if self._lib.lx_ckpt_shape(self._h, name.encode(), ctypes.byref(E), ctypes.byref(N), ctypes.byref(K), ctypes.byref(stack)) != 0:
            raise RuntimeError("no projection " + name)
        return Shape(E.value, N.value, K.value, bool(stack.value))

    def projection_format(self, name):
        return self._lib.lx_ckpt_format_of(self._h, name.encode())

    def projection_expert(self, name, e):
        out = LxWeight()
        if self._lib.lx_ckpt_expert(self._h, name.encode(), e, ctypes.byref(out)) != 0:
            raise _error(self._lib)
        return out

    def expert_bytes(self, name):
        data, scale = ctypes.c_int64(), ctypes.c_int64()
        if self._lib.lx_ckpt_expert_bytes(self._h, name.encode(), ctypes.byref(data), ctypes.byref(scale)) != 0:
            raise RuntimeError("no projection " + name)
        return data.value, scale.value

    def find(self, name):
        dtype, rank = ctypes.c_int(), ctypes.c_int()
        shape = (ctypes.c_int64 * 8)()
        ptr = self._lib.lx_ckpt_tensor(self._h, name.encode(), ctypes.byref(dtype), ctypes.byref(rank), shape, 8)
        return WeightView(ptr, dtype.value, tuple(shape[: rank.value])) if ptr else None

    def format(self):
        return self._lib.lx_ckpt_target(self._h)

    def device_bytes(self):
        return int(self._lib.lx_ckpt_device_bytes(self._h))

    def peak_device_bytes(self):
        return int(self._lib.lx_ckpt_peak_device_bytes(self._h))
