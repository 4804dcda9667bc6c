"""dromos_amd: the decode matrix-product path of Dromos as a hand-written HIP backend library for MI355X.

The product is ``lib/libdromos_hip.so`` (C ABI declared in ``include/dromos_hip.h``); this package holds its
sources (``csrc/``), the build recipe (``build.py``) and a ctypes harness (``abi.py``, ``formats.py``) that
calls the library the way the reference's kernel tests call any backend library
(tests/kernels/conftest.py:79-121 of the reference).
"""

from .abi import (  # noqa: F401
    BF16,
    DTYPE,
    F32,
    MATH_BF16,
    MATH_FP4,
    MATH_FP8,
    MATH_INT8,
    NOT_SUPPORTED,
    W_BF16,
    W_FP8,
    W_INT8,
    W_NVFP4,
    Kernels,
    LxWeight,
    hip_library_path,
    load_hip,
)
