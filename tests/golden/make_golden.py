"""Writes reference_cpu_generic.npz: the outputs of the reference's CPU backend, at its generic ISA level
(lx_set_arch_override(1): four-lane f32 sums), for every case in cases.py.

Run here, where oracle/_ref/libdromos_cpu.so has been compiled from the reference's sources
(make -C oracle ref); the fixture then travels with the repository and the reference does not.

    python tests/golden/make_golden.py
"""

import ctypes
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))
sys.path.insert(0, str(HERE.parent))
sys.path.insert(0, str(HERE))

import cases  # noqa: E402
from dromos_amd.abi import Kernels  # noqa: E402


def main():
    lib = HERE.parent.parent / "oracle" / "_ref" / "libdromos_cpu.so"
    ref = Kernels(lib, "cpu")
    ref.lib.lx_set_arch_override.restype = ctypes.c_int
    ref.lib.lx_set_arch_override.argtypes = [ctypes.c_int]
    assert ref.lib.lx_set_arch_override(1) == 1
    arrays = {}
    for name in cases.CASES:
        check, outputs = cases.run_case(ref, name)
        arrays[f"{name}/inputs_checksum"] = np.array([check], dtype=np.int64)
        for key, value in outputs.items():
            arrays[f"{name}/{key}"] = value.numpy()
    np.savez_compressed(HERE / "reference_cpu_generic.npz", **arrays)
    print(f"{len(arrays)} arrays, {(HERE / 'reference_cpu_generic.npz').stat().st_size} bytes")


if __name__ == "__main__":
    main()
