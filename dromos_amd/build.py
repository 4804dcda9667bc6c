"""Compiles the HIP library for gfx950 (in-tree, so the built .so travels with the tree) and the CPU checkers.

    python -m dromos_amd.build            # libdromos_hip.so + oracle/liboracle.so (+ oracle/_ref when the
                                          # reference sources are present)
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "dromos_amd" / "csrc"
LIB_DIR = ROOT / "dromos_amd" / "lib"
HIP_LIB = LIB_DIR / "libdromos_hip.so"
SOURCES = ["runtime.hip", "quant.hip", "gemv.hip", "gemv_bf16.hip", "gemv_int8.hip", "gemv_fp8.hip", "gemv_nvfp4.hip", "gemv_bf16x.hip", "bf16x.hip", "gemm.hip", "gemm_walk_bf16.hip", "gemm_walk_int8.hip", "gemm_walk_fp8.hip", "gemm_walk_nvfp4.hip",
           "moe.hip", "moe_grouped.hip", "router.hip", "checkpoint.hip"]

# -ffp-contract=off: the epilogues and the ordered sums are written as separate multiplies and adds, as the
# CPU reference computes them; fused operations are spelled __builtin_fmaf where they are meant.
# packed-fp32-ops off: scalar float code must not be turned into v_pk_*_f32 by the optimiser.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(map(str, cmd))}\n{proc.stdout}\n{proc.stderr}")
    return proc


def build_hip(verbose=False):
    """Compiles every .hip source and links lib/libdromos_hip.so. Always recompiles."""
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    hipcc = _hipcc()
    objs = [LIB_DIR / (Path(s).stem + ".o") for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        _run([hipcc, *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)])
        if verbose:
            print(f"compiled {src}", flush=True)

    with ThreadPoolExecutor(max_workers=8) as pool:
        list(pool.map(compile_one, zip(SOURCES, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(HIP_LIB), *map(str, objs)])
    return HIP_LIB


def build_oracle(verbose=False):
    """The CPU checkers (test infrastructure): oracle/liboracle.so, and oracle/_ref/libdromos_cpu.so from the
    reference's own sources when they are present on this machine."""
    proc = _run(["make", "-C", str(ROOT / "oracle"), "-j8", "all"])
    if verbose:
        print(proc.stdout[-2000:], flush=True)
    return ROOT / "oracle" / "liboracle.so"


if __name__ == "__main__":
    print(build_hip(verbose=True))
    print(build_oracle(verbose="-v" in sys.argv))
