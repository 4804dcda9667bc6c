"""Times a kernel's variants through the C ABI and fills the library's variant table, the way the engine's autotuner
drives a backend (engine/cuda/tunable.h:57-75: lx_tune_run on the kernel's own inputs, every variant checked against
variant 0, the pick stored with lx_tune_set so that the kernel's admission rule has the last word).

    python -m dromos_amd.tune gemm_w_fp8 32 6144 4096 [gemm_w_int8 64 14336 4096 ...]     # prints one JSON line per problem

From Python: `tune(lx, "gemm_w_fp8", 32, 6144, 4096)` returns the timings and stores the pick; `table(lx, problems)` does
it for a list and returns {key: variant name}. Between two timed launches 512 MB are written, so every launch streams its
weights from HBM as a decode step does (the inputs lx_tune_run keeps per problem would otherwise sit in the 256 MB
Infinity Cache).
"""

import ctypes
import json
import sys

import torch

from .abi import load_hip

FLUSH_BYTES = 512 << 20


class Problem(ctypes.Structure):
    """lx_tune_problem (engine/cuda/tunable.h:61-66)."""

    _fields_ = [(n, ctypes.c_int) for n in ("M", "N", "K", "experts", "weight", "math")]


def variants(lx, kernel):
    lib = lx.lib
    lib.lx_tune_variant_name.restype = ctypes.c_char_p
    return [lib.lx_tune_variant_name(kernel.encode(), v).decode() for v in range(lib.lx_tune_variants(kernel.encode()))]


def time_variants(lx, kernel, M, N, K, repeats=7):
    """{variant name: (median microseconds of one launch, bits equal variant 0's)} for the variants that run here."""
    lib = lx.lib
    name = kernel.encode()
    if not lib.lx_tune_runnable(name):
        raise ValueError(f"{kernel} has no runner")
    problem = Problem(M, N, K, 1, 0, 0)
    events = []
    for _ in range(2):
        e = ctypes.c_void_p()
        assert lib.lx_rt_event_create_timed(ctypes.byref(e)) == 0
        events.append(e)
    flush = torch.empty(FLUSH_BYTES, dtype=torch.uint8, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # The variants that keep partial sums in the stream's buffer run only on a stream that has one; the stream keeps it
    # afterwards (reserving twice is harmless, and releasing here would take away a buffer the caller had reserved).
    assert lib.lx_rt_stream_reserve(stream) == 0
    first, result = None, {}
    try:
        for v, vname in enumerate(variants(lx, kernel)):
            out = torch.empty(M, N, dtype=torch.float32, device="cuda")
            if lx.status("tune_run", name, v, ctypes.byref(problem), out) != 0:
                continue  # LX_ERR_NOT_SUPPORTED: this variant or problem does not run here
            torch.cuda.synchronize()
            first = out if first is None else first
            same = bool(torch.equal(out.view(torch.int32), first.view(torch.int32)))
            times = []
            for _ in range(repeats):
                flush.fill_(1)
                assert lib.lx_rt_event_record(events[0], stream) == 0
                assert lx.status("tune_run", name, v, ctypes.byref(problem), out) == 0
                assert lib.lx_rt_event_record(events[1], stream) == 0
                torch.cuda.synchronize()
                ms = ctypes.c_float()
                assert lib.lx_rt_event_elapsed(events[0], events[1], ctypes.byref(ms)) == 0
                times.append(ms.value * 1e3)
            times.sort()
            result[vname] = (round(times[len(times) // 2], 2), same)
    finally:
        for e in events:
            lib.lx_rt_event_destroy(e)
    return result


def tune(lx, kernel, M, N, K, repeats=7, tolerance=1e-5):
    """Times the variants, stores the fastest one the kernel admits for the shape (lx_tune_set), and returns
    {"key", "us": {variant: microseconds}, "pick": variant name or None}. A variant whose result is neither variant 0's
    bits nor within `tolerance` (relative L2) of it is never picked."""
    lib = lx.lib
    names = variants(lx, kernel)
    timed = time_variants(lx, kernel, M, N, K, repeats)
    key = ctypes.create_string_buffer(128)
    lib.lx_tune_key(kernel.encode(), ctypes.byref(Problem(M, N, K, 1, 0, 0)), key, 128)
    pick = None
    for vname, (us, same) in sorted(timed.items(), key=lambda kv: kv[1][0]):
        if not same and not _close(lx, kernel, names.index(vname), M, N, K, tolerance):
            continue
        if lib.lx_tune_set(kernel.encode(), M, N, K, names.index(vname)) == 0:  # 802: the order-class rule refuses it
            pick = vname
            break
    return {"key": f"{key.value.decode()} M={M} N={N} K={K}", "us": {k: v[0] for k, v in timed.items()}, "pick": pick}


def _close(lx, kernel, variant, M, N, K, tolerance):
    problem = Problem(M, N, K, 1, 0, 0)
    a, b = (torch.empty(M, N, dtype=torch.float32, device="cuda") for _ in range(2))
    assert lx.status("tune_run", kernel.encode(), 0, ctypes.byref(problem), a) == 0
    assert lx.status("tune_run", kernel.encode(), variant, ctypes.byref(problem), b) == 0
    torch.cuda.synchronize()
    return ((a - b).norm() / a.norm().clamp_min(1e-30)).item() <= tolerance


def table(lx, problems, repeats=7):
    """tune() over [(kernel, M, N, K), ...]; returns the list of its results."""
    return [tune(lx, *p, repeats=repeats) for p in problems]


def main(argv):
    if len(argv) < 4 or len(argv) % 4:
        sys.exit(__doc__)
    lx = load_hip()
    for i in range(0, len(argv), 4):
        print(json.dumps(tune(lx, argv[i], int(argv[i + 1]), int(argv[i + 2]), int(argv[i + 3]))), flush=True)


if __name__ == "__main__":
    main(sys.argv[1:])
