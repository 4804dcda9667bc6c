#!/usr/bin/env python3
"""Measures the decode matrix-product path on one MI355X: weight-stream GB/s and fraction of the 8 TB/s HBM peak.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--cases all|headline|gemv|layer] [--no-cpu]
    python bench.py --pmc-probe      (for rocprofv3 --pmc: a plain copy of known size, then headline launches)

A step is one pass of the hot path over one batch: one lx_gemv_w call (the headline), one skinny GEMM, or one
routed-experts step, always on a weight copy that was not touched recently (the copies rotate through more
than 512 MB, past the 256 MB Infinity Cache, so every step streams from HBM). The K timed steps are recorded
once into a HIP graph through the library's own lx_rt_capture_* entry points (as the engine runs its decode
steps) and the graph is launched between two HIP events on its stream; W untimed steps run first.

Prints one JSON line. `value` is the headline case (INT8 weight-only GEMV, W 14336 x 4096, M = 1, bf16 x);
`cases` lists every measured case (by default one per benchmark configuration: C1, C2 int8 / fp8 at M = 1, 4, 16, 64 in
both modes, C3 M = 1, 8, C4 T = 1, 8, 32, 64, C5 and its four dense products) with its own time, GB/s and fraction of peak. Bytes per step are the
algorithmic bytes: weights + scales + x + y (bench/bench_gemv.py:51-56 of the reference uses the same count).
`floor` states what the memory system allows at these sizes, measured the same way in the same run: an empty launch,
and a plain read of the same weight copies (lx_probe_read: the GEMV's access pattern without the product); a GEMV case
carries `floor_us` (the plain read of its bytes) and `vs_floor` (its time over that).
"""

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0


def algorithmic_bytes_gemv(fmt, M, N, K, y_bytes=4):
    w = {"bf16": 2 * N * K, "int8": N * K, "fp8": N * K, "nvfp4": N * K // 2}[fmt]
    s = {"bf16": 0, "int8": 4 * N, "fp8": 4 * N, "nvfp4": N * K // 16 + 4}[fmt]
    return w + s + M * K * 2 + M * N * y_bytes


class Timer:
    """K steps captured into one graph, launched between two timed HIP events on the capture stream."""

    def __init__(self, lx, torch):
        self.lx, self.torch = lx, torch
        self.stream = torch.cuda.Stream()
        lx.reserve_stream(self.stream.cuda_stream)  # what lx_rt_stream_create gives the engine's own streams
        lib = lx.lib
        self.ev = []
        for _ in range(2):
            e = ctypes.c_void_p()
            assert lib.lx_rt_event_create_timed(ctypes.byref(e)) == 0
            self.ev.append(e)

    def run(self, step, steps, warmup, repeats=5):
        """step(i) issues step i on the current stream. Returns the median microseconds per step."""
        torch, lib = self.torch, self.lx.lib
        with torch.cuda.stream(self.stream):
            s = ctypes.c_void_p(self.stream.cuda_stream)
            for i in range(warmup):
                step(i)
            torch.cuda.synchronize()
            assert lib.lx_rt_capture_begin(s) == 0
            for i in range(steps):
                step(warmup + i)
            graph = ctypes.c_void_p()
            assert lib.lx_rt_capture_end(s, ctypes.byref(graph)) == 0
            assert lib.lx_rt_graph_launch(graph, s) == 0  # untimed: uploads the graph
            torch.cuda.synchronize()
            times = []
            for _ in range(repeats):
                torch.cuda.synchronize()
                assert lib.lx_rt_event_record(self.ev[0], s) == 0
                assert lib.lx_rt_graph_launch(graph, s) == 0
                assert lib.lx_rt_event_record(self.ev[1], s) == 0
                torch.cuda.synchronize()
                ms = ctypes.c_float()
                assert lib.lx_rt_event_elapsed(self.ev[0], self.ev[1], ctypes.byref(ms)) == 0
                times.append(ms.value * 1e3 / steps)
            assert lib.lx_rt_graph_destroy(graph) == 0
        times.sort()
        return times[len(times) // 2]


def make_gemv_case(lx, torch, fmt, M, N, K, seed, entry, invariant=False, math=0):
    """Returns (step, bytes_per_step, cleanup-free holder). Weight copies: one quantised master, cloned."""
    from dromos_amd.abi import DTYPE, F32, FORMATS
    from dromos_amd.formats import Weight, master_weight, quantize_with

    g = torch.Generator(device="cpu").manual_seed(seed)
    master = master_weight(N, K, g).cuda()
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w0 = quantize_with(lx, master, FORMATS[fmt])
    del master
    per_copy = w0.nbytes()
    copies = max(3, -(-(640 << 20) // per_copy))
    ws = [w0] + [Weight(w0.fmt, w0.data.clone(), None if w0.scale is None else w0.scale.clone(), w0.glob) for _ in range(copies - 1)]
    structs = [w.lx() for w in ws]
    ptrs = [ctypes.pointer(s) for s in structs]
    y = torch.empty(M, N, dtype=torch.float32, device="cuda")
    nbytes = algorithmic_bytes_gemv(fmt, M, N, K)
    ws_buf = torch.empty(max(int(lx.size("gemm_workspace_bytes", M, K, math)), 256), dtype=torch.uint8, device="cuda")

    def floor_step(i, flat=[]):
        # A plain read of the same number of bytes (weights + scales) from a flat buffer of rotating copies.
        if not flat:
            flat.append(torch.empty(copies * ((per_copy + 255) // 256 * 256), dtype=torch.uint8, device="cuda"))
        at = (i % copies) * ((per_copy + 255) // 256 * 256)
        st = lx.status("probe_read", flat[0][at:], ctypes.c_int64(per_copy // 16 * 16))
        assert st == 0, st

    def step(i):
        p = ptrs[i % copies]
        if entry == "gemv_w":
            st = lx.status("gemv_w", x, DTYPE[x.dtype], K, p, None, F32, y, F32, N, M, N, K, 1.0, 0.0)
        elif entry == "gemm_skinny":
            st = lx.status("gemm_skinny", x, DTYPE[x.dtype], K, p, None, F32, y, F32, N, M, N, K, 1.0, 0.0)
        else:
            st = lx.status("gemm_w", x, DTYPE[x.dtype], K, p, math, None, F32, y, F32, N, M, N, K, 1.0, 0.0, ws_buf)
        assert st == 0, st

    step.floor = floor_step
    return step, nbytes, (ws, structs, ptrs, x, y, ws_buf)


def make_bf16x_case(lx, torch, M, N, K, seed):
    """lx_gemv_bf16x on rotated encodings of one bf16 master. Bytes: the encoded weight + x + y."""
    from dromos_amd.abi import F32
    from dromos_amd.formats import master_weight

    g = torch.Generator(device="cpu").manual_seed(seed)
    master = master_weight(N, K, g).cuda()
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    n = int(lx.status("bf16x_bytes", master, N, K))
    enc = torch.empty(n, dtype=torch.uint8, device="cuda")
    assert lx.status("bf16x_encode", master, ctypes.c_int64(N), K, enc, ctypes.c_int64(n)) == 0
    torch.cuda.synchronize()
    del master
    copies = max(3, -(-(640 << 20) // n))
    encs = [enc] + [enc.clone() for _ in range(copies - 1)]
    y = torch.empty(M, N, dtype=torch.float32, device="cuda")
    nbytes = n + M * K * 2 + M * N * 4

    def step(i):
        st = lx.status("gemv_bf16x", x, 1, K, encs[i % copies], None, F32, y, F32, N, M, N, K, 1.0, 0.0)
        assert st == 0, st

    return step, nbytes, (encs, x, y)


def make_moe_case(lx, torch, fmt, T, E, L, I, top_k, seed, steps_total):
    """A routed-experts step (route + experts) on bf16 / quantised stacks. Bytes: distinct experts x per-expert
    bytes, averaged over the steps' seeded routings, + latent + out + routing."""
    from dromos_amd.abi import FORMATS
    from dromos_amd.formats import Weight

    g = torch.Generator(device="cpu").manual_seed(seed)
    gu = (torch.randn(E, 2 * I, L, generator=g) * 0.02).to(torch.bfloat16).cuda()
    dn = (torch.randn(E, L, I, generator=g) * 0.02).to(torch.bfloat16).cuda()
    if fmt == "bf16":
        first = (Weight(0, gu), Weight(0, dn))
    else:
        from dromos_amd.formats import alloc_quantized

        pair = []
        for w, n, k in ((gu, 2 * I, L), (dn, L, I)):
            out = alloc_quantized(FORMATS[fmt], E * n, k, "cuda")
            s = out.lx()
            lx("quantize_weight", w.view(E * n, k), ctypes.pointer(s), ctypes.c_int64(E * n), k)
            pair.append(out)
        first = tuple(pair)
        del gu, dn
    # Rotating copies of the stacks at other addresses: at least four, and enough that the steps between two uses of one
    # copy stream more than 640 MB (the Infinity Cache holds 256 MB), however few experts a step touches.
    step_bytes = min(E, T * top_k) * (first[0].nbytes() + first[1].nbytes()) // E
    copies = max(4, -(-(640 << 20) // step_bytes))
    clone = lambda w: Weight(w.fmt, w.data.clone(), None if w.scale is None else w.scale.clone(), w.glob)  # noqa: E731
    stacks = [first] + [(clone(first[0]), clone(first[1])) for _ in range(copies - 1)]
    per_expert = (stacks[0][0].nbytes() + stacks[0][1].nbytes()) // E
    n_routings = max(8, steps_total)
    logits = torch.randn(n_routings, T, E, generator=g).cuda()
    latent = torch.randn(T, L, generator=g).to(torch.bfloat16).cuda()
    ids = torch.empty(n_routings, T, top_k, dtype=torch.int32, device="cuda")
    weights = torch.empty(n_routings, T, top_k, dtype=torch.float32, device="cuda")
    ent = torch.empty(T, device="cuda")
    conf = torch.empty(T, device="cuda")
    for r in range(n_routings):
        lx("moe_route", logits[r], None, ids[r], weights[r], ent, conf, T, E, top_k)
    distinct = sum(len(set(ids[r].flatten().tolist())) for r in range(n_routings)) / n_routings
    out = torch.empty(T, L, dtype=torch.float32, device="cuda")
    decode = T <= 8
    if decode:
        nws = int(lx.size("moe_decode_workspace_bytes", T, I, top_k))
    else:
        fn = lx.lib.lx_moe_grouped_workspace_bytes
        fn.restype = ctypes.c_int64
        nws = int(fn(T, L, I, E, top_k, 0))
    ws = torch.empty(max(nws, 256), dtype=torch.uint8, device="cuda")
    structs = [(a.lx(), b.lx()) for a, b in stacks]
    ptrs = [(ctypes.pointer(a), ctypes.pointer(b)) for a, b in structs]
    nbytes = distinct * per_expert + T * L * 2 + T * L * 4 + T * E * 4 + T * top_k * 8

    def step(i):
        r = i % n_routings
        gu, dn = ptrs[i % copies]
        st = lx.status("moe_route", logits[r], None, ids[r], weights[r], ent, conf, T, E, top_k)
        assert st == 0, st
        if decode:
            st = lx.status("moe_experts_decode", latent, ids[r], weights[r], gu, dn, out, ws, T, L, I, top_k)
        else:
            st = lx.status("moe_experts_grouped", latent, ids[r], weights[r], gu, dn, 0, out, ws, T, L, I, E, top_k)
        assert st == 0, st

    return step, nbytes, (stacks, structs, ptrs, logits, latent, ids, weights, out, ws), distinct


def cpu_baseline(torch, fmt, M, N, K, seed, seconds=12.0):
    """The same GEMV on the host cores: the reference's own CPU backend when oracle/_ref holds it (kind
    "reference"), else this repository's plain-C restatement (kind "port"). A bounded sample: calls are
    repeated on rotated weight copies (1 GiB in all, past any last-level cache) for about `seconds`."""
    from dromos_amd.abi import DTYPE, F32, FORMATS, Kernels
    from dromos_amd.formats import Weight, master_weight, quantize_with

    # One thread per physical core, at most the 16 a one-GPU box is given.
    physical = physical_cores()
    threads = min(16, physical)
    os.environ.setdefault("LX_THREADS", str(threads))
    os.environ.setdefault("OMP_NUM_THREADS", str(threads))
    ref = ROOT / "oracle" / "_ref" / "libdromos_cpu.so"
    port = ROOT / "oracle" / "liboracle.so"
    if ref.exists():
        lib, kind = Kernels(ref, "cpu"), "reference"
    elif port.exists():
        lib, kind = Kernels(port, "cpu"), "port"
    else:
        return None
    threads = int(os.environ["LX_THREADS"]) if kind == "reference" else int(os.environ["OMP_NUM_THREADS"])
    g = torch.Generator(device="cpu").manual_seed(seed)
    master = master_weight(N, K, g)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w0 = quantize_with(lib, master, FORMATS[fmt])
    copies = max(2, -(-(1 << 30) // w0.nbytes()))
    ws = [w0] + [Weight(w0.fmt, w0.data.clone(), None if w0.scale is None else w0.scale.clone(), w0.glob) for _ in range(copies - 1)]
    structs = [w.lx() for w in ws]
    y = torch.empty(M, N, dtype=torch.float32)
    nbytes = algorithmic_bytes_gemv(fmt, M, N, K)

    def call(i):
        st = lib.status("gemv_w", x, DTYPE[x.dtype], K, ctypes.pointer(structs[i % copies]), None, F32, y, F32, N, M, N, K, 1.0, 0.0)
        assert st == 0

    for i in range(3):
        call(i)
    times, i, t_end = [], 3, time.perf_counter() + seconds
    while time.perf_counter() < t_end and len(times) < 200000:
        t0 = time.perf_counter()
        call(i)
        times.append(time.perf_counter() - t0)
        i += 1
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": round(nbytes / med / 1e9, 2),
        "unit": "GB/s",
        "cores": threads,
        "kind": kind,
        "sample": f"{len(times)} calls of lx_gemv_w {fmt} {N}x{K} M={M} on {copies} rotated weight copies, median {med * 1e6:.0f} us/call, "
                  f"{threads} threads; the host has {physical_cores()} physical cores ({os.cpu_count()} logical cpus)",
    }


def physical_cores():
    """Distinct (package, core) pairs of /proc/cpuinfo; the logical count where that file does not say."""
    seen, package = set(), None
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("physical id"):
                package = line.split(":")[1].strip()
            elif line.startswith("core id"):
                seen.add((package, line.split(":")[1].strip()))
    except OSError:
        pass
    return len(seen) or (os.cpu_count() or 1)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cases", default="all", choices=["headline", "gemv", "all", "layer", "moe"])
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="no timing: one 256 MiB device copy (the counters' yardstick), then eager launches of the headline "
                         "GEMV, the 16- and 64-row products, the one- and eight-token experts and the 32-token grouped experts")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus N with N > 1 is not supported (one MI355X per box)")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from dromos_amd.abi import load_hip

    lx = load_hip()  # raises when the library is not built: there is no fallback
    if args.pmc_probe:
        a = torch.zeros(256 << 20, dtype=torch.uint8, device="cuda")
        b = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        for _ in range(3):
            a.copy_(b)  # reads 256 MiB and writes 256 MiB
        del a, b
        probe = {"copy_bytes_read": 256 << 20, "copy_bytes_written": 256 << 20, "launches": {}}

        def launches(name, step, nbytes, n):
            for i in range(n):
                step(i)
            torch.cuda.synchronize()
            probe["launches"][name] = {"algorithmic_bytes_per_step": int(nbytes), "steps": n}

        step, nbytes, keep = make_gemv_case(lx, torch, "int8", 1, 14336, 4096, 1001, "gemv_w")
        launches("C2 int8 M=1 (gemv_stream_kernel)", step, nbytes, 20)
        del keep
        for M in (16, 64):
            step, nbytes, keep = make_gemv_case(lx, torch, "int8", M, 14336, 4096, 1000 + M, "gemm_w")
            launches(f"C2 int8 M={M} (walk_kernel)", step, nbytes, 10)
            del keep
        os.environ["LX_BATCH_INVARIANT"] = "1"
        step, nbytes, keep = make_gemv_case(lx, torch, "int8", 4, 14336, 4096, 1004, "gemv_w")
        launches("C2 int8 M=4 batch-invariant (tile16_kernel)", step, nbytes, 10)
        del keep
        os.environ.pop("LX_BATCH_INVARIANT", None)
        step, nbytes, keep = make_gemv_case(lx, torch, "fp8", 64, 6144, 4096, 5064, "gemm_w")
        launches("fp8 6144x4096 M=64 (slab_kernel + slab_reduce_kernel)", step, nbytes, 10)
        del keep
        torch.cuda.empty_cache()
        step, nbytes, keep, _ = make_moe_case(lx, torch, "bf16", 1, 64, 2048, 1024, 8, 3001, 16)
        launches("C4 moe bf16 T=1 (route + decode_gate_up + decode_down)", step, nbytes, 16)
        del keep
        torch.cuda.empty_cache()
        step, nbytes, keep, _ = make_moe_case(lx, torch, "bf16", 8, 64, 2048, 1024, 8, 3008, 8)
        launches("C4 moe bf16 T=8 (route + decode_gate_up + decode_down)", step, nbytes, 8)
        del keep
        torch.cuda.empty_cache()
        step, nbytes, keep, _ = make_moe_case(lx, torch, "fp8", 32, 128, 4096, 1536, 8, 5032, 8)
        launches("C5 moe fp8 T=32 E=128 (route + group + grouped_gate_up + grouped_down + grouped_sum)", step, nbytes, 8)
        del keep
        print(json.dumps({"pmc_probe": probe}))
        return
    timer = Timer(lx, torch)
    K_STEPS, W = args.steps, args.warmup

    cases = []
    floors = {}

    def empty_step(i):
        assert lx.status("probe_empty") == 0

    floors["empty_launch_us"] = round(timer.run(empty_step, K_STEPS, W), 3)

    def run_gemv(name, fmt, M, N, K, seed, entry="gemv_w", invariant=False, math=0):
        if invariant:
            os.environ["LX_BATCH_INVARIANT"] = "1"
        else:
            os.environ.pop("LX_BATCH_INVARIANT", None)
        step, nbytes, keep = make_gemv_case(lx, torch, fmt, M, N, K, seed, entry, math=math)
        us = timer.run(step, K_STEPS, W)
        os.environ.pop("LX_BATCH_INVARIANT", None)
        key = f"read_{fmt}_{N}x{K}_us"
        if key not in floors:
            floors[key] = round(timer.run(step.floor, K_STEPS, W), 3)
        gbps = nbytes / us / 1e3
        case = {"case": name, "entry": "lx_" + entry, "format": fmt, "math": ["bf16", "int8", "fp8", "fp4"][math], "M": M, "N": N, "K": K,
                "batch_invariant": invariant,
                "us_per_step": round(us, 3), "bytes_per_step": int(nbytes), "GBps": round(gbps, 1),
                "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "floor_us": floors[key], "vs_floor": round(us / floors[key], 3)}
        cases.append(case)
        del keep
        torch.cuda.empty_cache()
        return case

    def run_moe(name, fmt, T, E, L, I, top_k, seed):
        step, nbytes, keep, distinct = make_moe_case(lx, torch, fmt, T, E, L, I, top_k, seed, min(K_STEPS + W, 64))
        us = timer.run(step, K_STEPS, W)
        gbps = nbytes / us / 1e3
        case = {"case": name, "entry": "lx_moe_route + lx_moe_experts_" + ("decode" if T <= 8 else "grouped"), "format": fmt,
                "T": T, "E": E, "L": L, "I": I, "top_k": top_k, "distinct_experts": round(distinct, 2),
                "us_per_step": round(us, 3), "bytes_per_step": int(nbytes), "GBps": round(gbps, 1),
                "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4)}
        cases.append(case)
        del keep
        torch.cuda.empty_cache()
        return case

    def run_layer():
        """C5: the matrix set of one hybrid decode layer at 32 streams in FP8, back to back: four dense products
        (lx_gemm_w, BF16 math on fp8 weights) and the routed experts (E = 128, top-8, fp8 stacks)."""
        dense = [("qkv", 6144, 4096), ("o", 4096, 4096), ("in_proj", 16384, 4096), ("out_proj", 4096, 8192)]
        parts, nbytes, keep = [], 0, []
        for i, (_, N, K) in enumerate(dense):
            step, nb, k = make_gemv_case(lx, torch, "fp8", 32, N, K, 5000 + i, "gemm_w")
            parts.append(step)
            nbytes += nb
            keep.append(k)
        moe_step, moe_bytes, k, distinct = make_moe_case(lx, torch, "fp8", 32, 128, 4096, 1536, 8, 5032, min(K_STEPS + W, 64))
        keep.append(k)
        nbytes += moe_bytes

        def step(i):
            for p in parts:
                p(i)
            moe_step(i)

        us = timer.run(step, min(K_STEPS, 50), min(W, 5))
        gbps = nbytes / us / 1e3
        cases.append({"case": "C5 fp8 layer, 32 streams", "entry": "4 x lx_gemm_w + lx_moe_route + lx_moe_experts_grouped", "format": "fp8",
                      "M": 32, "distinct_experts": round(distinct, 2), "us_per_step": round(us, 3), "bytes_per_step": int(nbytes),
                      "GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4)})
        del keep
        torch.cuda.empty_cache()

    head = run_gemv("C2 int8 M=1", "int8", 1, 14336, 4096, 1001)
    if args.cases in ("gemv", "all"):
        run_gemv("C1 bf16 M=1", "bf16", 1, 4096, 4096, 0)
        run_gemv("C2 fp8 M=1", "fp8", 1, 14336, 4096, 1001)
        run_gemv("C3 nvfp4 M=1", "nvfp4", 1, 4096, 14336, 2001)
        run_gemv("C2 int8 M=4", "int8", 4, 14336, 4096, 1004)
        run_gemv("C2 fp8 M=4", "fp8", 4, 14336, 4096, 1004)
        run_gemv("C3 nvfp4 M=8", "nvfp4", 8, 4096, 14336, 2008)
        run_gemv("C3 nvfp4 M=8 invariant", "nvfp4", 8, 4096, 14336, 2008, invariant=True)
    if args.cases == "all":
        for fmt in ("int8", "fp8"):
            for M in (16, 64):
                for inv in (False, True):
                    run_gemv(f"C2 {fmt} M={M}" + (" invariant" if inv else ""), fmt, M, 14336, 4096, 1000 + M, entry="gemm_w", invariant=inv)
            for M in (1, 4):
                run_gemv(f"C2 {fmt} M={M} invariant", fmt, M, 14336, 4096, 1000 + M, invariant=True)
        for M in (1, 16, 64):
            # Not one of the headline configurations: the low-precision math of the same product (activations quantised per token
            # inside the call, exact int32 sums); the bytes are the weight-only count.
            run_gemv(f"C2 int8 M={M} INT8 math", "int8", M, 14336, 4096, 1000 + M, entry="gemm_w", math=1)
            run_gemv(f"C2 fp8 M={M} FP8 math", "fp8", M, 14336, 4096, 1000 + M, entry="gemm_w", math=2)
        for N, K in ((4096, 4096), (14336, 4096)):
            # Not a headline configuration: the lossless 12-bit form of bf16 weights; the bytes are the encoding's, so
            # GB/s is what the kernel streams and us_per_step compares with the bf16 product of the same shape.
            step, nbytes, keep = make_bf16x_case(lx, torch, 1, N, K, 7000 + N)
            us = timer.run(step, K_STEPS, W)
            cases.append({"case": f"bf16x {N}x{K} M=1", "entry": "lx_gemv_bf16x", "format": "bf16x", "M": 1, "N": N, "K": K,
                          "us_per_step": round(us, 3), "bytes_per_step": int(nbytes), "GBps": round(nbytes / us / 1e3, 1),
                          "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4), "bf16_bytes": 2 * N * K})
            del keep
            torch.cuda.empty_cache()
            if (N, K) != (4096, 4096):
                run_gemv(f"bf16 {N}x{K} M=1", "bf16", 1, N, K, 7000 + N)
        for T in (1, 8, 32, 64):
            run_moe(f"C4 moe bf16 T={T}", "bf16", T, 64, 2048, 1024, 8, 3000 + T)
        for name, N, K in (("QKV", 6144, 4096), ("O", 4096, 4096), ("in_proj", 16384, 4096), ("out_proj", 4096, 8192)):
            # The dense products of the C5 layer one by one (the layer case below runs them back to back with the experts).
            run_gemv(f"C5 fp8 M=32 {name} {N}x{K}", "fp8", 32, N, K, 5000 + N + K, entry="gemm_w")
        run_layer()
    elif args.cases == "headline":
        run_moe("C4 moe bf16 T=1", "bf16", 1, 64, 2048, 1024, 8, 3001)
    elif args.cases == "layer":
        run_layer()
    elif args.cases == "moe":
        for T in (1, 8, 32, 64):
            run_moe(f"C4 moe bf16 T={T}", "bf16", T, 64, 2048, 1024, 8, 3000 + T)

    result = {
        "metric": "weight-stream GB/s and % of HBM peak: M=1 GEMV and top-8 MoE decode",
        "value": head["GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K_STEPS,
        "warmup": W,
        "ms_per_step": round(head["us_per_step"] / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 weights, bf16 activations, f32 accumulate",
        "data": "synthetic: N(0, 0.02) bf16 masters quantised by lx_quantize_weight, x ~ N(0, 1) bf16, seeded",
        "config": {"workload": "C2: INT8 weight-only GEMV, W 14336x4096 (per-channel f32 scale), M=1 bf16 x, f32 y, "
                               "lx_gemv_w on rotated weight copies (> 512 MB)"},
        "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(head["GBps"] / HBM_PEAK_GBPS, 4), "traffic": load_traffic()},
        "floor": floors,
        "cases": cases,
    }
    if not args.no_cpu:
        # The headline shape for about 12 s, then the other formats' M = 1 configurations for about 4 s each.
        result["cpu_baseline"] = cpu_baseline(torch, "int8", 1, 14336, 4096, 1001)
        if result["cpu_baseline"] and args.cases in ("gemv", "all"):
            others = {}
            for name, fmt, N, K, seed in (("C1 bf16 M=1", "bf16", 4096, 4096, 0), ("C2 fp8 M=1", "fp8", 14336, 4096, 1001),
                                          ("C3 nvfp4 M=1", "nvfp4", 4096, 14336, 2001)):
                c = cpu_baseline(torch, fmt, 1, N, K, seed, seconds=4.0)
                others[name] = {"value": c["value"], "unit": c["unit"], "sample": c["sample"]}
            result["cpu_baseline"]["other_formats"] = others
    print(json.dumps(result))


def load_traffic():
    """HBM bytes per launch of the headline kernel from the committed rocprofv3 --pmc summary, or None."""
    p = ROOT / "profiles" / "gemv_w_int8_14336x4096_m1_traffic.txt"
    if not p.exists():
        return None
    for line in p.read_text().splitlines():
        if line.startswith("hbm_bytes_per_launch:"):
            return int(float(line.split(":", 1)[1]))
    return None


if __name__ == "__main__":
    main()
