"""GPU parity: the walk kernel of lx_gemm_w / lx_gemm_skinny (9 .. 64 bf16 activation rows, a wavefront walking a whole
tile) against float64 on the decoded values, and bit for bit against the tile kernels it replaces on the shapes it
takes: the variant table forces each family ("gemm_w_<format>": 0 = the tile kernels, 1 .. 3 = walk with 1, 2, 4 tiles
a workgroup, 4 / 5 = the tile kernels without / with the slab kernel, 6 = walks of single slices whose sums meet in the
stream's partial-tile buffer, 7 = a tile's slices split over the wavefronts of a workgroup), and no variant may change an output bit, a row's bits may not depend on the batch."""

import pytest
import torch

import checks
import ops
from dromos_amd.abi import FORMATS, MATH_BF16, MATH_FP8
from dromos_amd.formats import random_weight

pytestmark = pytest.mark.gpu
FMT = checks.FMT_NAMES
# K whose rows are whole slices of whole four-group walks in the format (what the kernel takes without its clamps), N with a ragged last tile
SHAPES = {"bf16": [(150, 512), (4096, 1024)], "int8": [(150, 1024), (4096, 2048)], "fp8": [(150, 1024), (4096, 4096)], "nvfp4": [(150, 2048), (4096, 4096)]}


def force(hip, fmt, M, N, K, variant):
    hip.lib.lx_tune_clear()
    if variant is not None:
        assert hip.lib.lx_tune_force(f"gemm_w_{fmt}".encode(), M, N, K, variant) == 0


@pytest.fixture(autouse=True)
def clear_table(hip):
    yield
    hip.lib.lx_tune_clear()


def test_variants_are_registered(hip):
    import ctypes

    hip.lib.lx_tune_variant_name.restype = ctypes.c_char_p
    for fmt in FMT:
        key = f"gemm_w_{fmt}".encode()
        assert hip.lib.lx_tune_variants(key) == 8
        assert [hip.lib.lx_tune_variant_name(key, v).decode() for v in range(8)] == ["tiles", "walk1", "walk2", "walk4", "window", "slab", "walkparts", "walksplit"]
        assert all(hip.lib.lx_tune_set(key, 32, 4096, 4096, v) == 0 for v in range(8))  # none changes a sum: all admitted
        assert hip.lib.lx_tune_set(key, 32, 4096, 4096, 8) == 803


@pytest.mark.parametrize("M", [9, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("fmt", FMT)
def test_every_variant_gives_the_same_bits(hip, fmt, M):
    for N, K in SHAPES[fmt]:
        g = torch.Generator().manual_seed(M + N)
        w = random_weight(FORMATS[fmt], N, K, N + K)
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        bias = torch.randn(N, generator=g)
        want = ops.gemv_reference(x, w.dense(), bias, 1.0, 0.0, None)
        wd, xd, bd = w.to("cuda"), x.cuda(), bias.cuda()
        outs = {}
        for variant in (0, 1, 2, 3, 4, 5, 6, 7, None):
            force(hip, fmt, M, N, K, variant)
            y = torch.full((M, N), float("nan"), device="cuda")
            outs[variant] = ops.gemm_w(hip, xd, wd, MATH_BF16, bias=bd, y=y).clone()
        checks.check_product(outs[0].cpu(), want)
        for variant, out in outs.items():
            assert torch.equal(out.view(torch.int32), outs[0].view(torch.int32)), f"variant {variant} changes bits at {fmt} {N}x{K} M={M}"


# Rows that are not whole walks: load steps that are not a multiple of 16 (11 and 21.5 groups of four) and a last step
# cut short by K (bf16 43.25 steps, one-byte formats 22.25).
# The last of each: a quarter of a step (NVFP4: one step) past 16, so that three of the walk's last four groups hold nothing.
RAGGED = {"bf16": [(150, 1408), (2048, 1384), (300, 520)], "int8": [(150, 1408), (2048, 5504), (300, 1424), (300, 1040)],
          "fp8": [(150, 1408), (2048, 5504), (300, 1424), (300, 1040)], "nvfp4": [(150, 2688), (2048, 5504), (300, 2176)]}


@pytest.mark.parametrize("M", [9, 24, 33, 64])
@pytest.mark.parametrize("fmt", FMT)
def test_rows_that_are_not_whole_walks(hip, fmt, M):
    for N, K in RAGGED[fmt]:
        g = torch.Generator().manual_seed(M + N)
        w = random_weight(FORMATS[fmt], N, K, N + K)
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        bias = torch.randn(N, generator=g)
        want = ops.gemv_reference(x, w.dense(), bias, 1.0, 0.0, None)
        wd, xd, bd = w.to("cuda"), x.cuda(), bias.cuda()
        outs = {}
        for variant in (0, 1, 2, 3, 6, 7, None):
            force(hip, fmt, M, N, K, variant)
            y = torch.full((M, N), float("nan"), device="cuda")
            outs[variant] = ops.gemm_w(hip, xd, wd, MATH_BF16, bias=bd, y=y).clone()
        checks.check_product(outs[0].cpu(), want)
        for variant, out in outs.items():
            assert torch.equal(out.view(torch.int32), outs[0].view(torch.int32)), f"variant {variant} changes bits at {fmt} {N}x{K} M={M}"


@pytest.mark.parametrize("fmt", FMT)
def test_walk_rows_do_not_depend_on_the_batch(hip, fmt):
    N, K = SHAPES[fmt][1]
    w = random_weight(FORMATS[fmt], N, K, 3).to("cuda")
    g = torch.Generator().manual_seed(8)
    x = torch.randn(64, K, generator=g).to(torch.bfloat16).cuda()
    force(hip, fmt, 64, N, K, 3)
    full = ops.gemm_skinny(hip, x, w)
    for M in (1, 8, 9, 16, 31, 40):
        for variant in (2, 3, 7):
            force(hip, fmt, M, N, K, variant)
            part = ops.gemm_skinny(hip, x[:M].contiguous(), w)
            assert torch.equal(part, full[:M]), f"rows of an M={M} call (variant {variant}) differ from the rows of the M=64 call"


@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (-1.5, 1.0)])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias_dtype", [None, torch.bfloat16])
@pytest.mark.parametrize("fmt", FMT)
def test_walk_epilogue_matrix(hip, fmt, bias_dtype, y_dtype, alpha, beta):
    # Both epilogue forms (the 16-byte store, the element-wise one), strided x and y, nothing written past N.
    N, K = SHAPES[fmt][0]
    M, pad = 20, 8
    g = torch.Generator().manual_seed(5)
    w = random_weight(FORMATS[fmt], N, K, 6)
    xb = torch.randn(M, K + pad, generator=g).to(torch.bfloat16)
    bias = None if bias_dtype is None else torch.randn(N, generator=g).to(bias_dtype)
    y0 = torch.randn(M, N + pad, generator=g).to(y_dtype)
    want = ops.gemv_reference(xb[:, :K], w.dense(), bias, alpha, beta, y0[:, :N])
    for variant in (0, 3, 7):
        force(hip, fmt, M, N, K, variant)
        y = y0.clone().cuda()
        ops.gemm_w(hip, xb.cuda(), w.to("cuda"), MATH_BF16, bias=None if bias is None else bias.cuda(), y=y, alpha=alpha, beta=beta,
                   ld_x=K + pad, ld_y=N + pad, N=N)
        checks.check_product(y.cpu()[:, :N], want)
        assert torch.equal(y.cpu()[:, N:], y0[:, N:]), "wrote past the N columns of y"
        if variant == 0:
            first = y.clone()
        else:
            assert torch.equal(y.view(torch.int16 if y_dtype == torch.bfloat16 else torch.int32),
                               first.view(torch.int16 if y_dtype == torch.bfloat16 else torch.int32))


def test_walk_under_a_quantised_math(hip):
    # The FP8 math on NVFP4 weights runs the BF16-math kernels on the activations' images with the rows' scales in the
    # epilogue: the walk kernel and the tile kernels agree there too.
    N, K, M = 4096, 4096, 32
    w = random_weight(FORMATS["nvfp4"], N, K, 4).to("cuda")
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).cuda()
    outs = []
    for variant in (0, 3, 7):
        force(hip, "nvfp4", M if variant != 7 else 16, N, K, variant)  # the split form takes NVFP4 up to 16 rows
        outs.append(ops.gemm_w(hip, x if variant != 7 else x[:16].contiguous(), w, MATH_FP8).clone())
    assert torch.equal(outs[0].view(torch.int32), outs[1].view(torch.int32))
    assert torch.equal(outs[0][:16].view(torch.int32), outs[2].view(torch.int32))


class TuneProblem(__import__("ctypes").Structure):
    _fields_ = [(n, __import__("ctypes").c_int) for n in ("M", "N", "K", "experts", "weight", "math")]


@pytest.mark.parametrize("fmt", FMT)
def test_tune_run_times_what_the_table_would_pick(hip, fmt):
    # engine/cuda/tunable.h:57-75: every variant of a runnable kernel runs on the kernel's own inputs and writes f32
    # [M, N]; the products' variants agree bit for bit, the GEMV's K splits within the sums' rounding.
    import ctypes

    N, K = SHAPES[fmt][1]
    for kernel, M, exact in ((f"gemm_w_{fmt}", 32, True), (f"gemv_w_{fmt}", 4, False)):
        p = TuneProblem(M, N, K, 1, 0, 0)
        outs = []
        for v in range(hip.lib.lx_tune_variants(kernel.encode())):
            out = torch.full((M, N), float("nan"), device="cuda")
            assert hip.status("tune_run", kernel.encode(), v, ctypes.byref(p), out) == 0, (kernel, v)
            torch.cuda.synchronize()
            assert torch.isfinite(out).all() and out.abs().max() > 0
            outs.append(out)
        for v, out in enumerate(outs):
            if exact:
                assert torch.equal(out.view(torch.int32), outs[0].view(torch.int32)), (kernel, v)
            else:
                assert ((out - outs[0]).norm() / outs[0].norm()).item() < 1e-5, (kernel, v)
        assert hip.lib.lx_tune_get(kernel.encode(), M, N, K) == -1  # running a variant leaves the table alone
    p = TuneProblem(32, N, K, 1, 0, 0)
    out = torch.zeros(32, N, device="cuda")
    assert hip.status("tune_run", b"attention", 0, ctypes.byref(p), out) == 801
    assert hip.status("tune_run", f"gemm_w_{fmt}".encode(), 99, ctypes.byref(p), out) == 801
    assert hip.status("tune_run", f"gemm_w_{fmt}".encode(), 0, ctypes.byref(TuneProblem(32, N, K, 8, 0, 0)), out) == 801  # stacks
    assert hip.status("tune_run", f"gemv_w_{fmt}".encode(), 0, ctypes.byref(TuneProblem(9, N, K, 1, 0, 0)), out) == 801  # M > 8


def test_the_tuner_times_checks_and_stores(hip):
    # dromos_amd/tune.py drives lx_tune_run / lx_tune_set as the engine's autotuner does (engine/cuda/tunable.h:57-75).
    from dromos_amd import tune

    try:
        got = tune.tune(hip, "gemm_w_fp8", 32, 2048, 4096, repeats=3)
        names = tune.variants(hip, "gemm_w_fp8")
        assert set(got["us"]) == set(names) and all(us > 0 for us in got["us"].values())
        assert got["pick"] in names and hip.lib.lx_tune_get(b"gemm_w_fp8", 32, 2048, 4096) == names.index(got["pick"])
        assert got["key"].startswith("gemm_w_fp8 ")
        split = tune.tune(hip, "gemv_w_int8", 4, 2048, 4096, repeats=3)  # the order-class rule admits one split for the shape
        assert split["pick"] in tune.variants(hip, "gemv_w_int8")
    finally:
        hip.lib.lx_tune_clear()


@pytest.mark.parametrize("fmt,N,K", [("fp8", 4096, 14336), ("nvfp4", 4096, 14336), ("bf16", 4096, 14336)])
def test_long_slices_in_several_slab_passes(hip, fmt, N, K):
    # Rows whose slices are too long for one LDS image: the slab kernel takes a slice in two or three launches, each going
    # on from the partial tiles of the one before; the sums are the one-pass chain's, bit for bit the other kernels'.
    w = random_weight(FORMATS[fmt], N, K, N + K)
    g = torch.Generator().manual_seed(K)
    wd = w.to("cuda")
    dense = w.dense()
    for M in (12, 33, 64):
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        outs = {}
        for variant in (0, 4, 5, 6, 7, None):
            force(hip, fmt, M, N, K, variant)
            outs[variant] = ops.gemm_w(hip, x.cuda(), wd, MATH_BF16).clone()
        checks.check_product(outs[5].cpu(), ops.gemv_reference(x, dense, None, 1.0, 0.0, None))
        for variant, out in outs.items():
            assert torch.equal(out.view(torch.int32), outs[4].view(torch.int32)), f"variant {variant} at {fmt} M={M}"
        # a row's bits are those of the row alone
        force(hip, fmt, 1, N, K, None)
        alone = ops.gemm_skinny(hip, x[M - 1 : M].cuda(), wd)
        assert torch.equal(alone[0].view(torch.int32), outs[None][M - 1].view(torch.int32))


@pytest.mark.parametrize("fmt,N,K", [("fp8", 8192, 7168), ("int8", 8192, 7168), ("nvfp4", 8192, 14336), ("bf16", 8192, 3584)])
def test_a_short_last_slice(hip, fmt, N, K):
    # 112 load steps in four slices of 32: the last slice is half as long as the others. Every walk takes it as the tile
    # kernels do (whole walks that start anywhere in the row, and walks of single slices).
    w = random_weight(FORMATS[fmt], N, K, N + K)
    g = torch.Generator().manual_seed(K)
    wd = w.to("cuda")
    dense = w.dense()
    for M in (16, 40, 64):
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        outs = {}
        for variant in (0, 1, 2, 3, 4, 6, None):
            force(hip, fmt, M, N, K, variant)
            outs[variant] = ops.gemm_w(hip, x.cuda(), wd, MATH_BF16).clone()
        checks.check_product(outs[0].cpu(), ops.gemv_reference(x, dense, None, 1.0, 0.0, None))
        for variant, out in outs.items():
            assert torch.equal(out.view(torch.int32), outs[0].view(torch.int32)), f"variant {variant} at {fmt} M={M}"
        force(hip, fmt, 1, N, K, None)
        alone = ops.gemm_skinny(hip, x[M - 1 : M].cuda(), wd)
        assert torch.equal(alone[0].view(torch.int32), outs[None][M - 1].view(torch.int32))


@pytest.mark.parametrize("fmt,N,K", [("fp8", 4096, 4096), ("int8", 4000, 4096), ("bf16", 2048, 2048), ("nvfp4", 4096, 4096), ("fp8", 4096, 8192)])
def test_a_tile_split_over_a_workgroup(hip, fmt, N, K):
    # Matrices of at most a tile per compute unit at 9 .. 32 rows: the rule takes the split form by itself (variant None),
    # and its bits are the tile kernels' (variant 0) and the whole walk's (variant 2), a row's those of the row alone.
    w = random_weight(FORMATS[fmt], N, K, N + K)
    g = torch.Generator().manual_seed(K + 1)
    wd = w.to("cuda")
    dense = w.dense()
    bias = torch.randn(N, generator=g)
    for M in (9, 16, 17, 32):
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        outs = {}
        for variant in (0, 2, 7, None):
            force(hip, fmt, M, N, K, variant)
            outs[variant] = ops.gemm_w(hip, x.cuda(), wd, MATH_BF16, bias=bias.cuda()).clone()
        checks.check_product(outs[None].cpu(), ops.gemv_reference(x, dense, bias, 1.0, 0.0, None))
        for variant, out in outs.items():
            assert torch.equal(out.view(torch.int32), outs[0].view(torch.int32)), f"variant {variant} at {fmt} M={M}"
        force(hip, fmt, 1, N, K, None)
        alone = ops.gemm_skinny(hip, x[M - 1 : M].cuda(), wd)
        force(hip, fmt, M, N, K, None)
        assert torch.equal(alone[0].view(torch.int32), ops.gemm_skinny(hip, x.cuda(), wd)[M - 1].view(torch.int32))
