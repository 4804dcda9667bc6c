"""GPU parity: the matrix-core products lx_gemm_w (BF16 math) and lx_gemm_skinny through the C ABI, against
float64 on the decoded values with bf16-rounded activations, against the CPU oracle at the headline decode shapes, and the
bitwise invariants: a row's bits do not depend on the batch, and in batch-invariant mode lx_gemv_w and lx_gemm_w
give the same bits for every row count from 1 up."""

import os

import pytest
import torch

import checks
import ops
from conftest import rel_l2
from dromos_amd.abi import FORMATS, MATH_BF16, MATH_FP4, MATH_FP8, MATH_INT8
from dromos_amd.formats import master_weight, quantize_with, random_weight

pytestmark = pytest.mark.gpu
FMT = checks.FMT_NAMES


def gemm_case(hip, fmt, M, N, K, seed, x_dtype=torch.bfloat16, bias_dtype=None, y_dtype=torch.float32, alpha=1.0, beta=0.0,
              entry="gemm_w"):
    g = torch.Generator().manual_seed(seed)
    w = random_weight(FORMATS[fmt], N, K, seed + 1)
    x = torch.randn(M, K, generator=g).to(x_dtype)
    bias = None if bias_dtype is None else torch.randn(N, generator=g).to(bias_dtype)
    y0 = torch.randn(M, N, generator=g).to(y_dtype)
    y = y0.clone() if beta != 0.0 else torch.full((M, N), float("nan"), dtype=y_dtype)
    call = ops.gemm_w if entry == "gemm_w" else ops.gemm_skinny
    kw = dict(bias=None if bias is None else bias.cuda(), y=y.cuda(), alpha=alpha, beta=beta)
    got = call(hip, x.cuda(), w.to("cuda"), **kw) if entry != "gemm_w" else call(hip, x.cuda(), w.to("cuda"), MATH_BF16, **kw)
    want = ops.gemv_reference(x.to(torch.bfloat16), w.dense(), bias, alpha, beta, y0)
    checks.check_product(got.cpu(), want)
    return got


@pytest.mark.parametrize("M", [1, 5, 9, 16, 17, 33, 64, 70, 130])
@pytest.mark.parametrize("fmt", FMT)
def test_gemm_w_every_m(hip, fmt, M):
    gemm_case(hip, fmt, M, 300, 1024, seed=M, bias_dtype=torch.float32)


@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, 0.0), (-1.5, 1.0)])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias_dtype", [None, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fmt", FMT)
def test_gemm_w_dtype_matrix(hip, fmt, x_dtype, bias_dtype, y_dtype, alpha, beta):
    gemm_case(hip, fmt, 20, 37, 544, seed=11, x_dtype=x_dtype, bias_dtype=bias_dtype, y_dtype=y_dtype, alpha=alpha, beta=beta)


@pytest.mark.parametrize("K", [16, 32, 48, 64, 128, 256, 272, 512, 544, 1024, 1040, 2064, 4096, 14336])
@pytest.mark.parametrize("fmt", FMT)
def test_gemm_w_k_boundaries(hip, fmt, K):
    # K around the load-step sizes (32 / 64 / 128 k per step), rows that end inside a step, and K = 48, whose
    # rows cannot be read 16 bytes at a time in every format (the plain kernel).
    gemm_case(hip, fmt, 12, 21, K, seed=K)


# The last two: rows that are not whole walks (K = 11 and 61 NVFP4 load steps) on matrices with the tiles for few,
# long slices: the tile kernel that reads its activations where they lie, in workgroups of at most 4 and 8 wavefronts.
@pytest.mark.parametrize("N,K", [(10304, 2048), (2048, 4096), (256, 6400), (8, 2048), (1, 512), (11008, 1408), (4096, 7808)])
@pytest.mark.parametrize("fmt", FMT)
def test_gemm_w_decode_shapes(hip, fmt, N, K):
    gemm_case(hip, fmt, 32, N, K, seed=N % 89)


def test_gemm_w_strided_and_untouched_padding(hip):
    for fmt in FMT:
        M, N, K, pad = 19, 300, 1024, 8
        g = torch.Generator().manual_seed(5)
        w = random_weight(FORMATS[fmt], N, K, 6)
        xb = torch.randn(M, K + pad, generator=g).to(torch.bfloat16)
        y0 = torch.randn(M, N + pad, generator=g)
        y = y0.clone().cuda()
        ops.gemm_w(hip, xb.cuda(), w.to("cuda"), MATH_BF16, y=y, alpha=2.0, beta=0.5, ld_x=K + pad, ld_y=N + pad, N=N)
        want = ops.gemv_reference(xb[:, :K], w.dense(), None, 2.0, 0.5, y0[:, :N])
        checks.check_product(y.cpu()[:, :N], want)
        assert torch.equal(y.cpu()[:, N:], y0[:, N:]), "wrote past the N columns of y"


def test_other_maths_and_arguments(hip):
    w = random_weight(FORMATS["int8"], 32, 64, 1).to("cuda")
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
    for math in (MATH_FP8, MATH_FP4):
        assert ops.gemm_w(hip, x, w, math, status=True) == 801  # int8 weights take the BF16 and INT8 maths
    w8 = random_weight(FORMATS["fp8"], 32, 64, 1).to("cuda")
    assert ops.gemm_w(hip, x, w8, MATH_FP8, status=True) == 0
    assert ops.gemm_w(hip, x, w8, MATH_FP4, status=True) == 801  # the FP4 math takes NVFP4 weights only
    w4 = random_weight(FORMATS["nvfp4"], 32, 64, 1).to("cuda")
    assert ops.gemm_w(hip, x, w4, MATH_FP8, status=True) == 0 and ops.gemm_w(hip, x, w4, MATH_FP4, status=True) == 0
    assert ops.gemm_w(hip, x, w4, MATH_INT8, status=True) == 801
    assert ops.gemm_w(hip, x, random_weight(FORMATS["bf16"], 32, 64, 1).to("cuda"), MATH_FP8, status=True) == 801
    assert ops.gemm_w(hip, x, w, MATH_INT8, status=True) == 0
    assert ops.gemm_w(hip, x, random_weight(FORMATS["fp8"], 32, 64, 1).to("cuda"), MATH_INT8, status=True) == 801  # int8 weights only
    assert ops.gemm_w(hip, x, w, 7, status=True) == 1
    assert ops.gemm_w(hip, x[:0], w, MATH_BF16, status=True) == 0
    assert ops.gemm_skinny(hip, x.float(), w, status=True) == 801  # bf16 activations only
    assert ops.gemm_skinny(hip, x, w, status=True) == 0


@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("N,K", [(1024, 2048), (300, 4096), (2048, 1024), (11008, 1408), (4096, 7808)])
def test_skinny_rows_do_not_depend_on_the_batch(hip, fmt, N, K):
    # engine/cuda/kernels.h:466-471: M = 1, 2, 8, 16, 32, 64 and across chunks of 64.
    w = random_weight(FORMATS[fmt], N, K, N + K).to("cuda")
    g = torch.Generator().manual_seed(N)
    x = torch.randn(100, K, generator=g).to(torch.bfloat16).cuda()
    bias = torch.randn(N, generator=g).cuda()
    full = ops.gemm_skinny(hip, x, w, bias=bias)
    for M in (1, 2, 8, 16, 32, 64):
        part = ops.gemm_skinny(hip, x[:M].contiguous(), w, bias=bias)
        assert torch.equal(part, full[:M]), f"rows of an M={M} call differ from the same rows of an M=100 call"
    for m in (0, 17, 63, 64, 99):
        alone = ops.gemm_skinny(hip, x[m : m + 1].contiguous(), w, bias=bias)
        assert torch.equal(alone[0], full[m]), f"row {m} alone differs from the row in the batch"
    assert torch.equal(ops.gemm_skinny(hip, x, w, bias=bias), full)  # and from run to run
    assert torch.equal(ops.gemm_w(hip, x, w, MATH_BF16, bias=bias), full)  # lx_gemm_w is the same kernel


@pytest.mark.parametrize("fmt", FMT)
def test_batch_invariant_mode_spans_gemv_and_gemm(hip, fmt):
    # With LX_BATCH_INVARIANT set, lx_gemv_w (M <= 8, bf16 x) and lx_gemm_w give a row the same bits whatever the
    # row count, 1 included; without it lx_gemv_w takes the streaming kernel (its own, also batch-independent, sums).
    N, K = 512, 4096
    w = random_weight(FORMATS[fmt], N, K, 3).to("cuda")
    x = torch.randn(64, K, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).cuda()
    os.environ["LX_BATCH_INVARIANT"] = "1"
    try:
        ref64 = ops.gemm_w(hip, x, w, MATH_BF16)
        for M in (1, 4, 8):
            y = ops.gemv_w(hip, x[:M].contiguous(), w)
            assert torch.equal(y, ref64[:M]), f"M={M}"
        assert torch.equal(ops.gemm_w(hip, x[:16].contiguous(), w, MATH_BF16), ref64[:16])
    finally:
        del os.environ["LX_BATCH_INVARIANT"]
    os.environ["LX_BATCH_INVARIANT"] = "0"  # starts with '0': off
    try:
        y1 = ops.gemv_w(hip, x[:1].contiguous(), w)
    finally:
        del os.environ["LX_BATCH_INVARIANT"]
    assert torch.equal(y1, ops.gemv_w(hip, x[:1].contiguous(), w))
    assert rel_l2(y1, ref64[:1]) < 1e-5


@pytest.mark.parametrize("fmt,M", [("int8", 16), ("int8", 64), ("fp8", 16), ("fp8", 64)])
def test_baseline_config_against_the_oracle(hip, oracle, fmt, M):
    N, K = 14336, 4096
    g = torch.Generator().manual_seed(1000 + M)
    master = master_weight(N, K, g)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = quantize_with(hip, master.cuda(), FORMATS[fmt])
    y = ops.gemm_w(hip, x.cuda(), w, MATH_BF16)
    want = ops.gemm_w(oracle, x, w.to("cpu"), MATH_BF16)
    err = rel_l2(y.cpu(), want)
    assert err <= 1e-2 and err <= 1e-4, err


# ---- the INT8 math: exact sums, so every output equals the oracle's bit for bit ---------------------------


@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (5, 300, 4096), (12, 37, 1030), (16, 96, 512), (17, 2048, 1024), (40, 300, 528),
                                   (64, 1024, 2048), (70, 96, 4096), (130, 50, 1040), (33, 21, 48)])
def test_int8_math_is_bit_exact(hip, oracle, M, N, K, x_dtype, y_dtype):
    g = torch.Generator().manual_seed(M * 7 + K)
    x = torch.randn(M, K, generator=g).to(x_dtype)
    x[M // 2] = 0
    w = random_weight(FORMATS["int8"], N, K, M + 3)
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g).to(y_dtype)
    want = ops.gemm_w(oracle, x, w, MATH_INT8, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    got = ops.gemm_w(hip, x.cuda(), w.to("cuda"), MATH_INT8, bias=bias.cuda(), y=y0.clone().cuda(), alpha=1.25, beta=-0.5)
    assert torch.equal(got.cpu().view(torch.int16 if y_dtype == torch.bfloat16 else torch.int32),
                       want.view(torch.int16 if y_dtype == torch.bfloat16 else torch.int32))


@pytest.mark.parametrize("M", [1, 16, 64])
def test_int8_math_baseline_shape(hip, oracle, M):
    # C2: W 14336 x 4096. Rows of the result do not depend on how many rows ride along (the sums are exact).
    N, K = 14336, 4096
    g = torch.Generator().manual_seed(M)
    x = torch.randn(64, K, generator=g).to(torch.bfloat16)
    w = random_weight(FORMATS["int8"], N, K, 5)
    full = ops.gemm_w(hip, x.cuda(), w.to("cuda"), MATH_INT8)
    part = ops.gemm_w(hip, x[:M].contiguous().cuda(), w.to("cuda"), MATH_INT8)
    assert torch.equal(part, full[:M])
    if M == 16:
        want = ops.gemm_w(oracle, x[:M].contiguous(), w, MATH_INT8)
        assert torch.equal(part.cpu().view(torch.int32), want.view(torch.int32))


# ---- the FP8 math: exact e4m3 products, f32 sums on the device against the oracle's exact sums ------------


@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (5, 300, 4096), (12, 37, 1030), (16, 96, 512), (17, 2048, 1024), (40, 300, 528),
                                   (64, 1024, 2048), (70, 96, 4096), (130, 50, 1040), (33, 21, 48)])
def test_fp8_math_against_the_oracle(hip, oracle, M, N, K, x_dtype, y_dtype):
    g = torch.Generator().manual_seed(M * 7 + K)
    x = torch.randn(M, K, generator=g).to(x_dtype)
    x[M // 2] = 0
    w = random_weight(FORMATS["fp8"], N, K, M + 3)
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g).to(y_dtype)
    want = ops.gemm_w(oracle, x, w, MATH_FP8, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    got = ops.gemm_w(hip, x.cuda(), w.to("cuda"), MATH_FP8, bias=bias.cuda(), y=y0.clone().cuda(), alpha=1.25, beta=-0.5)
    # Tolerance of the path: relative L2 of 1e-2 at most; the matrix instruction's f32 sums of the exact products come
    # out near 1e-5 at K = 4096 (bf16 outputs: one rounding of the result, 2^-9 relative).
    err = rel_l2(got, want)
    assert err <= (4e-3 if y_dtype == torch.bfloat16 else 1e-4), err


def test_fp8_math_rows_do_not_depend_on_the_batch(hip):
    N, K = 2048, 4096
    g = torch.Generator().manual_seed(2)
    x = torch.randn(64, K, generator=g).to(torch.bfloat16).cuda()
    w = random_weight(FORMATS["fp8"], N, K, 5).to("cuda")
    full = ops.gemm_w(hip, x, w, MATH_FP8)
    for M in (1, 7, 16, 33):
        part = ops.gemm_w(hip, x[:M].contiguous(), w, MATH_FP8)
        assert torch.equal(part, full[:M]), M


# ---- the FP8 math on NVFP4 weights and the FP4 math: quantised activations times exact weight values ----------


@pytest.mark.parametrize("math", [MATH_FP8, MATH_FP4])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (5, 300, 4096), (12, 37, 1040), (16, 96, 512), (17, 2048, 1024), (40, 300, 528),
                                   (64, 1024, 2048), (130, 50, 1040), (33, 21, 48)])
def test_nvfp4_under_the_fp8_and_fp4_maths(hip, oracle, math, M, N, K, x_dtype, y_dtype):
    g = torch.Generator().manual_seed(M * 7 + K + math)
    x = torch.randn(M, K, generator=g).to(x_dtype)
    x[M // 2] = 0
    w = random_weight(FORMATS["nvfp4"], N, K, M + 3)
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g).to(y_dtype)
    want = ops.gemm_w(oracle, x, w, math, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    got = ops.gemm_w(hip, x.cuda(), w.to("cuda"), math, bias=bias.cuda(), y=y0.clone().cuda(), alpha=1.25, beta=-0.5)
    # The activations' quantised bytes are the oracle's bit for bit (tests/test_gpu_quant.py), the products are exact; the
    # device sums them in f32 where the oracle sums in double: near 1e-6 (bf16 outputs: one rounding of the result).
    err = rel_l2(got, want)
    assert err <= (4e-3 if y_dtype == torch.bfloat16 else 1e-4), err


@pytest.mark.parametrize("math", [MATH_FP8, MATH_FP4])
def test_nvfp4_maths_rows_do_not_depend_on_the_batch(hip, math):
    N, K = 2048, 4096
    g = torch.Generator().manual_seed(2)
    x = torch.randn(64, K, generator=g).to(torch.bfloat16).cuda()
    w = random_weight(FORMATS["nvfp4"], N, K, 5).to("cuda")
    full = ops.gemm_w(hip, x, w, math)
    for M in (1, 7, 16, 33):
        part = ops.gemm_w(hip, x[:M].contiguous(), w, math)
        assert torch.equal(part, full[:M]), M


def test_c3_shape_under_the_fp4_math(hip, oracle):
    # W 4096 x 14336 NVFP4 (the NVFP4 GEMV configuration's weight), 8 rows, under the FP4 math against the oracle.
    N, K, M = 4096, 14336, 8
    g = torch.Generator().manual_seed(2008)
    master = master_weight(N, K, g)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = quantize_with(hip, master.cuda(), FORMATS["nvfp4"])
    got = ops.gemm_w(hip, x.cuda(), w, MATH_FP4)
    want = ops.gemm_w(oracle, x, w.to("cpu"), MATH_FP4)
    err = rel_l2(got, want)
    assert err <= 1e-2 and err <= 1e-4, err


# ---- the slab kernel (a workgroup per K slice of many tiles, partial tiles added by a second kernel) ----------------


@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("M,N,K", [(64, 6144, 4096), (32, 4096, 8192), (40, 2048, 8192), (57, 6000, 2048)])
def test_slab_shapes_give_the_bits_of_every_other_kernel(hip, fmt, M, N, K):
    # Shapes the slab kernel takes by itself: their rows equal the same rows computed sixteen at a time (the lean tile
    # kernel) bit for bit, with bias, alpha and a bf16 output in the epilogue of the second pass.
    g = torch.Generator().manual_seed(M + N)
    w = random_weight(FORMATS[fmt], N, K, N + K).to("cuda")
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    bias = torch.randn(N, generator=g).cuda()
    for y_dtype in (torch.float32, torch.bfloat16):
        big = ops.gemm_w(hip, x, w, MATH_BF16, bias=bias, alpha=0.5, y_dtype=y_dtype)
        for m0 in (0, 16, M - 16):
            part = ops.gemm_w(hip, x[m0:m0 + 16].contiguous(), w, MATH_BF16, bias=bias, alpha=0.5, y_dtype=y_dtype)
            assert torch.equal(big[m0:m0 + 16].view(torch.int16 if y_dtype == torch.bfloat16 else torch.int32),
                               part.view(torch.int16 if y_dtype == torch.bfloat16 else torch.int32)), (y_dtype, m0)
    want = ops.gemv_reference(x.cpu(), w.to("cpu").dense(), bias.cpu(), 0.5, 0.0, None)
    checks.check_product(ops.gemm_w(hip, x, w, MATH_BF16, bias=bias, alpha=0.5).cpu(), want)


@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("M,N,K", [(17, 1027, 2048), (64, 300, 4096), (33, 4096, 1040), (48, 14336, 4096)])
def test_slab_forced_equals_the_windowed_kernel(hip, fmt, M, N, K):
    # The variant table sends any row count to the slab kernel where it fits (ragged N and K included), or keeps it
    # away: same bits, for f32 and bf16 activations and beta != 0.
    g = torch.Generator().manual_seed(N)
    w = random_weight(FORMATS[fmt], N, K - K % 16, N).to("cuda")
    K = K - K % 16
    for x_dtype in (torch.bfloat16, torch.float32):
        x = torch.randn(M, K, generator=g).to(x_dtype).cuda()
        y0 = torch.randn(M, N, generator=g).cuda()
        key = f"gemm_w_{fmt}".encode()
        try:
            assert hip.lib.lx_tune_force(key, M, N, K, 4) == 0  # "window": never the slab kernel
            a = ops.gemm_w(hip, x, w, MATH_BF16, y=y0.clone(), alpha=1.25, beta=-0.5)
            assert hip.lib.lx_tune_force(key, M, N, K, 5) == 0  # "slab": wherever it fits
            b = ops.gemm_w(hip, x, w, MATH_BF16, y=y0.clone(), alpha=1.25, beta=-0.5)
        finally:
            hip.lib.lx_tune_clear()
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), x_dtype


def test_streams_with_and_without_the_partial_sum_buffer(hip):
    """The slab kernel's partial tiles belong to the stream (lx_rt_stream_create makes them, a host with its own streams
    calls lx_rt_stream_reserve): a product allocates nothing, and a stream without the buffer takes another kernel with
    the same bits, eagerly and under graph capture alike."""
    import ctypes

    M, N, K = 64, 4096, 8192  # a shape the rule sends to the slab kernel
    g = torch.Generator().manual_seed(31)
    w = random_weight(FORMATS["fp8"], N, K, 7).to("cuda")
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    lib = hip.lib
    plain, owned = torch.cuda.Stream(), torch.cuda.Stream()
    assert lib.lx_rt_stream_reserve(ctypes.c_void_p(owned.cuda_stream)) == 0
    assert lib.lx_rt_stream_reserve(ctypes.c_void_p(owned.cuda_stream)) == 0  # once is enough, twice is no error
    made = ctypes.c_void_p()
    assert lib.lx_rt_stream_create(ctypes.byref(made)) == 0
    try:
        y = torch.full((M, N), float("nan"), device="cuda")
        wl = w.lx()
        # Once before the memory is looked at: torch's allocator takes its blocks for the outputs and the runtime sets up
        # each stream's queue on its first launch.
        for s in (plain, owned):
            with torch.cuda.stream(s):
                ops.gemm_w(hip, x, w, MATH_BF16)
        assert lib.lx_gemm_w(x.data_ptr(), 1, K, ctypes.byref(wl), MATH_BF16, None, 0, y.data_ptr(), 0, N, M, N, K, 1.0, 0.0, None, made) == 0
        torch.cuda.synchronize()
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        outs = []
        for s in (plain, owned):
            with torch.cuda.stream(s):
                outs.append(ops.gemm_w(hip, x, w, MATH_BF16))
        assert lib.lx_gemm_w(x.data_ptr(), 1, K, ctypes.byref(wl), MATH_BF16, None, 0, y.data_ptr(), 0, N, M, N, K, 1.0, 0.0, None, made) == 0
        assert lib.lx_rt_stream_sync(made) == 0
        assert torch.equal(outs[0].view(torch.int32), outs[1].view(torch.int32)) and torch.equal(y.view(torch.int32), outs[0].view(torch.int32))
        assert torch.cuda.mem_get_info()[0] == free0, "a product allocated device memory"
        # under capture on the stream that owns a buffer: the same result on every replay
        graph = ctypes.c_void_p()
        y2 = torch.zeros(M, N, device="cuda")
        assert lib.lx_rt_capture_begin(made) == 0
        assert lib.lx_gemm_w(x.data_ptr(), 1, K, ctypes.byref(wl), MATH_BF16, None, 0, y2.data_ptr(), 0, N, M, N, K, 1.0, 0.0, None, made) == 0
        assert lib.lx_rt_capture_end(made, ctypes.byref(graph)) == 0
        for _ in range(3):
            y2.zero_()
            torch.cuda.synchronize()
            assert lib.lx_rt_graph_launch(graph, made) == 0 and lib.lx_rt_stream_sync(made) == 0
            assert torch.equal(y2.view(torch.int32), outs[0].view(torch.int32))
        assert lib.lx_rt_graph_destroy(graph) == 0
    finally:
        torch.cuda.synchronize()
        assert lib.lx_rt_stream_release(ctypes.c_void_p(owned.cuda_stream)) == 0
        assert lib.lx_rt_stream_release(ctypes.c_void_p(owned.cuda_stream)) == 0  # nothing left: no error
        assert lib.lx_rt_stream_destroy(made) == 0


@pytest.mark.parametrize("math,fmt", [(MATH_INT8, "int8"), (MATH_FP8, "fp8")])
def test_slab_under_the_byte_maths(hip, oracle, math, fmt):
    M, N, K = 64, 6144, 4096
    g = torch.Generator().manual_seed(9)
    w = random_weight(FORMATS[fmt], N, K, 5)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    got = ops.gemm_w(hip, x.cuda(), w.to("cuda"), math)
    part = ops.gemm_w(hip, x[:16].contiguous().cuda(), w.to("cuda"), math)
    assert torch.equal(got[:16].view(torch.int32), part.view(torch.int32))
    want = ops.gemm_w(oracle, x, w, math)
    if math == MATH_INT8:
        assert torch.equal(got.cpu().view(torch.int32), want.view(torch.int32))  # exact integer sums
    else:
        assert rel_l2(got, want) <= 1e-4  # f32 sums of exact products against the double sums of the reference
