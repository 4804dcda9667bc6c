"""Pins the oracle's GEMV / GEMM: float64 x @ W^T on the decoded values (a dropped scale, a swapped nibble, a
transposed operand or a wrong epilogue order fails it), the contract's edge cases, and bit-for-bit agreement
of the f32 sums with the reference's CPU backend at its generic level."""

import pytest
import torch

import checks
import ops
from conftest import rel_l2
from dromos_amd.abi import FORMATS, MATH_BF16, MATH_INT8, W_BF16, W_INT8
from dromos_amd.formats import random_weight

FMT = checks.FMT_NAMES


@pytest.mark.parametrize("K", [48, 528, 2048])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (-1.5, 1.0)])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias_dtype", [None, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 8])
def test_gemv_dtype_matrix(oracle, M, x_dtype, fmt, bias_dtype, y_dtype, alpha, beta, K):
    checks.gemv_case(oracle, fmt, M, 37, K, seed=M * 101 + K, x_dtype=x_dtype, bias_dtype=bias_dtype, y_dtype=y_dtype,
                     alpha=alpha, beta=beta)


@pytest.mark.parametrize("pad", [0, 3, 8])
@pytest.mark.parametrize("fmt", FMT)
def test_gemv_strided(oracle, fmt, pad):
    checks.gemv_case(oracle, fmt, 5, 300, 1024, seed=pad + 9, bias_dtype=torch.bfloat16, alpha=2.0, beta=0.5, pad=pad)


@pytest.mark.parametrize("fmt", FMT)
def test_gemv_rows_do_not_depend_on_batch(oracle, fmt):
    checks.gemv_rows_do_not_depend_on_batch(oracle, fmt, 256, 2048, seed=5)


def test_gemv_nvfp4_global_is_linear(oracle):
    checks.gemv_nvfp4_global_is_linear(oracle)


def test_gemv_argument_errors(oracle):
    w = random_weight(W_BF16, 8, 64, 1)
    x = torch.zeros(9, 64)
    assert ops.gemv_w(oracle, x, w, status=True) == 1  # M > 8
    assert ops.gemv_w(oracle, x[:0], w, M=0, status=True) == 0
    assert ops.gemv_w(oracle, x[:2], w, ld_x=32, status=True) == 1  # ld_x < K
    w3 = random_weight(FORMATS["nvfp4"], 8, 64, 1)
    assert ops.gemv_w(oracle, torch.zeros(1, 40), w3, K=40, N=8, status=True) == 1  # K % 16 != 0


def test_gemv_wrapper_entry_points(oracle):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(4, 1024, generator=g)
    for fmt in (W_BF16, W_INT8):
        w = random_weight(fmt, 300, 1024, fmt + 1)
        a = torch.empty(4, 300)
        oracle("gemv", x, 0, 1024, w.data, fmt, w.scale, None, 0, a, 0, 300, 4, 300, 1024, 1.0, 0.0)
        assert torch.equal(a, ops.gemv_w(oracle, x, w))
    w = random_weight(W_BF16, 300, 1024, 1)
    a = torch.empty(4, 300)
    oracle("gemv_decode_bf16", x, 0, 1024, w.data, None, 0, a, 0, 300, 4, 300, 1024, 1.0, 0.0)
    assert torch.equal(a, ops.gemv_w(oracle, x, w))


@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("M", [1, 16, 64, 70])
def test_gemm_w_bf16_math(oracle, fmt, M):
    # Weight-only BF16 math: x is rounded to bf16 first, so the reference uses the rounded activations.
    N, K = 96, 512
    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, K, generator=g)
    w = random_weight(FORMATS[fmt], N, K, M + 3)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    y = ops.gemm_w(oracle, x, w, MATH_BF16, bias=bias, alpha=0.5)
    want = ops.gemv_reference(x.to(torch.bfloat16), w.dense(), bias, 0.5, 0.0, None)
    checks.check_product(y, want)
    assert ops.gemm_w(oracle, x, w, MATH_INT8, status=True) == (0 if fmt == "int8" else 801)  # int8 weights only
    assert ops.gemm_w(oracle, x, w, 2, status=True) == (0 if fmt in ("fp8", "nvfp4") else 801)  # fp8 or NVFP4 weights
    assert ops.gemm_w(oracle, x, w, 3, status=True) == (0 if fmt == "nvfp4" else 801)  # NVFP4 weights only
    ys = ops.gemm_skinny(oracle, x.to(torch.bfloat16), w, bias=bias, alpha=0.5)
    assert torch.equal(ys, y)


@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
def test_f32_sums_equal_the_reference_generic_level(oracle, ref, fmt, x_dtype):
    # The reference at level 1 sums four lanes with unfused steps, a fixed horizontal order and a fused tail;
    # the oracle restates exactly that, so the f32 outputs agree to the last bit (K = 1030 leaves a tail).
    real = ref.lib.lx_set_arch_override(0)
    try:
        assert ref.lib.lx_set_arch_override(1) == 1
        for M, N, K in [(1, 64, 1024), (8, 37, 1030 if fmt != "nvfp4" else 1040), (3, 300, 528)]:
            g = torch.Generator().manual_seed(K + M)
            x = torch.randn(M, K, generator=g).to(x_dtype)
            w = random_weight(FORMATS[fmt], N, K, K)
            bias = torch.randn(N, generator=g)
            y0 = torch.randn(M, N, generator=g)
            a = ops.gemv_w(oracle, x, w, bias, y0.clone(), alpha=1.25, beta=-0.5)
            b = ops.gemv_w(ref, x, w, bias, y0.clone(), alpha=1.25, beta=-0.5)
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (M, N, K)
    finally:
        ref.lib.lx_set_arch_override(0)
    assert real >= 1


@pytest.mark.parametrize("fmt", FMT)
def test_agrees_with_the_reference_best_level(oracle, ref, fmt):
    # Whatever vector width the reference picks on this CPU, the two agree far inside the path's tolerance.
    g = torch.Generator().manual_seed(7)
    x = torch.randn(4, 4096, generator=g).to(torch.bfloat16)
    w = random_weight(FORMATS[fmt], 512, 4096, 11)
    a, b = ops.gemv_w(oracle, x, w), ops.gemv_w(ref, x, w)
    assert rel_l2(a, b) < 1e-5
    x64 = torch.randn(40, 4096, generator=g).to(torch.bfloat16)
    a, b = ops.gemm_w(oracle, x64, w), ops.gemm_w(ref, x64, w)
    assert rel_l2(a, b) < 1e-5


def int8_math_reference(x, w, bias, alpha, beta, y0):
    """The INT8 math from closed forms: the activations by the per-token rule (quantize_act_reference), an exact
    integer product, and the epilogue's f32 operations in the reference's order (rowscale * xscale) * sum."""
    from dromos_amd.formats import quantize_act_reference

    q, xs, _ = quantize_act_reference(x, 1)
    sums = (q.view(torch.int8).double() @ w.data.cpu().double().T).float()  # exact below 2^53, then one rounding to f32
    t = (w.scale.cpu().float().unsqueeze(0) * xs.float().unsqueeze(1)) * sums
    if bias is not None:
        t = t + bias.float()
    v = alpha * t
    if beta != 0.0:
        v = beta * y0.float() + v
    return v


@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (12, 37, 1030), (40, 300, 528), (70, 96, 4096)])
def test_gemm_w_int8_math(oracle, M, N, K, x_dtype):
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).to(x_dtype)
    x[M // 2] = 0  # a zero row: scale 1, zero sums
    w = random_weight(FORMATS["int8"], N, K, M + 3)
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g)
    y = ops.gemm_w(oracle, x, w, MATH_INT8, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    want = int8_math_reference(x, w, bias, 1.25, -0.5, y0)
    assert torch.equal(y.view(torch.int32), want.view(torch.int32)), "the INT8 math is exact up to the epilogue's f32 operations"


@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (12, 37, 1030), (40, 300, 528)])
def test_int8_math_equals_the_reference_backend(oracle, ref, M, N, K):
    g = torch.Generator().manual_seed(K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = random_weight(FORMATS["int8"], N, K, K + 1)
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g)
    a = ops.gemm_w(oracle, x, w, MATH_INT8, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    b = ops.gemm_w(ref, x, w, MATH_INT8, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    assert torch.equal(a.view(torch.int32), b.view(torch.int32))


def fp8_math_reference(x, w, bias, alpha, beta, y0):
    """The FP8 math from closed forms: activations by the per-token e4m3 rule, exact products summed in float64 (exactly:
    the terms span fewer than 53 bits), t = float(rowscale * xscale * sum), then the f32 epilogue."""
    from dromos_amd.formats import e4m3_table, quantize_act_reference

    q, xs, _ = quantize_act_reference(x, 2)
    table = e4m3_table()
    sums = table[q.long()] @ table[w.data.cpu().long()].T
    t = (w.scale.cpu().double().unsqueeze(0) * xs.double().unsqueeze(1) * sums).float()
    if bias is not None:
        t = t + bias.float()
    v = alpha * t
    if beta != 0.0:
        v = beta * y0.float() + v
    return v


@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (12, 37, 1030), (40, 300, 528)])
def test_gemm_w_fp8_math(oracle, M, N, K, x_dtype):
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).to(x_dtype)
    x[M // 2] = 0
    w = random_weight(FORMATS["fp8"], N, K, M + 3)
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g)
    y = ops.gemm_w(oracle, x, w, 2, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    want = fp8_math_reference(x, w, bias, 1.25, -0.5, y0)
    assert torch.equal(y.view(torch.int32), want.view(torch.int32))


@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (12, 37, 1030), (40, 300, 528)])
def test_fp8_math_equals_the_reference_backend(oracle, ref, M, N, K):
    g = torch.Generator().manual_seed(K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = random_weight(FORMATS["fp8"], N, K, K + 1)
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g)
    a = ops.gemm_w(oracle, x, w, 2, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    b = ops.gemm_w(ref, x, w, 2, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    assert torch.equal(a.view(torch.int32), b.view(torch.int32))


def exact_math_reference(x, w, math, bias, alpha, beta, y0):
    """The FP8 math on NVFP4 weights and the FP4 math from closed forms: the activations' quantised values (the
    per-token rules of quantize_act_reference) times the exact weight elements, summed in float64 (exactly),
    t = float(global * xscale * sum), then the f32 epilogue."""
    from dromos_amd.formats import e2m1_table, e4m3_table, quantize_act_reference, unpack_codes

    q, xs, bs = quantize_act_reference(x, math)
    if math == 2:
        xv = e4m3_table()[q.long()]
    else:
        xv = e2m1_table()[unpack_codes(q).long()] * e4m3_table()[bs.long()].repeat_interleave(16, dim=-1)
    elems = w.dense() / w.glob if w.fmt == 3 else w.dense() / w.scale.cpu().double().unsqueeze(-1)
    rf = torch.full((elems.shape[0],), w.glob, dtype=torch.float64) if w.fmt == 3 else w.scale.cpu().double()
    sums = xv @ elems.T
    t = (rf.unsqueeze(0) * xs.double().unsqueeze(1) * sums).float()
    if bias is not None:
        t = t + bias.float()
    v = alpha * t
    if beta != 0.0:
        v = beta * y0.float() + v
    return v


@pytest.mark.parametrize("fmt,math", [("nvfp4", 2), ("nvfp4", 3), ("fp8", 2)])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (12, 37, 1040), (40, 300, 528)])
def test_gemm_w_exact_maths(oracle, fmt, math, M, N, K, x_dtype):
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).to(x_dtype)
    x[M // 2] = 0
    w = random_weight(FORMATS[fmt], N, K, M + 3, glob=0.25)  # a power of two: the element values come back exactly
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g)
    y = ops.gemm_w(oracle, x, w, math, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    want = exact_math_reference(x, w, math, bias, 1.25, -0.5, y0)
    assert torch.equal(y.view(torch.int32), want.view(torch.int32))


@pytest.mark.parametrize("fmt,math", [("nvfp4", 2), ("nvfp4", 3)])
@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (12, 37, 1040), (40, 300, 528)])
def test_exact_maths_equal_the_reference_backend(oracle, ref, fmt, math, M, N, K):
    g = torch.Generator().manual_seed(K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = random_weight(FORMATS[fmt], N, K, K + 1)
    bias = torch.randn(N, generator=g)
    y0 = torch.randn(M, N, generator=g)
    a = ops.gemm_w(oracle, x, w, math, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    b = ops.gemm_w(ref, x, w, math, bias=bias, y=y0.clone(), alpha=1.25, beta=-0.5)
    assert torch.equal(a.view(torch.int32), b.view(torch.int32))


def test_maths_and_formats_that_do_not_pair(oracle):
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    for fmt, math, want in [("int8", 2, 801), ("int8", 3, 801), ("fp8", 1, 801), ("fp8", 3, 801), ("bf16", 1, 801), ("nvfp4", 1, 801),
                            ("nvfp4", 2, 0), ("nvfp4", 3, 0), ("fp8", 2, 0), ("int8", 1, 0)]:
        assert ops.gemm_w(oracle, x, random_weight(FORMATS[fmt], 32, 64, 1), math, status=True) == want, (fmt, math)
