"""GPU parity: lx_gemv_w / lx_gemv / lx_gemv_decode_bf16 through the C ABI against float64 on the decoded
values and against the CPU oracle on the same seeded inputs (float outputs: relative L2 <= 1e-2 is the path's
bar; the observed error is around 1e-6), with the reference tests' edge cases (odd N, K around the vector cut,
strides that break alignment, beta = 0 never reading y) and the bitwise invariants (determinism, rows that do
not depend on the batch, NVFP4 global linearity)."""

import ctypes

import pytest
import torch

import checks
import ops
from conftest import rel_l2
from dromos_amd.abi import FORMATS, W_BF16, W_INT8, W_NVFP4
from dromos_amd.formats import Weight, master_weight, quantize_with, random_weight

pytestmark = pytest.mark.gpu
FMT = checks.FMT_NAMES
# From (1024, 2560) on: rows of exactly five and six load steps in one format or another (bf16 2560 / 3072, one-byte 5120 /
# 6144, NVFP4 10240 / 12288), which a single activation row asks for whole, and rows of 9 .. 14 steps (two even batches:
# one-byte 10240 / 11008 / 12288, bf16 5120 / 6144, NVFP4 18432).
SHAPES = [(10304, 2048), (2048, 4096), (3072, 2048), (1024, 512), (256, 2048), (256, 6400), (8, 2048),
          (1024, 2560), (1024, 3072), (1024, 5120), (1024, 6144), (1024, 10240), (1024, 12288), (1024, 18432), (1024, 11008)]


@pytest.mark.parametrize("K", [48, 528, 2048])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, 0.0), (-1.5, 1.0)])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias_dtype", [None, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 8])
def test_dtype_matrix(hip, M, x_dtype, fmt, bias_dtype, y_dtype, alpha, beta, K):
    checks.gemv_case(hip, fmt, M, 37, K, seed=M * 101 + K, x_dtype=x_dtype, bias_dtype=bias_dtype, y_dtype=y_dtype,
                     alpha=alpha, beta=beta)


@pytest.mark.parametrize("M", list(range(1, 9)))
@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
def test_every_m(hip, x_dtype, fmt, M):
    checks.gemv_case(hip, fmt, M, 300, 1024, seed=M, x_dtype=x_dtype, bias_dtype=torch.float32)


@pytest.mark.parametrize("pad", [0, 3, 8])
@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 5])
def test_strided(hip, M, x_dtype, fmt, pad):
    checks.gemv_case(hip, fmt, M, 300, 1024, seed=M * 7 + pad, x_dtype=x_dtype, bias_dtype=torch.bfloat16, alpha=2.0,
                     beta=0.5, pad=pad)


@pytest.mark.parametrize("K", [16, 32, 48, 64, 128, 256, 272, 512, 544, 1024, 1040, 2064])
@pytest.mark.parametrize("fmt", FMT)
def test_k_boundaries(hip, fmt, K):
    checks.gemv_case(hip, fmt, 3, 21, K, seed=K, x_dtype=torch.bfloat16)


@pytest.mark.parametrize("N,K", SHAPES)
@pytest.mark.parametrize("M", [1, 2, 4, 8])
@pytest.mark.parametrize("fmt", FMT)
def test_decode_shapes(hip, N, K, M, fmt):
    checks.gemv_case(hip, fmt, M, N, K, seed=N % 97 + M)


@pytest.mark.parametrize("M,N,K", [(1, 256, 2048), (8, 8, 2048), (8, 10304, 2048), (3, 128, 1280)])
@pytest.mark.parametrize("fmt", FMT)
def test_deterministic(hip, M, N, K, fmt):
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).cuda()
    w = random_weight(FORMATS[fmt], N, K, N).to("cuda")
    assert torch.equal(ops.gemv_w(hip, x, w), ops.gemv_w(hip, x, w))


@pytest.mark.parametrize("N,K", SHAPES)
@pytest.mark.parametrize("fmt", FMT)
def test_rows_do_not_depend_on_the_batch(hip, fmt, N, K):
    checks.gemv_rows_do_not_depend_on_batch(hip, fmt, N, K, seed=N + K)


def test_nvfp4_global_is_linear(hip):
    checks.gemv_nvfp4_global_is_linear(hip)


def test_wrappers_match_gemv_w(hip):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(4, 1024, generator=g).cuda()
    for fmt in (W_BF16, W_INT8):
        w = random_weight(fmt, 300, 1024, fmt + 1).to("cuda")
        a = torch.empty(4, 300, device="cuda")
        hip("gemv", x, 0, 1024, w.data, fmt, w.scale, None, 0, a, 0, 300, 4, 300, 1024, 1.0, 0.0)
        assert torch.equal(a, ops.gemv_w(hip, x, w))
    w = random_weight(W_BF16, 300, 1024, 1).to("cuda")
    a = torch.empty(4, 300, device="cuda")
    hip("gemv_decode_bf16", x, 0, 1024, w.data, None, 0, a, 0, 300, 4, 300, 1024, 1.0, 0.0)
    assert torch.equal(a, ops.gemv_w(hip, x, w))


def test_argument_errors(hip):
    w = random_weight(W_BF16, 8, 64, 1).to("cuda")
    x = torch.zeros(9, 64, device="cuda")
    assert ops.gemv_w(hip, x, w, status=True) == 1  # M > 8
    y = torch.full((1, 8), 7.0, device="cuda")
    assert ops.gemv_w(hip, x[:0], w, y=y, M=0, status=True) == 0
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())  # nothing touched
    assert ops.gemv_w(hip, x[:2], w, ld_x=32, status=True) == 1
    w4 = random_weight(W_NVFP4, 8, 64, 1).to("cuda")
    assert ops.gemv_w(hip, torch.zeros(1, 40, device="cuda"), w4, K=40, N=8, status=True) == 1
    from dromos_amd.formats import Weight

    wx = Weight(7, w.data)  # no such format
    assert ops.gemv_w(hip, x[:1], wx, status=True) == 1


@pytest.mark.parametrize("fmt", FMT)
@pytest.mark.parametrize("variant", [0, 1, 2])
def test_every_variant(hip, fmt, variant):
    # Any K split the tuner can force computes the same product.
    lib = hip.lib
    kernel = f"gemv_w_{fmt}".encode()
    assert lib.lx_tune_variants(kernel) == 3
    try:
        for M, N, K in [(1, 300, 1040), (3, 77, 2048), (8, 129, 1024), (2, 64, 528)]:
            lib.lx_tune_clear()
            assert lib.lx_tune_force(kernel, M, N, K, variant) == 0
            checks.gemv_case(hip, fmt, M, N, K - K % 16, seed=M * 13 + N, x_dtype=torch.bfloat16, bias_dtype=torch.float32)
    finally:
        lib.lx_tune_clear()


@pytest.mark.parametrize("fmt", FMT)
def test_order_class_admission(hip, fmt):
    # lx_tune_set admits exactly one split for a shape, the same one at every M.
    lib = hip.lib
    key = f"gemv_w_{fmt}".encode()
    lib.lx_tune_variant_name.restype = ctypes.c_char_p
    try:
        for N, K in SHAPES:
            admitted = {}
            for M in (1, 2, 4, 8):
                lib.lx_tune_clear()
                admitted[M] = [v for v in range(3) if lib.lx_tune_set(key, M, N, K, v) == 0]
                for v in range(3):
                    assert lib.lx_tune_set(key, M, N, K, v) in (0, 802)
            assert len(admitted[1]) == 1 and admitted[1] == admitted[2] == admitted[4] == admitted[8]
    finally:
        lib.lx_tune_clear()


@pytest.mark.parametrize("fmt,N,K,M", [("bf16", 4096, 4096, 1), ("int8", 14336, 4096, 1), ("int8", 14336, 4096, 4),
                                       ("fp8", 14336, 4096, 1), ("fp8", 14336, 4096, 4), ("nvfp4", 4096, 14336, 1),
                                       ("nvfp4", 4096, 14336, 8)])
def test_baseline_configs_against_the_oracle(hip, oracle, fmt, N, K, M):
    # The headline decode shapes at full size: N(0, 0.02) bf16 masters, quantised by the library, x ~ N(0, 1) bf16, f32 y.
    g = torch.Generator().manual_seed({"bf16": 0, "int8": 1000, "fp8": 1000, "nvfp4": 2000}[fmt] + (0 if fmt == "bf16" else M))
    master = master_weight(N, K, g)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = quantize_with(hip, master.cuda(), FORMATS[fmt])
    y = ops.gemv_w(hip, x.cuda(), w)
    w_cpu = w.to("cpu")
    want = ops.gemv_w(oracle, x, w_cpu)
    err = rel_l2(y.cpu(), want)
    assert err <= 1e-2, err
    assert err <= 1e-4, f"unexpectedly large for f32 accumulation: {err}"
    # a checksum of checksums against float64 on the decoded values
    ref64 = x.double() @ w_cpu.dense().T
    assert rel_l2(y.cpu(), ref64) <= 1e-4


def test_weights_beyond_four_gigabytes(hip):
    # 70000 x 65536 int8 = 4.59 GB: row offsets past 2^32 bytes. Drawn on the device; checked on rows spread over the
    # matrix (the last ones lie past the 4 GB mark) against float64 on the same device.
    N, K = 70000, 65536
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8, device="cuda")
    scale = torch.rand(N, generator=g, device="cuda") * 0.02 + 0.001
    w = Weight(FORMATS["int8"], q, scale)
    rows = torch.tensor([0, 1, 32767, 65535, 65536, 69998, 69999], device="cuda")
    for M, x_dtype in ((1, torch.bfloat16), (3, torch.float32)):
        x = torch.randn(M, K, generator=g, device="cuda").to(x_dtype)
        y = ops.gemv_w(hip, x, w)
        want = (x.double() @ q[rows].double().T) * scale[rows].double()
        err = (y[:, rows].double() - want).abs().max().item()
        assert err <= 2e-4 * want.abs().max().item(), (M, err)
    x16 = torch.randn(16, K, generator=g, device="cuda").to(torch.bfloat16)
    y16 = ops.gemm_w(hip, x16, w)
    want = (x16.double() @ q[rows].double().T) * scale[rows].double()
    assert (y16[:, rows].double() - want).abs().max().item() <= 2e-4 * want.abs().max().item()


@pytest.mark.parametrize("fmt,N,K", [("nvfp4", 512, 14336), ("nvfp4", 4096, 14336), ("bf16", 300, 4096), ("int8", 256, 8192)])
def test_rows_do_not_depend_on_the_batch_long_rows(hip, fmt, N, K):
    # Rows long enough that eight activation rows do not fit one LDS image: the image then holds half of K at a time
    # (or the weights are passed over twice), and a row's bits must still be those of the row alone.
    checks.gemv_rows_do_not_depend_on_batch(hip, fmt, N, K, seed=N + K)


@pytest.mark.parametrize("fmt,N,K", [("int8", 14335, 4096), ("fp8", 14336, 4096), ("bf16", 9001, 4096), ("nvfp4", 14336, 4096), ("int8", 12000, 1024)])
def test_more_rows_than_the_device_holds_at_once(hip, fmt, N, K):
    # With several bf16 activation rows and more weight rows than the device's wavefronts hold in one go, a wavefront
    # streams several row groups in turn (the workgroup's groups go round its wavefronts; the last workgroup's run past N).
    # A row's bits are those of the row alone, the values the reference's, the bias and factors the row's own.
    checks.gemv_rows_do_not_depend_on_batch(hip, fmt, N, K, seed=N + K)
    for M in (2, 4, 8):
        checks.gemv_case(hip, fmt, M, N, K, seed=M + N, x_dtype=torch.bfloat16, bias_dtype=torch.float32, alpha=0.5)
    checks.gemv_case(hip, fmt, 8, N, K, seed=N, x_dtype=torch.bfloat16, bias_dtype=torch.bfloat16, y_dtype=torch.bfloat16, alpha=-1.5, beta=1.0, pad=8)
