"""Pins the oracle's number formats against closed forms and torch's own float8 / bfloat16 types.

A mistake such as a wrong exponent bias, a dropped subnormal, a tie rounded away from even or a sign on zero
fails one of these.
"""

import ctypes

import numpy as np
import torch

from dromos_amd.formats import e2m1_codes, e2m1_table, e4m3_table


def _fns(oracle):
    lib = oracle.lib
    lib.orc_e4m3_to_f32.restype = ctypes.c_float
    lib.orc_e4m3_to_f32.argtypes = [ctypes.c_uint8]
    lib.orc_f32_to_e4m3.restype = ctypes.c_uint8
    lib.orc_f32_to_e4m3.argtypes = [ctypes.c_float]
    lib.orc_e2m1_to_f32.restype = ctypes.c_float
    lib.orc_e2m1_to_f32.argtypes = [ctypes.c_uint32]
    lib.orc_f32_to_e2m1.restype = ctypes.c_uint32
    lib.orc_f32_to_e2m1.argtypes = [ctypes.c_float]
    return lib


def test_e4m3_decode_all_codes(oracle):
    lib = _fns(oracle)
    table = e4m3_table()
    torch_vals = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).double()
    for b in range(256):
        got = lib.orc_e4m3_to_f32(b)
        if (b & 0x7F) == 0x7F:
            assert abs(got) == 480.0  # the reference's table reads the two NaN codes by the same formula
            continue
        assert got == table[b].item() == torch_vals[b].item(), b
    assert lib.orc_e4m3_to_f32(0x7E) == 448.0 and lib.orc_e4m3_to_f32(0x01) == 2.0**-9 and lib.orc_e4m3_to_f32(0x08) == 2.0**-6


def test_e4m3_encode_every_bf16_input(oracle):
    # All 65536 bf16 bit patterns (a superset of what a quantiser feeds it after the clamp), against torch's cast.
    lib = _fns(oracle)
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    want = bits.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    vals = bits.numpy()
    for i in range(65536):
        v = float(vals[i])
        got = lib.orc_f32_to_e4m3(v)
        if np.isnan(v):
            assert got & 0x7F == 0x7F
        else:
            assert got == int(want[i]), (i, v, got, int(want[i]))


def test_e4m3_encode_ties_and_saturation(oracle):
    lib = _fns(oracle)
    assert lib.orc_f32_to_e4m3(1.0625) == 0x38  # halfway 1.0 / 1.125 -> even mantissa (1.0)
    assert lib.orc_f32_to_e4m3(1.1875) == 0x3A  # halfway 1.125 / 1.25 -> even mantissa (1.25)
    assert lib.orc_f32_to_e4m3(2.0**-10) == 0x00  # halfway 0 / 2^-9 -> 0
    assert lib.orc_f32_to_e4m3(3 * 2.0**-10) == 0x02  # halfway 1 / 2 steps -> 2
    assert lib.orc_f32_to_e4m3(464.0) == 0x7E and lib.orc_f32_to_e4m3(1e9) == 0x7E and lib.orc_f32_to_e4m3(-1e9) == 0xFE
    assert lib.orc_f32_to_e4m3(-0.0) == 0x80
    # random f32 values against torch
    g = torch.Generator().manual_seed(1)
    x = torch.randn(20000, generator=g) * torch.rand(20000, generator=g) * 100
    want = x.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    for i in range(x.numel()):
        assert lib.orc_f32_to_e4m3(float(x[i])) == int(want[i])


def test_e2m1_tables_and_encode(oracle):
    lib = _fns(oracle)
    table = e2m1_table()
    for c in range(16):
        assert lib.orc_e2m1_to_f32(c) == table[c].item()
    mids = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    tie_code = [0, 2, 2, 4, 4, 6, 6]
    for m, c in zip(mids, tie_code):
        assert lib.orc_f32_to_e2m1(m) == c and lib.orc_f32_to_e2m1(-m) == (c | 8 if c else 0), m
        assert lib.orc_f32_to_e2m1(np.nextafter(np.float32(m), np.float32(10))) == mids.index(m) + 1
        assert lib.orc_f32_to_e2m1(np.nextafter(np.float32(m), np.float32(0))) == mids.index(m)
    assert lib.orc_f32_to_e2m1(100.0) == 7 and lib.orc_f32_to_e2m1(-100.0) == 15 and lib.orc_f32_to_e2m1(-0.1) == 0
    # brute force: nearest grid value (ties to even code) for a sweep of inputs, and the torch restatement
    xs = torch.linspace(-7, 7, 5601)
    ref = e2m1_codes(xs)
    grid = table[:8]
    for i, x in enumerate(xs.tolist()):
        got = lib.orc_f32_to_e2m1(x)
        assert got == int(ref[i]), x
        mag = min(abs(x), 6.0)
        assert abs(grid[got & 7].item() - mag) == (grid - mag).abs().min().item()


def test_bf16_rounding_through_dequantize(oracle):
    # The oracle's f32 -> bf16 rounding (nearest even) as seen through lx_dequantize_weight of an INT8 weight:
    # q * scale rounded once, against torch's own cast.
    import ops
    from dromos_amd.abi import W_INT8
    from dromos_amd.formats import Weight

    g = torch.Generator().manual_seed(3)
    q = torch.randint(-127, 128, (64, 256), generator=g, dtype=torch.int32).to(torch.int8)
    scale = torch.rand(64, generator=g) * 0.1 + 1e-3
    w = Weight(W_INT8, q, scale)
    got = ops.dequantize(oracle, w, 64, 256)
    want = (q.float() * scale[:, None]).to(torch.bfloat16)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
