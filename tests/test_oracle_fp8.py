"""Pins the oracle's 8-bit float formats and its GEMM on them (CPU only).

The reference holds no golden vectors for fp8 (it only times cuBLASLt on __nv_fp8_e4m3 / __nv_fp8_e5m2,
nvidia/bench/bench_cublaslt_e4m3.cu:6-21, bench_cublaslt_e5m2.cu:6-21), so the formats are pinned against an
independent implementation (torch.float8_e4m3fn / torch.float8_e5m2, all 256 codes each), against the extreme
values the OCP specification tabulates, and the product against exact integer arithmetic.
"""
import numpy as np
import pytest
import torch

import oracle_lib as O

FORMATS = [(0, torch.float8_e4m3fn, "e4m3"), (1, torch.float8_e5m2, "e5m2")]


def decode_all(e5m2):
    return np.array([O.lib.oracle_fp8_to_f32(e5m2, c) for c in range(256)], dtype=np.float32)


def encode(e5m2, values):
    return np.array([O.lib.oracle_f32_to_fp8(e5m2, float(v)) for v in values], dtype=np.uint8)


@pytest.mark.parametrize("e5m2,tdtype,name", FORMATS)
def test_decode_matches_torch_for_every_code(e5m2, tdtype, name):
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    want = codes.view(tdtype).to(torch.float32).numpy()
    got = decode_all(e5m2)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))  # also the sign of zero


def test_extreme_values_of_the_specification():
    """OCP 8-bit Floating Point Specification v1.0, table 1."""
    e4, e5 = decode_all(0), decode_all(1)
    assert e4[0x7E] == 448.0 and e4[0x08] == 2.0 ** -6 and e4[0x07] == 0.875 * 2.0 ** -6 and e4[0x01] == 2.0 ** -9
    assert np.isnan(e4[0x7F]) and np.isnan(e4[0xFF]) and not np.isinf(e4).any()
    assert e4[0x78] == 256.0  # exponent 15 is an ordinary exponent in e4m3
    assert e5[0x7B] == 57344.0 and e5[0x04] == 2.0 ** -14 and e5[0x03] == 0.75 * 2.0 ** -14 and e5[0x01] == 2.0 ** -16
    assert np.isinf(e5[0x7C]) and e5[0xFC] == -np.inf and np.isnan(e5[[0x7D, 0x7E, 0x7F]]).all()
    assert e4[0x38] == 1.0 and e5[0x3C] == 1.0 and e4[0xB8] == -1.0
    # e5m2 is the upper byte of an IEEE half
    half = (np.arange(256, dtype=np.uint16) << 8).view(np.float16).astype(np.float32)
    ok = ~np.isnan(half)
    assert np.array_equal(e5[ok], half[ok])


@pytest.mark.parametrize("e5m2,tdtype,name", FORMATS)
def test_encode_inverts_decode_and_matches_torch(e5m2, tdtype, name):
    table = decode_all(e5m2)
    finite = np.isfinite(table)
    codes = np.arange(256, dtype=np.uint8)[finite]
    assert np.array_equal(encode(e5m2, table[finite]), codes)
    # random values inside the finite range: torch rounds to nearest even too
    rng = np.random.default_rng(5)
    top = 448.0 if not e5m2 else 57344.0
    x = np.concatenate([rng.normal(0, 1, 4000), rng.uniform(-top, top, 2000), rng.normal(0, 2.0 ** -8, 2000),
                        rng.normal(0, 2.0 ** -15, 1000)]).astype(np.float32)
    want = torch.from_numpy(x).to(tdtype).view(torch.uint8).numpy()
    got = encode(e5m2, x)
    assert np.array_equal(got, want)


def test_encode_ties_to_even_and_saturates():
    # e4m3 around 1.0 the spacing is 1/8: 1.0625 is halfway between 1.0 (0x38, even) and 1.125 (0x39)
    assert list(encode(0, [1.0625, 1.1875, 1.06251, -1.0625])) == [0x38, 0x3A, 0x39, 0xB8]
    # halfway between the largest subnormal (7 * 2^-9) and the smallest normal (2^-6): even is the normal
    assert list(encode(0, [7.5 * 2.0 ** -9, 0.5 * 2.0 ** -9, 0.50001 * 2.0 ** -9])) == [0x08, 0x00, 0x01]
    # beyond the largest finite value, infinities included: that value; NaN: all ones
    assert list(encode(0, [448.0, 464.0, 1e9, -np.inf])) == [0x7E, 0x7E, 0x7E, 0xFE]
    assert list(encode(1, [57344.0, 61440.0, 1e9, np.inf, -1e9])) == [0x7B, 0x7B, 0x7B, 0x7B, 0xFB]
    assert encode(0, [np.nan])[0] & 0x7F == 0x7F and encode(1, [np.nan])[0] & 0x7F == 0x7F
    # e5m2 around 1.0 the spacing is 1/4
    assert list(encode(1, [1.125, 1.375, 1.126])) == [0x3C, 0x3E, 0x3D]


@pytest.mark.parametrize("types,e5m2", [(O.E4M3E4M3F16, 0), (O.E5M2E5M2F16, 1)])
def test_gemm_on_small_codes_is_exact_integer_arithmetic(types, e5m2):
    """Values in {-2,...,2}: every product and partial sum is an exact integer, so numpy's product in another
    order and in float64 must agree bit for bit with the sequential fp32 sum; alpha = 2, beta = -1 on top."""
    m, n, k = 23, 31, 257
    rng = np.random.default_rng(11)
    av = rng.integers(-2, 3, (m, k)).astype(np.float32); bv = rng.integers(-2, 3, (n, k)).astype(np.float32)
    cv = rng.integers(-8, 9, (m, n)).astype(np.float32)
    a, b = encode(e5m2, av.ravel()), encode(e5m2, bv.ravel())
    assert np.array_equal(decode_all(e5m2)[a], av.ravel())
    c = cv.astype(np.float16).view(np.uint16).ravel()
    want = 2 * (av.astype(np.float64) @ bv.astype(np.float64).T) - cv
    assert np.abs(want).max() < 2048  # integers a half holds exactly
    got = O.out_to_f64(types, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 2, -1))
    assert np.array_equal(got, want)
    # row-major B: the same numbers through the other indexing
    b_rows = encode(e5m2, bv.T.ravel())
    got = O.out_to_f64(types, O.gemm(types, a, b_rows, c, m, n, k, O.ROW, O.ROW, 2, -1))
    assert np.array_equal(got, want)
    # column-major A
    a_cols = encode(e5m2, av.T.ravel())
    got = O.out_to_f64(types, O.gemm(types, a_cols, b, c, m, n, k, O.COL, O.COL, 2, -1))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("types,e5m2,tdtype", [(O.E4M3E4M3F16, 0, torch.float8_e4m3fn), (O.E5M2E5M2F16, 1, torch.float8_e5m2)])
def test_gemm_against_torch_decoded_fp64_truth(types, e5m2, tdtype):
    """Random codes: the inputs decoded by torch, multiplied in float64, bound the oracle's fp32 sum and its fp16
    epilogue; the naive and the blocked loop of the oracle agree bit for bit (same summation order)."""
    m, n, k = 32, 48, 1024
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=21)
    A = torch.from_numpy(a).view(tdtype).to(torch.float64).numpy().reshape(m, k)
    B = torch.from_numpy(b).view(tdtype).to(torch.float64).numpy().reshape(n, k)
    Cf = O.out_to_f64(types, c).reshape(m, n)
    truth = A @ B.T + Cf
    d = O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)
    got = O.out_to_f64(types, d)
    rms = np.sqrt((truth ** 2).mean())
    assert (np.abs(got - truth) <= 2e-3 * np.maximum(np.abs(truth), rms)).all()  # three fp16 roundings and the sum
    t64, _ = O.gemm_f64(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)
    assert np.allclose(t64, truth, rtol=1e-12, atol=1e-12)
    assert np.array_equal(d, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, naive=True))


def test_fill_fp8_is_the_rounded_float_fill():
    for dt, e5m2 in ((O.DT_E4M3, 0), (O.DT_E5M2, 1)):
        f = O.fill(5000, O.DT_F32, O.FILL_NORMAL, 1.0, 77)
        q = O.fill(5000, dt, O.FILL_NORMAL, 1.0, 77)
        assert np.array_equal(q, encode(e5m2, f))
        # large scale: saturates, never produces an infinity or a NaN code
        q = O.fill(5000, dt, O.FILL_NORMAL, 1e6, 78)
        assert np.isfinite(decode_all(e5m2)[q]).all()
