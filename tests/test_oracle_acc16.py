"""Pins the oracle's model of the reference kernels' 16-bit accumulators (CPU only).

The reference holds no output of intel::gemm_bf16_bf16_bf16_m8k16 (bf16 C operand of every DPAS,
intel/kernels/xe_gemm_bf16_bf16_bf16_m8k16.hpp:88-107) or of sm80::fp16_mma_gemm (fp16 C operand of every
mma.sync.m16n8k8, nvidia/kernels/sm_80/fp16_mma_gemm.cuh:179,279-290), and what either device does inside one
instruction is not published, so agreement with those devices stays unpinned.  What is pinned here is the arithmetic
of the model: chunks of 16 / 8 consecutive k summed in fp32, a running sum rounded to 16 bits after every chunk,
the bf16 epilogue rounded after every operation and the fp16 epilogue's single-rounding fused multiply-add.
"""
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle_lib as O

BF, FH = O.BF16BF16BF16_ACC16, O.F16F16F16_ACC16


def enc(types, x):
    """float array -> the type's 16-bit patterns (values must be representable)."""
    x = np.asarray(x, dtype=np.float32)
    if types == BF:
        bits = (x.view(np.uint32) >> 16).astype(np.uint16)
        assert np.array_equal(O.bf16_to_f32(bits), x)
        return bits
    h = x.astype(np.float16)
    assert np.array_equal(h.astype(np.float32), x)
    return h.view(np.uint16)


def dec(types, bits):
    return O.out_to_f64(types, bits)


def round16(types, x32):
    """fp32 -> the output type and back, through numpy / torch (independent of the oracle's converters)."""
    x32 = np.asarray(x32, dtype=np.float32)
    if types == BF:
        return torch.from_numpy(x32.copy()).to(torch.bfloat16).to(torch.float32).numpy()
    return x32.astype(np.float16).astype(np.float32)


@pytest.mark.parametrize("types,limit,other", [(BF, 4096, 2048), (FH, 16384, 32768)])
def test_ones_stop_growing_where_a_chunk_is_half_a_spacing(types, limit, other):
    """K ones: the running sum is exact until a chunk (16 for bf16, 8 for fp16) is half the spacing of the
    16-bit format; there sum + chunk is a tie, the even neighbour is the sum itself, and it stays.  bf16 has 8
    significant bits: spacing 32 from 4096 on.  fp16 has 11: spacing 16 from 16384 on.  An fp32 accumulator would
    give K, a chunk of the other length would stop at `other`."""
    for k in (limit // 2, limit, limit + 8 * 40, 2 * limit + 24):
        a = enc(types, np.ones(k)); b = enc(types, np.ones(k))
        d = O.gemm(types, a, b, None, 1, 1, k, O.ROW, O.COL, 1, 0)
        assert dec(types, d)[0, 0] == min(k, limit), k
        assert np.array_equal(d, O.gemm(types, a, b, None, 1, 1, k, O.ROW, O.COL, 1, 0, naive=True))
    assert limit != other


def test_last_chunk_may_be_shorter():
    # bf16, K = 4096 + 16 + 5: the short chunk adds 5 to 4096 -> 4101 rounds to 4096 (spacing 32); with K = 37 the
    # chunks are 16, 16, 5 and everything is exact
    for k, want in ((4096 + 16 + 5, 4096.0), (37, 37.0)):
        a = enc(BF, np.ones(k))
        assert dec(BF, O.gemm(BF, a, a, None, 1, 1, k, O.ROW, O.COL, 1, 0))[0, 0] == want
    # fp16, threes times ones, K = 8 * 700 + 3: every chunk adds 24 (the last one 9) and the running sum passes
    # through the ranges of spacing 8 and 16, where 24 is no longer a whole number of spacings
    k = 8 * 700 + 3
    a = enc(FH, np.full(k, 3.0)); b = enc(FH, np.ones(k))
    acc = np.float32(0)
    for c in range(0, k, 8):
        acc = round16(FH, np.float32(acc + np.float32(3.0 * min(8, k - c))))
    assert dec(FH, O.gemm(FH, a, b, None, 1, 1, k, O.ROW, O.COL, 1, 0))[0, 0] == float(acc)


def model(types, A, B, C, alpha, beta):
    """The same arithmetic spelled with numpy scalars: float32 adds in k order inside a chunk, numpy float16 /
    torch bfloat16 for every 16-bit rounding, exact rationals for the fp16 fused multiply-add."""
    chunk = O.ACC16_CHUNK[types]
    m, k = A.shape
    n = B.shape[1]
    out = np.zeros((m, n), dtype=np.float64)
    alpha = float(round16(types, np.float32(alpha))); beta = float(round16(types, np.float32(beta)))
    for i in range(m):
        for j in range(n):
            acc = np.float32(0)
            for c0 in range(0, k, chunk):
                part = np.float32(0)
                for p in range(c0, min(c0 + chunk, k)):
                    part = np.float32(part + np.float32(A[i, p] * B[p, j]))   # the product is exact in fp32
                acc = round16(types, np.float32(acc + part))[()]
            if types == BF:
                v = round16(types, np.float32(acc * np.float32(alpha)))[()]
                if beta != 0:
                    bc = round16(types, np.float32(np.float32(beta) * np.float32(C[i, j])))[()]
                    v = round16(types, np.float32(v + bc))[()]
                out[i, j] = v
            else:
                bc = float(round16(types, np.float32(np.float32(beta) * np.float32(C[i, j])))[()]) if beta != 0 else 0.0
                out[i, j] = round_fraction_to_f16(Fraction(alpha) * Fraction(float(acc)) + Fraction(bc))
    return out


def round_fraction_to_f16(x: Fraction) -> float:
    """Exact rational -> nearest fp16 value, ties to the even mantissa, by comparing with the neighbours."""
    if x == 0:
        return 0.0
    grid = np.arange(0x0000, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)   # all finite magnitudes
    a = abs(x)
    hi = int(np.searchsorted(grid, float(a)))   # float(a) is correctly rounded: off by at most one slot
    best = None
    for idx in range(max(hi - 2, 0), min(hi + 2, len(grid) - 1) + 1):
        dist = abs(Fraction(float(grid[idx])) - a)
        key = (dist, idx & 1)   # ties: even code = even mantissa
        if best is None or key < best[0]:
            best = (key, idx)
    v = float(grid[best[1]])
    assert a < Fraction(65520), "overflow is not part of this helper"
    return v if x > 0 else -v


@pytest.mark.parametrize("types", [BF, FH])
@pytest.mark.parametrize("alpha,beta", [(1, 0), (1, 1), (0.75, -1.5)])
def test_against_the_numpy_model_on_random_inputs(types, alpha, beta):
    m, n, k = 5, 6, 75   # 75: four whole bf16 chunks and a short one, nine fp16 chunks and a short one
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=31)
    A = dec(types, a).reshape(m, k).astype(np.float32); Bm = dec(types, b).reshape(n, k).T.astype(np.float32)
    Cm = dec(types, c).reshape(m, n)
    want = model(types, A, Bm, Cm, alpha, beta)
    got = dec(types, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, alpha, beta))
    assert np.array_equal(got, want)
    assert np.array_equal(got, dec(types, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, alpha, beta, naive=True)))
    # the other layouts are the same numbers through other indexing
    a_cols = a.reshape(m, k).T.copy().ravel(); b_rows = b.reshape(n, k).T.copy().ravel()
    got = dec(types, O.gemm(types, a_cols, b_rows, c, m, n, k, O.COL, O.ROW, alpha, beta))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("types,fp32_acc", [(BF, O.BF16BF16BF16), (FH, O.F16F16F16)])
def test_the_running_sum_is_visibly_coarser_than_fp32_accumulation(types, fp32_acc):
    """On N(0,1) inputs with K = 4096 the 16-bit running sum must lose accuracy against the fp64 truth by well
    over the final rounding alone (a sign that it is really rounded after every chunk) and still track it."""
    m, n, k = 8, 64, 4096
    a, b, _ = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=5, with_c=False)
    truth, _ = O.gemm_f64(fp32_acc, a, b, None, m, n, k, O.ROW, O.COL, 1, 0)
    e16 = np.abs(dec(types, O.gemm(types, a, b, None, m, n, k, O.ROW, O.COL, 1, 0)) - truth)
    e32 = np.abs(dec(fp32_acc, O.gemm(fp32_acc, a, b, None, m, n, k, O.ROW, O.COL, 1, 0)) - truth)
    rms = np.sqrt((truth ** 2).mean())
    assert e16.mean() > 3 * e32.mean()
    assert e16.max() < 0.25 * rms


def test_f64_to_f16_on_every_value_midpoint_and_neighbour():
    codes = np.arange(0, 0x7C00, dtype=np.uint16)
    vals = codes.view(np.float16).astype(np.float64)
    f = O.lib.oracle_f64_to_f16
    assert all(f(float(v)) == int(c) for c, v in zip(codes, vals))
    assert f(-0.0) == 0x8000 and f(-1.0) == 0xBC00
    nxt = np.append(vals[1:], 65536.0)
    mids = (vals + nxt) / 2
    for c, mid in zip(codes, mids):
        c = int(c)
        even = c if c % 2 == 0 else c + 1   # 0x7BFF's upper neighbour is 0x7C00 = infinity
        assert f(float(mid)) == even, hex(c)
        assert f(float(np.nextafter(mid, 0.0))) == c and f(float(np.nextafter(mid, np.inf))) == c + 1
    assert f(float("inf")) == 0x7C00 and f(1e300) == 0x7C00 and f(-1e300) == 0xFC00 and f(float("nan")) & 0x7FFF > 0x7C00
    # numpy's own double -> half conversion rounds once as well
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.normal(0, 1, 3000), rng.normal(0, 1e-6, 2000), rng.uniform(-65000, 65000, 2000)])
    assert all(f(float(v)) == int(np.float16(v).view(np.uint16)) for v in x)


def test_fma_f16_rounds_once():
    fma = O.lib.oracle_fma_f16
    h = lambda bits: float(np.uint16(bits).view(np.float16))
    # 1.5 * (1 + 2^-10) = 1.5 + 2^-10 + 2^-11: halfway between 1537/1024 and 1538/1024 -> even = 1538/1024 = 0x3E02
    assert fma(1.5, 1 + 2.0 ** -10, 0.0) == 0x3E02
    # a tiny addend must break the tie; done as multiply, round (to fp16 or to fp32), add it would not
    assert fma(1.5, 1 + 2.0 ** -10, -2.0 ** -24) == 0x3E01
    assert fma(1.5, 1 + 2.0 ** -10, 2.0 ** -24) == 0x3E02
    assert fma(-1.5, 1 + 2.0 ** -10, 2.0 ** -24) == 0xBE01
    # signs of zero: (+0) + (-0) = +0, (-0) + (-0) = -0
    assert fma(1.0, 0.0, 0.0) == 0x0000 and fma(-1.0, 0.0, 0.0) == 0x0000 and fma(-1.0, 0.0, -0.0) == 0x8000
    # overflow to infinity, exact cancellation, subnormal results
    assert fma(256.0, 256.0, 0.0) == 0x7C00 and fma(3.0, 5.0, -15.0) == 0x0000
    assert fma(2.0 ** -12, 2.0 ** -12, 0.0) == 0x0001 and fma(2.0 ** -13, 2.0 ** -12, 0.0) == 0x0000   # 2^-25 is a tie -> 0
    rng = np.random.default_rng(9)
    bits = rng.integers(0, 0x7C00, (4000, 3)).astype(np.uint16) | (rng.integers(0, 2, (4000, 3)).astype(np.uint16) << 15)
    checked = 0
    for x, y, z in bits:
        exact = Fraction(h(x)) * Fraction(h(y)) + Fraction(h(z))
        if abs(exact) >= 65520:
            continue
        want = round_fraction_to_f16(exact)
        got = float(np.uint16(fma(h(x), h(y), h(z))).view(np.float16))
        assert got == want, (hex(x), hex(y), hex(z))
        checked += 1
    assert checked > 2000
