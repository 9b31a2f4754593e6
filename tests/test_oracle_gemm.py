"""Pins the oracle's GEMM functions (CPU only): closed forms, brute force, invariants."""
import itertools

import numpy as np
import pytest

import oracle_lib as O


def bf16(x):
    """float array -> bf16 bit patterns (values here are exactly representable)."""
    b = (np.asarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(O.bf16_to_f32(b), np.asarray(x, dtype=np.float32))
    return b


def f16(x):
    h = np.asarray(x, dtype=np.float32).astype(np.float16)
    assert np.array_equal(h.astype(np.float32), np.asarray(x, dtype=np.float32))
    return h.view(np.uint16)


def literal_s8(a, b, c, m, n, k, alpha, beta):
    d = np.zeros(m * n, dtype=np.int32)
    O.lib.oracle_literal_s8s32(a.ctypes.data, b.ctypes.data, c.ctypes.data, d.ctypes.data, m, n, k, alpha, beta)
    return d.reshape(m, n)


def literal_f32(a, b, c, m, n, k, alpha, beta):
    d = np.zeros(m * n, dtype=np.float32)
    O.lib.oracle_literal_f32(a.ctypes.data, b.ctypes.data, c.ctypes.data, d.ctypes.data, m, n, k, alpha, beta)
    return d.reshape(m, n)


# ------------------------------------------------------------ literal loop: closed forms
def test_literal_s8_all_ones_gives_k():
    m, n, k = 5, 7, 300
    a = np.ones(m * k, np.int8); b = np.ones(k * n, np.int8); c = np.zeros(m * n, np.int32)
    assert np.all(literal_s8(a, b, c, m, n, k, 1, 0) == k)
    c[:] = 10
    assert np.all(literal_s8(a, b, c, m, n, k, 3, -2) == 3 * k - 20)


def test_literal_s8_identity_and_extremes():
    n = 16
    eye = np.eye(n, dtype=np.int8).ravel()
    b = np.arange(n * n, dtype=np.int64).astype(np.int8)
    c = np.zeros(n * n, np.int32)
    assert np.array_equal(literal_s8(eye, b, c, n, n, n, 1, 0).ravel(), b.astype(np.int32))
    assert np.array_equal(literal_s8(b, eye, c, n, n, n, 1, 0).ravel(), b.astype(np.int32))
    k = 8192
    a = np.full(2 * k, -128, np.int8); bb = np.full(k * 3, -128, np.int8)
    assert np.all(literal_s8(a, bb, np.zeros(6, np.int32), 2, 3, k, 1, 0) == 128 * 128 * k)  # 2^27, no overflow
    bb[:] = 127
    assert np.all(literal_s8(a, bb, np.zeros(6, np.int32), 2, 3, k, 1, 0) == -128 * 127 * k)


def test_literal_s8_single_nonzero_probes_indexing():
    """One nonzero in A and one in B: D has exactly one nonzero, at (row of a, column of b), iff the k's agree."""
    m, n, k = 3, 4, 5
    for (i, p, q, j) in itertools.product(range(m), range(k), range(k), range(n)):
        a = np.zeros((m, k), np.int8); b = np.zeros((k, n), np.int8)
        a[i, p] = 3; b[q, j] = -7
        d = literal_s8(a.ravel(), b.ravel(), np.zeros(m * n, np.int32), m, n, k, 1, 0)
        want = np.zeros((m, n), np.int32)
        if p == q:
            want[i, j] = -21
        assert np.array_equal(d, want)


def test_literal_s8_brute_force_python_ints():
    rng = np.random.default_rng(0)
    m, n, k = 6, 5, 9
    a = rng.integers(-128, 128, (m, k)).astype(np.int8); b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    c = rng.integers(-1000, 1000, (m, n)).astype(np.int32)
    want = [[-3 * sum(int(a[i, p]) * int(b[p, j]) for p in range(k)) + 5 * int(c[i, j]) for j in range(n)] for i in range(m)]
    assert literal_s8(a.ravel(), b.ravel(), c.ravel(), m, n, k, -3, 5).tolist() == want


def test_literal_f32_sequential_order_is_observable():
    """1 + 2^-24 + 2^-24 in k order stays 1 (each add rounds to even); the reverse order would give 1+2^-23."""
    a = np.array([1.0, 1.0, 1.0], np.float32); b = np.array([1.0, 2.0 ** -24, 2.0 ** -24], np.float32)
    d = literal_f32(a, b, np.zeros(1, np.float32), 1, 1, 3, 1.0, 0.0)
    assert d[0, 0] == np.float32(1.0)
    b2 = b[::-1].copy()
    d2 = literal_f32(a, b2, np.zeros(1, np.float32), 1, 1, 3, 1.0, 0.0)
    assert d2[0, 0] == np.float32(1.0 + 2.0 ** -23)


# ------------------------------------------------------------ general oracle vs literal loop
@pytest.mark.parametrize("shape", [(1, 1, 1), (7, 5, 3), (33, 65, 129), (64, 64, 64)])
@pytest.mark.parametrize("ab", [(1, 0), (1, 1), (2, -1), (0, 1), (-3, 5)])
def test_oracle_s8_equals_literal(shape, ab):
    m, n, k = shape
    a, b, c = O.make_inputs(O.S8S8S32, m, n, k, seed=m * 7 + n)
    want = literal_s8(a, b, c, m, n, k, *ab)
    assert np.array_equal(O.gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.ROW, *ab), want)
    assert np.array_equal(O.gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.ROW, *ab, naive=True), want)
    assert np.array_equal(O.gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.ROW, *ab, threads=1), want)


@pytest.mark.parametrize("shape", [(1, 1, 1), (7, 5, 3), (33, 65, 129)])
@pytest.mark.parametrize("ab", [(1.0, 0.0), (1.0, 1.0), (2.0, -1.0), (0.5, 0.25)])
def test_oracle_bf16_f32_equals_literal_on_normal_data(shape, ab):
    """TOut = float: same sequential fp32 sum and the same rounding of alpha*acc + beta*c (no FMA)."""
    m, n, k = shape
    a, b, c = O.make_inputs(O.BF16BF16F32, m, n, k, seed=3)
    af, bf_ = O.bf16_to_f32(a), O.bf16_to_f32(b)
    want = literal_f32(af, bf_, c, m, n, k, *ab)
    for naive in (False, True):
        got = O.gemm(O.BF16BF16F32, a, b, c, m, n, k, O.ROW, O.ROW, *ab, naive=naive)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_oracle_layouts_are_transposes():
    rng = np.random.default_rng(1)
    m, n, k = 9, 11, 13
    A = rng.integers(-128, 128, (m, k)).astype(np.int8); B = rng.integers(-128, 128, (k, n)).astype(np.int8)
    C = rng.integers(-99, 99, (m, n)).astype(np.int32)
    want = (2 * (A.astype(np.int64) @ B.astype(np.int64)) + 3 * C).astype(np.int32)
    for la, lb in itertools.product((O.ROW, O.COL), repeat=2):
        a = (A if la == O.ROW else A.T).copy().ravel()
        b = (B if lb == O.ROW else B.T).copy().ravel()
        for naive in (False, True):
            assert np.array_equal(O.gemm(O.S8S8S32, a, b, C.ravel(), m, n, k, la, lb, 2, 3, naive=naive), want)
    # and for a float bundle with small integers (exact)
    Af = rng.integers(-3, 4, (m, k)).astype(np.float32); Bf = rng.integers(-3, 4, (k, n)).astype(np.float32)
    wantf = (Af @ Bf).astype(np.float32)
    for la, lb in itertools.product((O.ROW, O.COL), repeat=2):
        a = bf16((Af if la == O.ROW else Af.T).copy().ravel()); b = bf16((Bf if lb == O.ROW else Bf.T).copy().ravel())
        assert np.array_equal(O.gemm(O.BF16BF16F32, a, b, None, m, n, k, la, lb, 1, 0), wantf)


def test_oracle_int32_wraps():
    k = 4
    a = np.full(k, 127, np.int8); b = np.full(k, 127, np.int8); c = np.array([2 ** 31 - 1], np.int32)
    acc = 127 * 127 * k
    want = ((70000 * acc + 3 * (2 ** 31 - 1) + 2 ** 31) % 2 ** 32) - 2 ** 31
    assert O.gemm(O.S8S8S32, a, b, c, 1, 1, k, O.ROW, O.ROW, 70000, 3)[0, 0] == want
    assert literal_s8(a, b, c, 1, 1, k, 70000, 3)[0, 0] == want


def test_oracle_beta_zero_never_reads_c():
    m, n, k = 4, 4, 8
    a, b, _ = O.make_inputs(O.BF16BF16F32, m, n, k, with_c=False)
    nan_c = np.full(m * n, np.nan, np.float32)
    d0 = O.gemm(O.BF16BF16F32, a, b, None, m, n, k, O.ROW, O.COL, 1, 0)
    d1 = O.gemm(O.BF16BF16F32, a, b, nan_c, m, n, k, O.ROW, O.COL, 1, 0)
    assert np.array_equal(d0, d1) and np.isfinite(d0).all()
    assert np.isnan(O.gemm(O.BF16BF16F32, a, b, nan_c, m, n, k, O.ROW, O.COL, 1, 1)).all()


def test_oracle_16bit_epilogue_rounds_after_every_operation():
    """generic_gemm order: v = T(sum); v = T(v*alpha); v = T(v + T(beta*c)), checked on hand-built values."""
    # bf16 has 8 significant bits.  sum = 257 -> T(sum) = 256 (tie to even); * alpha 1.5 = 384 (exact)
    a = bf16([1.0] * 257); b = bf16([1.0] * 257)
    d = O.gemm(O.BF16BF16BF16, a, b, None, 1, 1, 257, O.ROW, O.COL, 1.5, 0.0)
    assert O.bf16_to_f32(d)[0, 0] == 384.0  # (257*1.5 = 385.5 would round to 386 if rounded once)
    # beta*c rounded before the add: beta = 1.0078125 (1+2^-7), c = 1.0078125 -> product 1.01568.. -> T = 1.015625
    c = bf16([1.0078125])
    d = O.gemm(O.BF16BF16BF16, bf16([0.0]), bf16([0.0]), c, 1, 1, 1, O.ROW, O.COL, 1.0, 1.0078125)
    assert O.bf16_to_f32(d)[0, 0] == 1.015625
    # fp16 (11 bits): sum = 2049 -> 2048; alpha = 1 ; + T(beta*c) with beta*c = 1 -> 2049 -> T = 2048
    a = f16([1.0] * 2049); b = f16([1.0] * 2049)
    d = O.gemm(O.F16F16F16, a, b, f16([1.0]), 1, 1, 2049, O.ROW, O.COL, 1.0, 1.0)
    assert O.f16_to_f32(d)[0, 0] == 2048.0
    # alpha itself is rounded to the output type first: 1.001 -> 1.0 in bf16
    d = O.gemm(O.BF16BF16BF16, bf16([3.0]), bf16([1.0]), None, 1, 1, 1, O.ROW, O.COL, 1.001, 0.0)
    assert O.bf16_to_f32(d)[0, 0] == 3.0


@pytest.mark.parametrize("types", [O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16])
def test_oracle_float_small_integers_exact_any_order(types):
    """Inputs in {-1,0,1}: every partial sum is an exact integer, so numpy's (different-order) product must match bit for bit."""
    m, n, k = 37, 53, 300
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=9)
    conv = O.f16_to_f32 if types == O.F16F16F16 else O.bf16_to_f32
    A = conv(a).reshape(m, k).astype(np.float64); B = conv(b).reshape(n, k).T.astype(np.float64)
    Cf = O.out_to_f64(types, c).reshape(m, n)
    want = 2 * (A @ B) - Cf
    got = O.out_to_f64(types, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 2, -1))
    assert np.abs(want).max() < 256 and np.array_equal(got, want)


@pytest.mark.parametrize("types,tol", [(O.BF16BF16F32, 1e-3), (O.BF16BF16BF16, 1e-2), (O.F16F16F16, 1e-2)])
def test_oracle_within_tolerance_of_fp64_truth(types, tol):
    m, n, k = 48, 64, 2048
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL if types != O.F16F16F16 else O.FILL_UNIFORM_PM1, seed=4)
    got = O.out_to_f64(types, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1))
    truth, absum = O.gemm_f64(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)
    rms = np.sqrt((truth ** 2).mean())
    assert (np.abs(got - truth) <= tol * np.maximum(np.abs(truth), rms)).all()
    if types == O.BF16BF16F32:  # fp32 sequential sum: |err| <= k * 2^-24 * sum|a||b| (classical bound)
        assert (np.abs(got - truth) <= k * 2.0 ** -24 * (absum + np.abs(O.out_to_f64(types, c).reshape(m, n))) + 1e-30).all()


def test_oracle_rows_band_and_empty():
    m, n, k = 20, 8, 16
    a, b, c = O.make_inputs(O.S8S8S32, m, n, k)
    full = O.gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)
    band = O.gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, rows=(5, 9))
    assert np.array_equal(band[5:9], full[5:9]) and not band[:5].any() and not band[9:].any()
    # K = 0: D = beta * C
    d = O.gemm(O.S8S8S32, a, b, c, m, n, 0, O.ROW, O.COL, 7, 2)
    assert np.array_equal(d.ravel(), 2 * c)
    assert O.gemm(O.S8S8S32, a, b, c, 0, n, k).shape == (0, n)


# ---------------------------------------------------------------------------------------------------------
# fp32 x fp32 -> fp32 (the type of the reference's ladder drivers)
# ---------------------------------------------------------------------------------------------------------
def _round_f32(x):
    """Exact rational -> nearest float32, ties to even (normal range only); the result as a Fraction."""
    from fractions import Fraction
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    x = abs(x)
    e = 0
    while x >= 2:
        x /= 2; e += 1
    while x < 1:
        x *= 2; e -= 1
    assert -126 <= e <= 127
    scaled = x * (1 << 23)                      # in [2^23, 2^24)
    q, r = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * r
    if twice > scaled.denominator or (twice == scaled.denominator and (q & 1)):
        q += 1
    return sign * Fraction(q, 1 << 23) * (Fraction(2) ** e)


def test_oracle_f32_is_a_fused_sum_in_k_order():
    """Each step is round(a*b + acc) with ONE rounding, in k order: exact rational arithmetic says so.  The same data
    summed as round(round(a*b) + acc), or in another order, gives different bits (checked, so the test can tell)."""
    from fractions import Fraction
    rng = np.random.default_rng(7)
    m, n, k = 3, 4, 37
    a = rng.standard_normal(m * k).astype(np.float32)
    b = rng.standard_normal(k * n).astype(np.float32)
    c = rng.standard_normal(m * n).astype(np.float32)
    got = O.gemm(O.F32F32F32, a, b, c, m, n, k, O.ROW, O.ROW, 1.0, 0.0)
    fused = np.zeros((m, n), np.float32); unfused = np.zeros((m, n), np.float32)
    for i in range(m):
        for j in range(n):
            acc = Fraction(0); acc2 = np.float32(0)
            for p in range(k):
                x, y = Fraction(float(a[i * k + p])), Fraction(float(b[p * n + j]))
                acc = _round_f32(x * y + acc)
                acc2 = np.float32(np.float32(a[i * k + p] * b[p * n + j]) + acc2)
            fused[i, j] = np.float32(float(acc)); unfused[i, j] = acc2
    assert np.array_equal(got, fused)
    assert not np.array_equal(fused, unfused)
    # the literal one-output-per-work-item loop and column-major operands give the same bits
    assert np.array_equal(O.gemm(O.F32F32F32, a, b, c, m, n, k, O.ROW, O.ROW, 1.0, 0.0, naive=True), fused)
    at = a.reshape(m, k).T.copy().ravel(); bt = b.reshape(k, n).T.copy().ravel()
    assert np.array_equal(O.gemm(O.F32F32F32, at, bt, c, m, n, k, O.COL, O.COL, 1.0, 0.0), fused)
    # epilogue: v = acc*alpha, then v + beta*c, each rounded once (as for bf16 -> f32)
    got = O.gemm(O.F32F32F32, a, b, c, m, n, k, O.ROW, O.ROW, 1.5, -0.75)
    want = np.float32(fused * np.float32(1.5)) + np.float32(np.float32(-0.75) * c.reshape(m, n))
    assert np.array_equal(got, want.astype(np.float32))


def test_oracle_f32_small_integers_and_fp64_truth():
    m, n, k = 33, 65, 129
    a, b, c = O.make_inputs(O.F32F32F32, m, n, k, kind=O.FILL_SMALL_INT, seed=5)
    want = (a.reshape(m, k).astype(np.int64) @ b.reshape(k, n).astype(np.int64) * 2 - c.reshape(m, n).astype(np.int64))
    assert np.array_equal(O.gemm(O.F32F32F32, a, b, c, m, n, k, O.ROW, O.ROW, 2, -1), want.astype(np.float32))
    a, b, c = O.make_inputs(O.F32F32F32, m, n, k, seed=6)
    truth, mag = O.gemm_f64(O.F32F32F32, a, b, c, m, n, k, O.ROW, O.COL, 1.0, 1.0)
    got = O.gemm(O.F32F32F32, a, b, c, m, n, k, O.ROW, O.COL, 1.0, 1.0).astype(np.float64)
    assert np.all(np.abs(got - truth) <= (k + 2) * 2.0 ** -24 * (mag + np.abs(c.reshape(m, n))))
