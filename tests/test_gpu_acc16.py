"""GPU parity of the two opt-in modes with a 16-bit running sum (bf16bf16bf16_acc16, f16f16f16_acc16) against the
CPU oracle, through the C ABI.

Rungs 0-3 add a chunk's products in k order like the oracle: bit-exact on any data.  The MFMA rung takes a chunk's
fp32 sum from one matrix instruction, whose internal order is the hardware's: bit-exact where every chunk sum is an
exact integer (then the order cannot matter, while the 16-bit rounding of the running sum still happens), and
within a few 16-bit spacings of the oracle on N(0,1) data.
"""
import itertools

import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu

BF, FH = O.BF16BF16BF16_ACC16, O.F16F16F16_ACC16
TYPES = (BF, FH)
LAYOUTS = list(itertools.product((O.ROW, O.COL), repeat=2))
MFMA, SKINNY = 4, 5
SHAPES = [(1, 1, 1), (3, 5, 7), (65, 63, 33), (128, 128, 64), (100, 130, 70), (257, 129, 200), (31, 300, 1023), (256, 384, 2048)]
SPACING = {BF: 2.0 ** -8, FH: 2.0 ** -11}   # relative spacing of the output type


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def encode(types, x):
    x = np.asarray(x, dtype=np.float32)
    if types == BF:
        return (x.view(np.uint32) >> 16).astype(np.uint16)
    return x.astype(np.float16).view(np.uint16)


def integer_inputs(types, m, n, k, seed):
    """Integers large enough that the running sum outgrows the 16-bit mantissa (so it is rounded along the way)
    and small enough that every chunk sum is an exact fp32 integer."""
    top = 6 if types == BF else 30
    rng = np.random.default_rng(seed)
    a = encode(types, rng.integers(-top, top + 1, m * k)); b = encode(types, rng.integers(-top, top + 1, k * n))
    c = encode(types, rng.integers(-64, 65, m * n))
    return a, b, c


@pytest.mark.parametrize("types", TYPES)
@pytest.mark.parametrize("rung", (0, 1, 2, 3, MFMA))
def test_bit_exact_on_integer_data(G, types, rung):
    rounded = 0
    for (la, lb), (m, n, k), (al, be) in itertools.product(LAYOUTS, SHAPES, [(1, 0), (2, -1)]):
        a, b, c = integer_inputs(types, m, n, k, seed=m + 3 * n + 7 * k)
        print("case", types, rung, la, lb, m, n, k, al, be, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, al, be, rung)
        ref = O.gemm(types, a, b, c, m, n, k, la, lb, al, be)
        assert np.array_equal(got, ref), (types, rung, la, lb, m, n, k, al, be)
        if k >= 1023:
            fp32_acc = O.BF16BF16BF16 if types == BF else O.F16F16F16
            rounded += int((ref != O.gemm(fp32_acc, a, b, c, m, n, k, la, lb, al, be)).sum())
    assert rounded > 0   # the cases did reach the range where a 16-bit running sum differs from an fp32 one


@pytest.mark.parametrize("types", TYPES)
@pytest.mark.parametrize("rung", (0, 1, 2, 3))
def test_valu_rungs_bit_exact_on_normal_data(G, types, rung):
    for (la, lb), (m, n, k) in itertools.product(LAYOUTS, [(65, 63, 129), (128, 192, 260)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=11)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 1.0, 0.5, rung)
        ref = O.gemm(types, a, b, c, m, n, k, la, lb, 1.0, 0.5)
        assert np.array_equal(got, ref), (types, rung, la, lb, m, n, k)


@pytest.mark.parametrize("types", TYPES)
def test_mfma_close_to_the_oracle_on_normal_data(G, types):
    """The chunk sums differ from the oracle's in the last fp32 bits at most, which now and then moves a 16-bit
    rounding of the running sum by one spacing: most outputs equal, none further than 4 spacings of
    max(|value|, rms) away."""
    for (la, lb), (m, n, k) in itertools.product(LAYOUTS, [(256, 256, 512), (300, 200, 1000)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=17)
        got = O.out_to_f64(types, G.run_gemm(types, a, b, c, m, n, k, la, lb, 1.0, 1.0, MFMA))
        ref = O.out_to_f64(types, O.gemm(types, a, b, c, m, n, k, la, lb, 1.0, 1.0))
        rms = np.sqrt((ref ** 2).mean())
        assert (np.abs(got - ref) <= 4 * SPACING[types] * np.maximum(np.abs(ref), rms)).all(), (types, la, lb, m, n, k)
        assert (got == ref).mean() > 0.9, (types, la, lb, m, n, k, float((got == ref).mean()))


@pytest.mark.parametrize("types,limit", [(BF, 4096), (FH, 16384)])
@pytest.mark.parametrize("rung", (0, 2, MFMA))
def test_ones_stop_growing(G, types, limit, rung):
    """The closed form that tells the running sum's width and the chunk length: K ones give min(K, limit)."""
    m, n = 2, 3
    for k in (limit, limit + 8 * 37 + 5):
        ones = encode(types, np.ones(max(m, n) * k))
        got = O.out_to_f64(types, G.run_gemm(types, ones[:m * k], ones[:n * k], None, m, n, k, O.ROW, O.COL, 1, 0, rung))
        assert (got == limit).all(), (types, rung, k, got)


def test_fp16_epilogue_is_one_fused_multiply_add(G):
    """alpha * acc lands on a rounding tie that the product beta * c must break (multiply, round, add would not):
    acc = 1 + 2^-10 from a single product, alpha = 1.5, beta * c = -/+ 2^-24."""
    a = encode(FH, [1 + 2.0 ** -10]); b = encode(FH, [1.0])
    for cval, want in ((-2.0 ** -24, 0x3E01), (2.0 ** -24, 0x3E02), (0.0, 0x3E02)):
        c = encode(FH, [cval])
        for rung in (0, 1, 2, 3, MFMA):
            got = G.run_gemm(FH, a, b, c, 1, 1, 1, O.ROW, O.COL, 1.5, 1.0, rung)
            assert int(got[0, 0]) == want, (cval, rung, hex(int(got[0, 0])))
        assert int(O.gemm(FH, a, b, c, 1, 1, 1, O.ROW, O.COL, 1.5, 1.0)[0, 0]) == want


@pytest.mark.parametrize("types", TYPES)
def test_unaligned_operands_and_empty_k(G, types):
    m, n, k = 70, 66, 95
    a, b, c = integer_inputs(types, m, n, k, seed=3)
    for rung in (1, 3, MFMA):
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, rung, misalign=1)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)), rung
        got = G.run_gemm(types, a[:0], b[:0], c, m, n, 0, O.ROW, O.COL, 1, 1, rung)   # K = 0: D = beta * C
        assert np.array_equal(got, O.gemm(types, a[:0], b[:0], c, m, n, 0, O.ROW, O.COL, 1, 1)), rung


@pytest.mark.parametrize("types", TYPES)
def test_plan_variants_and_refusals(G, types):
    capi = G.capi
    assert capi.lib.gz_variant_count(types, MFMA) == 1 and capi.lib.gz_variant_count(types, SKINNY) == 0
    p = capi.plan(types, 1000, 500, 300, O.ROW, O.COL, capi.RUNG_AUTO, 0)
    assert (p.rung, p.tile_m, p.tile_n, p.threads, p.grid) == (MFMA, 128, 128, 256, 8 * 4)
    a, b, c = integer_inputs(types, 16, 256, 128, seed=1)
    with pytest.raises(capi.GzError) as e:   # decode shape: the weight-streaming rung is fp32-accumulate only
        G.run_gemm(types, a, b, c, 16, 256, 128, O.ROW, O.COL, 1, 0, SKINNY)
    assert e.value.status == capi.ERR_UNSUPPORTED
    with pytest.raises(capi.GzError) as e:
        G.run_gemm(types, a, b, c, 16, 256, 128, O.ROW, O.COL, 1, 0, MFMA, variant=2)
    assert e.value.status == capi.ERR_UNSUPPORTED
    # AUTO on the decode shape takes the MFMA rung
    got = G.run_gemm(types, a, b, c, 16, 256, 128, O.ROW, O.COL, 1, 0, capi.RUNG_AUTO)
    assert np.array_equal(got, O.gemm(types, a, b, c, 16, 256, 128, O.ROW, O.COL, 1, 0))
