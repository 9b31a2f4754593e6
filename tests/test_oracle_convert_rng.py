"""Pins the oracle's converters, Philox and fills (CPU only)."""
import json
import math
from pathlib import Path

import numpy as np
import pytest
import torch

import oracle_lib as O

GOLDEN = Path(__file__).parent / "golden"


# ---------------------------------------------------------------- bf16 / fp16 converters
def f32(x):
    return float(np.float32(x))


@pytest.mark.parametrize("value,bits", [
    (1.0, 0x3F80), (-1.0, 0xBF80), (0.0, 0x0000), (-0.0, 0x8000),
    (1.0 + 2.0 ** -8, 0x3F80),        # tie -> even (down)
    (1.0 + 3 * 2.0 ** -8, 0x3F82),    # tie -> even (up)
    (1.0 + 2.0 ** -8 + 2.0 ** -20, 0x3F81),  # just above the tie
    (float("inf"), 0x7F80), (float("-inf"), 0xFF80),
    (3.3895313892515355e38, 0x7F7F),  # largest finite bf16
    (3.4028234663852886e38, 0x7F80),  # FLT_MAX rounds to inf
])
def test_bf16_known_answers(value, bits):
    assert O.lib.oracle_f32_to_bf16(f32(value)) == bits


def test_bf16_nan_is_quiet():
    b = O.lib.oracle_f32_to_bf16(float("nan"))
    assert (b & 0x7F80) == 0x7F80 and (b & 0x007F) != 0 and (b & 0x0040)


@pytest.mark.parametrize("value,bits", [
    (1.0, 0x3C00), (-2.0, 0xC000), (0.0, 0x0000), (-0.0, 0x8000),
    (65504.0, 0x7BFF), (65519.996, 0x7BFF), (65520.0, 0x7C00), (1e9, 0x7C00),
    (2.0 ** -24, 0x0001),              # smallest subnormal
    (2.0 ** -25, 0x0000),              # tie -> even (0)
    (2.0 ** -25 * 1.0000001, 0x0001),  # just above the tie
    (1.5 * 2.0 ** -24, 0x0002),        # tie between subnormals 1 and 2 -> even
    (2.0 ** -14, 0x0400),              # smallest normal
    (2.0 ** -14 - 2.0 ** -25, 0x0400), # rounds up into the normal range
    (1.0 + 2.0 ** -11, 0x3C00), (1.0 + 3 * 2.0 ** -11, 0x3C02),
    (float("inf"), 0x7C00), (float("-inf"), 0xFC00),
])
def test_f16_known_answers(value, bits):
    assert O.lib.oracle_f32_to_f16(f32(value)) == bits


def test_16bit_round_trip_exhaustive():
    """x == to16(to32(x)) for every non-NaN 16-bit pattern, and to32 matches numpy / torch."""
    allbits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    t = torch.from_numpy(allbits.view(np.int16))
    bf_torch = t.view(torch.bfloat16).float().numpy()
    f16_np = allbits.view(np.float16).astype(np.float32)
    for b in range(1 << 16):
        vb = O.lib.oracle_bf16_to_f32(b)
        vh = O.lib.oracle_f16_to_f32(b)
        if math.isnan(vb):
            assert math.isnan(bf_torch[b])
        else:
            assert np.float32(vb).view(np.uint32) == bf_torch[b].view(np.uint32)
            assert O.lib.oracle_f32_to_bf16(vb) == b
        if math.isnan(vh):
            assert math.isnan(f16_np[b])
        else:
            assert np.float32(vh).view(np.uint32) == f16_np[b].view(np.uint32)
            assert O.lib.oracle_f32_to_f16(vh) == b


def test_converters_match_numpy_and_torch_on_random_floats():
    rng = np.random.default_rng(5)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(20000) * 1e-6).astype(np.float32),     # fp16 subnormal range
        (rng.standard_normal(20000) * 3e4).astype(np.float32),      # near fp16 overflow
        rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32),  # any bit pattern
    ])
    x = x[np.isfinite(x)]
    want_h = x.astype(np.float16).view(np.uint16)
    want_b = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got_h = np.array([O.lib.oracle_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    got_b = np.array([O.lib.oracle_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got_h, want_h)
    assert np.array_equal(got_b, want_b)


# ---------------------------------------------------------------- Philox
def test_philox_known_answer_vectors():
    kat = json.loads((GOLDEN / "philox4x32_10_kat.json").read_text())["vectors"]
    assert len(kat) == 3
    for v in kat:
        out = O.philox([int(x, 16) for x in v["counter"]], [int(x, 16) for x in v["key"]])
        assert out == [int(x, 16) for x in v["output"]]


def test_fill_is_keyed_by_seed_and_element_index():
    """Element i uses counter {i,0,0,0}, key {seed,0}: int8 = low byte of word 0."""
    seed, n = 2025, 257
    got = O.fill(n, O.DT_INT8, O.FILL_INT8_UNIFORM, 1.0, seed)
    want = np.array([np.uint8(O.philox([i, 0, 0, 0], [seed, 0])[0] & 0xFF).astype(np.int8) for i in range(n)])
    assert np.array_equal(got, want)
    # a 64-bit seed feeds both key words
    big = (7 << 32) | 9
    got = O.fill(4, O.DT_INT32, O.FILL_INT8_UNIFORM, 1.0, big)
    want = [int(np.uint8(O.philox([i, 0, 0, 0], [9, 7])[0] & 0xFF).astype(np.int8)) for i in range(4)]
    assert got.tolist() == want
    # different seeds give different streams, same seed the same stream
    assert not np.array_equal(O.fill(64, O.DT_INT8, 0, 1.0, 1), O.fill(64, O.DT_INT8, 0, 1.0, 2))
    assert np.array_equal(O.fill(64, O.DT_INT8, 0, 1.0, 1), O.fill(64, O.DT_INT8, 0, 1.0, 1, threads=1))


def test_fill_int8_covers_range_uniformly():
    x = O.fill(1 << 20, O.DT_INT8, O.FILL_INT8_UNIFORM, 1.0, 11)
    counts = np.bincount(x.astype(np.int32) + 128, minlength=256)
    assert counts.min() > 0 and x.min() == -128 and x.max() == 127
    expected = (1 << 20) / 256
    chi2 = ((counts - expected) ** 2 / expected).sum()
    assert chi2 < 400  # 255 dof: mean 255, sd 22.6


def test_fill_normal_moments_and_shape():
    x = O.fill(1 << 21, O.DT_F32, O.FILL_NORMAL, 1.0, 2025).astype(np.float64)
    n = x.size
    assert abs(x.mean()) < 4 / math.sqrt(n)
    assert abs(x.var() - 1.0) < 4 * math.sqrt(2.0 / n)
    assert abs((x ** 3).mean()) < 4 * math.sqrt(15.0 / n)
    assert abs((x ** 4).mean() - 3.0) < 4 * math.sqrt(96.0 / n)
    # distribution function against the exact normal CDF
    xs = np.sort(x)
    cdf = 0.5 * (1.0 + np.vectorize(math.erf)(xs[::997] / math.sqrt(2.0)))
    emp = (np.arange(n)[::997] + 0.5) / n
    assert np.abs(cdf - emp).max() < 2.0 / math.sqrt(n) * 1.36 * 1.5  # Kolmogorov-Smirnov, generous
    # scale multiplies the variate
    y = O.fill(1024, O.DT_F32, O.FILL_NORMAL, 0.02, 2025)
    assert np.allclose(y, O.fill(1024, O.DT_F32, O.FILL_NORMAL, 1.0, 2025) * np.float32(0.02), rtol=1e-6)


def test_normal_transform_accuracy():
    """The libm-free log / cos used by the fill agree with libm to fp32 accuracy."""
    rng = np.random.default_rng(3)
    w0 = rng.integers(0, 2 ** 32, 5000, dtype=np.uint64)
    w1 = rng.integers(0, 2 ** 32, 5000, dtype=np.uint64)
    for a, b in zip(w0.tolist(), w1.tolist()):
        u1 = ((a >> 8) + 1) * 2.0 ** -24
        u2 = (b >> 8) * 2.0 ** -24
        want = math.sqrt(-2.0 * math.log(u1)) * math.cos(2.0 * math.pi * u2)
        got = O.lib.oracle_normal_from_words(a, b)
        assert abs(got - want) < 5e-6 * max(1.0, abs(want)) + 2e-6


def test_fill_uniform_and_small_int():
    u = O.fill(1 << 18, O.DT_F32, O.FILL_UNIFORM_PM1, 1.0, 3)
    assert u.min() >= -1.0 and u.max() < 1.0 and abs(u.mean()) < 0.01 and abs(u.var() - 1 / 3) < 0.01
    s = O.fill(1 << 18, O.DT_BF16, O.FILL_SMALL_INT, 1.0, 3)
    vals = set(np.unique(O.bf16_to_f32(s)).tolist())
    assert vals <= {-2.0, -1.0, 0.0, 1.0} and {-1.0, 0.0, 1.0} <= vals
    h = O.fill(1 << 12, O.DT_F16, O.FILL_UNIFORM_PM1, 1.0, 3)
    f = O.fill(1 << 12, O.DT_F32, O.FILL_UNIFORM_PM1, 1.0, 3)
    assert np.array_equal(h, f.astype(np.float16).view(np.uint16))
