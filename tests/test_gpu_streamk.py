"""Stream-K on the GPU: the tiles past the last whole round of the compute units cut along K, partial sums through the
library's workspace, pieces added in a fixed order (reference's tail problem: the persistent grid of
nvidia/kernel_functors/bf16_mma_gemm.cuh:42-48).  Bit-exact against the CPU oracle on integer-valued data, where
every summation order gives the same bits; N(0,1) data within the bundle's tolerance and the same bits on every run."""
import itertools

import numpy as np
import pytest
import torch

import oracle_lib as O

pytestmark = pytest.mark.gpu

MFMA = 4
TYPES = (O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16)


def exact_kind(types):
    return O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def slab(types):
    return 128 // np.dtype(O.IN_DTYPE[types]).itemsize


@pytest.mark.parametrize("types", TYPES)
def test_small_grids_bit_exact(G, types):
    """Fewer tiles than compute units: every tile is cut.  Runs of 2..7 slabs, pieces that end with their tile and
    pieces that cross into the next, ragged M and N, alpha / beta and C in the second launch."""
    s = slab(types)
    cases = [(512, 512, 24), (768, 1024, 9), (300, 520, 40), (1024, 256, 64), (257, 255, 31), (2048, 1792, 5),
             (1024, 1024, 100), (2048, 1792, 40)]
    for variant, (m, n, slabs), (al, be), lb in itertools.product((7, 8), cases, [(1, 0), (2, -1)], (O.COL, O.ROW)):
        k = s * slabs
        if lb == O.ROW and n % (16 * s // 128):
            continue   # rows of a row-major B that are not whole 16-byte pieces: the register-staged kernel, no stream-K
        p = G.capi.plan(types, m, n, k, O.ROW, lb, MFMA, variant)
        assert p.streamk_tiles > 0 and p.streamk_blocks > p.streamk_tiles and p.workspace_bytes > 0, (m, n, k)
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs + variant)
        print("case", types, variant, m, n, k, al, be, lb, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, lb, al, be, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, lb, al, be)), (types, variant, m, n, k, lb)


@pytest.mark.parametrize("types", (O.S8S8S32, O.BF16BF16F32))
@pytest.mark.parametrize("shape", [(5120, 5120, 4), (4864, 4864, 6), (5000, 5100, 5)])
def test_one_and_a_half_rounds_bit_exact(G, types, shape):
    """400 / 361 / 400 tiles on 256 compute units: a whole round of plain tiles and the stream-K runs in one launch."""
    m, n, slabs = shape
    k = slab(types) * slabs
    for variant, lb in itertools.product((7, 8), (O.COL, O.ROW)):
        if lb == O.ROW and n % (16 * slab(types) // 128):
            continue
        p = G.capi.plan(types, m, n, k, O.ROW, lb, MFMA, variant, *G.capi.device_props())
        assert p.streamk_tiles == (-(-m // 256)) * (-(-n // 256)) % G.capi.device_props()[0]
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=7)
        print("case", types, variant, m, n, k, lb, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, lb, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, lb, 1, 1)), (types, variant, m, n, k, lb)


@pytest.mark.parametrize("types", TYPES[1:])
def test_normal_data_within_tolerance_and_repeatable(G, types):
    """N(0,1) operands: within the bundle's tolerance of the fp64 truth, and the same bits on every run (the pieces
    of a tile are added in the order of their blocks, not of their arrival)."""
    m, n, k = 1280, 1536, 2048
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=5)
    truth, _ = O.gemm_f64(types, a, b, c, m, n, k, O.ROW, O.COL, 1.0, 1.0)
    first = None
    for rep in range(3):
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1.0, 1.0, MFMA, 7)
        G.assert_within(types, got, truth, f"stream-K vs fp64 truth {types}")
        if first is None:
            first = got
        assert np.array_equal(got, first)


def test_unaligned_operands_fall_back(G):
    """An explicit stream-K variant on operands that are not 16-byte aligned runs the plain launch."""
    types, (m, n, k) = O.BF16BF16F32, (512, 512, 1024)
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=3)
    got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, MFMA, 7, misalign=1)
    assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1))


def test_two_streams_at_once(G):
    """Stream-K launches from two host threads on two streams, different shapes, twenty calls each: every
    (device, stream) has its own workspace in the library's pool, which grows under a lock, so neither side may see the
    other's partial sums.  Every result bit-exact against the oracle."""
    import threading

    types = O.S8S8S32
    shapes = [(1024, 1024, 16384), (768, 512, 24576)]
    jobs = []
    for i, (m, n, k) in enumerate(shapes):
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_INT8_UNIFORM, seed=31 + i)
        assert G.capi.plan(types, m, n, k, O.ROW, O.COL, MFMA, 7, *G.capi.device_props()).streamk_blocks > 0
        jobs.append(dict(m=m, n=n, k=k, a=G.up(a), b=G.up(b), c=G.up(c), stream=torch.cuda.Stream(),
                         want=O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1), outs=[], err=None))
    torch.cuda.synchronize()

    def work(j):
        try:
            for _ in range(20):
                d = torch.empty(j["m"] * j["n"], dtype=torch.int32, device="cuda")
                G.capi.gemm(types, j["a"], j["b"], j["c"], d, j["m"], j["n"], j["k"], O.ROW, O.COL, 1, 1, MFMA, 7,
                            j["stream"].cuda_stream)
                j["outs"].append(d)
            j["stream"].synchronize()
        except Exception as e:   # reported by the main thread
            j["err"] = e

    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    for j in jobs:
        assert j["err"] is None, j["err"]
        for d in j["outs"]:
            assert np.array_equal(d.cpu().numpy().reshape(j["m"], j["n"]), j["want"]), (j["m"], j["n"], j["k"])
