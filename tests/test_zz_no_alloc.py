"""gz_gemm_static_scratch on the GPU: the entry point for callers that cannot allocate.  Its stream-K launches keep
their partial sums in the library's static device buffer; everything else is gz_gemm.  It has no counterpart in the
reference, so the check is against gz_gemm on the same inputs (bit for bit, same decomposition) and, for int8,
against the CPU oracle; two calls in a row share the buffer, the second on a smaller problem."""
import importlib

import numpy as np
import pytest
import torch

import oracle_lib as O

pytestmark = pytest.mark.gpu

MFMA = 4


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def run(G, entry, types, a, b, c, m, n, k, alpha, beta, variant, rung=MFMA):
    """D of one call through `entry` (capi.gemm or capi.gemm_static_scratch), with guard words around it."""
    da, db, dc = G.up(a), G.up(b), G.up(c)
    sentinel = 0x5A5A if O.OUT_DTYPE[types] == np.uint16 else 0x5A5A5A5A
    guard = 64
    full = torch.full((m * n + 2 * guard,), sentinel, dtype=G.out_torch_dtype(types), device=G.dev())
    dd = full[guard:guard + m * n]
    entry(types, da, db, dc, dd, m, n, k, O.ROW, O.COL, alpha, beta, rung, variant,
          torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    host = full.cpu()
    assert (host[:guard] == sentinel).all() and (host[guard + m * n:] == sentinel).all(), "wrote outside D"
    return host[guard:guard + m * n].numpy().view(O.OUT_DTYPE[types]).reshape(m, n)


@pytest.mark.parametrize("types,kind", [(O.S8S8S32, O.FILL_INT8_UNIFORM), (O.BF16BF16F32, O.FILL_NORMAL),
                                        (O.F16F16F16, O.FILL_NORMAL)])
def test_two_calls_in_a_row_match_gz_gemm(G, types, kind):
    capi = G.capi
    slab = 128 // np.dtype(O.IN_DTYPE[types]).itemsize
    # the launcher's own choice on a small grid with a long K, then a smaller problem on an explicit stream-K variant
    calls = [((1024, 1024, 128 * slab), 0), ((512, 768, 48 * slab), 7)]
    for (m, n, k), variant in calls:
        p = capi.plan(types, m, n, k, O.ROW, O.COL, MFMA, variant, *capi.device_props())
        assert p.streamk_tiles > 0 and 0 < p.workspace_bytes <= capi.STATIC_SCRATCH_BYTES, (m, n, k, p.as_dict())
    outs = []
    for (m, n, k), variant in calls:   # back to back: the second call finds the first one's sums in the buffer
        a, b, c = O.make_inputs(types, m, n, k, kind=kind, seed=11 + m)
        print("static scratch", types, m, n, k, variant, flush=True)
        outs.append((run(G, capi.gemm_static_scratch, types, a, b, c, m, n, k, 2, -1, variant), (a, b, c, m, n, k, variant)))
    for got, (a, b, c, m, n, k, variant) in outs:
        want = run(G, capi.gemm, types, a, b, c, m, n, k, 2, -1, variant)
        assert np.array_equal(got, want), (types, m, n, k, variant)
        if types == O.S8S8S32:   # bit-exact against the CPU oracle as well
            assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 2, -1)), (m, n, k)
        else:                    # within the bundle's tolerance of the fp64 truth
            truth, _ = O.gemm_f64(types, a, b, c, m, n, k, O.ROW, O.COL, 2.0, -1.0)
            G.assert_within(types, got, truth, f"static scratch {types} {m}x{n}x{k}")


def test_split_k_of_the_streaming_rung_uses_the_same_buffer(G):
    """The weight-streaming rung's split K (65 ... 128 rows, K >= 8192) leaves its partial sums in the same static
    buffer: two calls in a row, the second smaller, against gz_gemm bit for bit and against the oracle."""
    capi = G.capi
    types = O.BF16BF16F32
    outs = []
    for (m, n, k) in [(128, 14336, 8192), (96, 8200, 8192)]:
        p = capi.plan_static_scratch(types, m, n, k, O.ROW, O.COL, 5, 0)
        assert p.split_k > 1 and 0 < p.workspace_bytes <= capi.STATIC_SCRATCH_BYTES, p.as_dict()
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=m)
        print("static scratch, streaming rung", m, n, k, flush=True)
        outs.append((run(G, capi.gemm_static_scratch, types, a, b, c, m, n, k, 2, -1, 0, rung=5), (a, b, c, m, n, k)))
    for got, (a, b, c, m, n, k) in outs:
        assert np.array_equal(got, run(G, capi.gemm, types, a, b, c, m, n, k, 2, -1, 0, rung=5)), (m, n, k)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 2, -1)), (m, n, k)


def test_more_than_the_buffer_holds_is_refused(G):
    """400 tiles with 144 past the whole round, forced onto stream-K: 399 slots, more than the buffer's 384.
    gz_gemm_static_scratch says so and launches nothing; gz_gemm runs it; the next call that fits still works."""
    capi = G.capi
    types, (m, n, k) = O.S8S8S32, (5120, 5120, 512)
    p = capi.plan(types, m, n, k, O.ROW, O.COL, MFMA, 7, *capi.device_props())
    assert p.workspace_bytes > capi.STATIC_SCRATCH_BYTES
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_INT8_UNIFORM, seed=2)
    with pytest.raises(capi.GzError) as e:
        run(G, capi.gemm_static_scratch, types, a, b, c, m, n, k, 1, 0, 7)
    assert e.value.status == capi.ERR_UNSUPPORTED and "scratch" in str(e.value)
    want = O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 0)
    assert np.array_equal(run(G, capi.gemm, types, a, b, c, m, n, k, 1, 0, 7), want)
    # without stream-K nothing is needed, and a launch that fits runs after the refusal
    assert np.array_equal(run(G, capi.gemm_static_scratch, types, a, b, c, m, n, k, 1, 0, 5), want)
    m, n, k = 512, 512, 3072
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_INT8_UNIFORM, seed=3)
    assert np.array_equal(run(G, capi.gemm_static_scratch, types, a, b, c, m, n, k, 1, 1, 7),
                          O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1))


def test_launchers_choice_stays_within_the_buffer(G):
    """bf16 3328 x 3328 x 43264 on 256 compute units: gz_plan takes stream-K over all 169 tiles with a workspace above
    the static buffer.  Under the launcher's own choice (variant 0) gz_gemm_static_scratch does not refuse: it takes
    the best plan that fits, which gz_plan_static_scratch reports.  Another decomposition is another summation order,
    so the result is held to the fp64 truth on bands of rows, as gz_gemm's is."""
    capi = G.capi
    types, (m, n, k) = O.BF16BF16F32, (3328, 3328, 43264)
    cus, lds = capi.device_props()
    p = capi.plan(types, m, n, k, O.ROW, O.COL, -1, 0, cus, lds)
    ps = capi.plan_static_scratch(types, m, n, k, O.ROW, O.COL, -1, 0, cus, lds)
    assert ps.workspace_bytes <= capi.STATIC_SCRATCH_BYTES
    if cus == 256:
        assert p.workspace_bytes > capi.STATIC_SCRATCH_BYTES and p.streamk_blocks > 0
    it = torch.int16
    a = torch.empty(m * k, dtype=it, device="cuda"); b = torch.empty(k * n, dtype=it, device="cuda")
    capi.fill(a, m * k, O.DT_BF16, O.FILL_NORMAL, 1.0, 11); capi.fill(b, k * n, O.DT_BF16, O.FILL_NORMAL, 1.0, 12)
    sptr = torch.cuda.current_stream().cuda_stream
    outs = []
    for entry in (capi.gemm_static_scratch, capi.gemm):
        d = torch.empty(m * n, dtype=torch.float32, device="cuda")
        entry(types, a, b, None, d, m, n, k, O.ROW, O.COL, 1, 0, -1, 0, sptr)
        torch.cuda.synchronize()
        outs.append(d.cpu().numpy().reshape(m, n))
    ha = a.cpu().numpy().view(np.uint16); hb = b.cpu().numpy().view(np.uint16)
    for rows in ((0, 4), (1660, 1664), (m - 4, m)):
        truth, _ = O.gemm_f64(types, ha, hb, None, m, n, k, O.ROW, O.COL, 1.0, 0.0, rows=rows)
        for got in outs:
            G.assert_within(types, got[rows[0]:rows[1]], truth, f"static scratch, launcher's choice, rows {rows}")


def test_plan_static_scratch_equals_plan_where_it_fits(G):
    capi = G.capi
    for types, m, n, k in [(O.BF16BF16F32, 4352, 4096, 4096), (O.S8S8S32, 1024, 1024, 16384), (O.F16F16F16, 4096, 4096, 4096)]:
        p = capi.plan(types, m, n, k, O.ROW, O.COL).as_dict()
        assert p["workspace_bytes"] <= capi.STATIC_SCRATCH_BYTES
        assert capi.plan_static_scratch(types, m, n, k, O.ROW, O.COL).as_dict() == p
