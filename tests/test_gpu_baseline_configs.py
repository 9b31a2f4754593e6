"""The five benchmark configurations (int8 1024^3 and 8192^3, bf16 4096^3, ragged fp16, decode shapes) at their full sizes, through the C ABI.

Small ones are compared element for element with the CPU oracle.  The large ones (4096^3, 8192^3)
are checked through size-independent properties that are exact for integers -- D x = A (B x) and
x^T D = (x^T A) B in int64 for random x -- plus bands of rows against the oracle.
"""
import numpy as np
import pytest
import torch

import oracle_lib as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def device_inputs(G, types, m, n, k, kind, seed, scale_b=1.0):
    it = torch.int8 if types == O.S8S8S32 else torch.int16
    a = torch.empty(m * k, dtype=it, device="cuda"); b = torch.empty(k * n, dtype=it, device="cuda")
    G.capi.fill(a, m * k, O.IN_DT[types], kind, 1.0, seed); G.capi.fill(b, k * n, O.IN_DT[types], kind, scale_b, seed + 1)
    torch.cuda.synchronize()
    ha = a.cpu().numpy(); hb = b.cpu().numpy()
    if types != O.S8S8S32:
        ha = ha.view(np.uint16); hb = hb.view(np.uint16)
    return a, b, ha, hb


def test_c1_s8_1024_row_row_bit_exact_every_rung(G):
    m = n = k = 1024
    a, b, c = O.make_inputs(O.S8S8S32, m, n, k, seed=2025)
    ref = O.gemm(O.S8S8S32, a, b, None, m, n, k, O.ROW, O.ROW, 1, 0)
    lit = np.zeros((m, n), np.int32)  # the literal reference loop on a band, as a cross-check of the checker
    band = O.gemm(O.S8S8S32, a, b, None, m, n, k, O.ROW, O.ROW, 1, 0, rows=(100, 116), naive=True)
    assert np.array_equal(band[100:116], ref[100:116])
    for rung in (-1, 0, 1, 2, 3, 4):
        got = G.run_gemm(O.S8S8S32, a, b, None, m, n, k, O.ROW, O.ROW, 1, 0, rung)
        assert np.array_equal(got, ref), rung
    ref11 = O.gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.ROW, 1, 1)
    assert np.array_equal(G.run_gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.ROW, 1, 1, -1), ref11)


def test_c2_bf16_4096_row_col_f32(G):
    m = n = k = 4096
    types = O.BF16BF16F32
    a, b, ha, hb = device_inputs(G, types, m, n, k, O.FILL_NORMAL, 2025)
    assert np.array_equal(ha, O.fill(m * k, O.DT_BF16, O.FILL_NORMAL, 1.0, 2025))  # same bytes on both sides
    d = torch.empty(m * n, dtype=torch.float32, device="cuda")
    G.capi.gemm(types, a, b, None, d, m, n, k, O.ROW, O.COL, 1, 0)
    torch.cuda.synchronize()
    got = d.cpu().numpy().reshape(m, n)
    for r0 in (0, 1777, 4088):  # bands of rows against fp64 truth and against the sequential fp32 oracle
        truth, _ = O.gemm_f64(types, ha, hb, None, m, n, k, O.ROW, O.COL, 1, 0, rows=(r0, r0 + 8))
        G.assert_within(types, got[r0:r0 + 8], truth, f"C2 rows {r0}")
        ref = O.gemm(types, ha, hb, None, m, n, k, O.ROW, O.COL, 1, 0, rows=(r0, r0 + 8))[r0:r0 + 8]
        G.assert_within(types, got[r0:r0 + 8], ref.astype(np.float64), f"C2 rows {r0} vs fp32 oracle")
    # Freivalds: D x == A (B x) in fp64, for every row at once
    rng = np.random.default_rng(0)
    x = rng.choice([-1.0, 1.0], n)
    A = O.bf16_to_f32(ha).reshape(m, k).astype(np.float64); Bt = O.bf16_to_f32(hb).reshape(n, k).astype(np.float64)
    lhs = got.astype(np.float64) @ x
    rhs = A @ (x @ Bt)
    scale = np.sqrt(k * n)  # magnitude of a row's signed sum
    assert np.abs(lhs - rhs).max() <= 1e-4 * scale
    # integer-valued inputs: bit-exact at full size
    G.capi.fill(a, m * k, O.DT_BF16, O.FILL_SMALL_INT, 1.0, 7); G.capi.fill(b, k * n, O.DT_BF16, O.FILL_SMALL_INT, 1.0, 8)
    G.capi.gemm(types, a, b, None, d, m, n, k, O.ROW, O.COL, 1, 0)
    torch.cuda.synchronize()
    A = O.bf16_to_f32(a.cpu().numpy().view(np.uint16)).reshape(m, k); Bt = O.bf16_to_f32(b.cpu().numpy().view(np.uint16)).reshape(n, k)
    want = (A.astype(np.float64) @ Bt.T.astype(np.float64))
    assert np.array_equal(d.cpu().numpy().reshape(m, n).astype(np.float64), want)


def test_c3_s8_8192_row_col_bit_exact(G):
    m = n = k = 8192
    types = O.S8S8S32
    a, b, ha, hb = device_inputs(G, types, m, n, k, O.FILL_INT8_UNIFORM, 2025)
    d = torch.empty(m * n, dtype=torch.int32, device="cuda")
    G.capi.gemm(types, a, b, None, d, m, n, k, O.ROW, O.COL, 1, 0)
    torch.cuda.synchronize()
    got = d.cpu().numpy().reshape(m, n)
    A = ha.reshape(m, k).astype(np.int64); Bt = hb.reshape(n, k).astype(np.int64)
    rng = np.random.default_rng(1)
    for _ in range(2):  # exact in int64: |entries| <= 2^27 * 8192 * 3
        x = rng.integers(-3, 4, n).astype(np.int64)
        assert np.array_equal(got.astype(np.int64) @ x, A @ (Bt.T @ x) if False else A @ (x @ Bt))
        y = rng.integers(-3, 4, m).astype(np.int64)
        assert np.array_equal(y @ got.astype(np.int64), (y @ A) @ Bt.T)
    for r0 in (0, 4093, 8184):
        ref = O.gemm(types, ha, hb, None, m, n, k, O.ROW, O.COL, 1, 0, rows=(r0, r0 + 8))
        assert np.array_equal(got[r0:r0 + 8], ref[r0:r0 + 8])


def test_c4_f16_ragged_row_row(G):
    m, n, k = 4095, 4097, 1023
    types = O.F16F16F16
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_UNIFORM_PM1, seed=2025)
    got = G.run_gemm(types, a, b, None, m, n, k, O.ROW, O.ROW, 1, 0, -1)
    ref = O.gemm(types, a, b, None, m, n, k, O.ROW, O.ROW, 1, 0)
    G.assert_within(types, got, O.out_to_f64(types, ref), "C4 vs oracle")
    truth, _ = O.gemm_f64(types, a, b, None, m, n, k, O.ROW, O.ROW, 1, 0, rows=(4000, 4095))
    G.assert_within(types, got[4000:], truth, "C4 last rows vs fp64 truth")
    # exact on integer-valued inputs, with beta
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=3)
    got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.ROW, 1, 1, -1)
    assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.ROW, 1, 1))


@pytest.mark.parametrize("m", [1, 8, 32, 128])
def test_c5_skinny_bf16(G, m):
    n, k = 14336, 4096
    types = O.BF16BF16BF16
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=2025, scale_b=0.02)
    got = G.run_gemm(types, a, b, None, m, n, k, O.ROW, O.COL, 1, 0, -1)
    truth, _ = O.gemm_f64(types, a, b, None, m, n, k, O.ROW, O.COL, 1, 0)
    G.assert_within(types, got, truth, f"C5 M={m} vs fp64 truth")
    ref = O.gemm(types, a, b, None, m, n, k, O.ROW, O.COL, 1, 0)
    G.assert_within(types, got, O.out_to_f64(types, ref), f"C5 M={m} vs oracle")
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=4)
    got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, -1)
    assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1))


@pytest.mark.parametrize("types", [O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16])
@pytest.mark.parametrize("shape,tile,variant", [((4096, 4096, 512), (256, 256), 0), ((2048, 4096, 1024), (128, 128), 0),
                                                ((2048, 4096, 1024), (256, 128), 4), ((512, 384, 256), (64, 64), 0),
                                                ((256, 128, 128), (64, 64), 0), ((512, 384, 256), (128, 128), 3),
                                                ((512, 384, 256), (128, 128), 11), ((256, 128, 128), (128, 128), 11)])
def test_reference_driver_layout_row_row_direct_kernels(G, types, shape, tile, variant):
    """Row-major A and B (every driver of the reference).  The first shape gives each compute unit a whole 256x256
    tile (hand-scheduled ring kernel, transposing LDS reads for B), the others take the smaller tiles without
    predication: 128x128 on the same ring kernel with two work-groups per compute unit (the launcher's choice, and
    variant 11 on the small grids), 64x64 on the register-staged kernel where larger tiles would leave most compute
    units idle (the launcher's choice; int8 runs that tile on two waves), 256x128 on the
    register-staged kernel and 128x128 on the compiler-scheduled direct-to-LDS kernel (variants 4 and 3)."""
    m, n, k = shape
    p = G.capi.plan(types, m, n, k, O.ROW, O.ROW, 4 if variant else -1, variant)
    assert p.rung == 4 and m % p.tile_m == 0 and n % p.tile_n == 0          # whole tiles: no predicated kernel
    assert (p.tile_m, p.tile_n) == tile
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT   # exact partial sums in any order
    a, b, ha, hb = device_inputs(G, types, m, n, k, kind, 77)
    hc = O.fill(m * n, O.OUT_DT[types], O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT, 1.0, 79)
    got = G.run_gemm(types, ha, hb, hc, m, n, k, O.ROW, O.ROW, 1, 1, 4 if variant else -1, variant)
    rows = (0, m) if m <= 512 else (m - 24, m)
    ref = O.gemm(types, ha, hb, hc, m, n, k, O.ROW, O.ROW, 1, 1, rows=rows)
    assert np.array_equal(got[rows[0]:rows[1]], ref[rows[0]:rows[1]])
    if types != O.S8S8S32:  # N(0,1) operands against fp64 truth
        a, b, ha, hb = device_inputs(G, types, m, n, k, O.FILL_NORMAL, 78)
        got = G.run_gemm(types, ha, hb, None, m, n, k, O.ROW, O.ROW, 1, 0, 4 if variant else -1, variant)
        truth, _ = O.gemm_f64(types, ha, hb, None, m, n, k, O.ROW, O.ROW, 1, 0, rows=(8, 24))
        G.assert_within(types, got[8:24], truth, f"row/row {shape}")


def test_ragged_grid_takes_the_small_tile(G):
    # N = 4097 would need a 17th column of 256-wide tiles for one column of data
    assert G.capi.plan(O.F16F16F16, 4095, 4096 + 100, 1023, O.ROW, O.ROW).tile_m == 128
    assert G.capi.plan(O.BF16BF16F32, 4096, 4096, 4096, O.ROW, O.COL).tile_m == 256
    assert G.capi.plan(O.BF16BF16F32, 2048, 2048, 2048, O.ROW, O.COL).tile_m == 128


@pytest.mark.parametrize("types", [O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16])
@pytest.mark.parametrize("shape,lb", [((4000, 3976, 512), O.COL), ((4000, 3976, 512), O.ROW), ((3841, 4001, 256), O.COL),
                                      ((4090, 4080, 384), O.ROW)])
def test_ragged_m_n_on_the_hand_scheduled_kernels(G, types, shape, lb):
    """M and N that are not multiples of the 256x256 tile (K whole slabs, aligned rows): the direct-to-LDS kernels
    clamp the rows they fetch and predicate the stores.  N = 4001 also makes the rows of D unaligned."""
    m, n, k = shape
    p = G.capi.plan(types, m, n, k, O.ROW, lb)
    assert (p.rung, p.tile_m, p.tile_n) == (4, 256, 256)
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT
    a, b, ha, hb = device_inputs(G, types, m, n, k, kind, 91)
    hc = O.fill(m * n, O.OUT_DT[types], kind, 1.0, 93)
    got = G.run_gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, -1)
    for rows in ((0, 8), (m - 40, m)):   # the first rows and the rows of the last, partial tile
        ref = O.gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, rows=rows)
        assert np.array_equal(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]), (types, shape, lb, rows)
    # every column of the last partial tile column, a few rows spread over M
    for r in (255, 1024, m - 1):
        ref = O.gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, rows=(r, r + 1))
        assert np.array_equal(got[r], ref[r])


@pytest.mark.parametrize("types", [O.S8S8S32, O.BF16BF16F32, O.F16F16F16, O.E4M3E4M3F16])
@pytest.mark.parametrize("shape,lb", [((4352, 4096), O.ROW), ((7168, 7168), O.ROW), ((4352, 4096), O.COL)])
def test_mostly_empty_last_round_runs_as_two_launches(G, types, shape, lb):
    """272 (or 784) tiles of 256x256 on 256 compute units leave a last round of 16 tiles: the launcher cuts the rows
    in two launches (whole rounds of 256x256 tiles, then the remaining rows with a smaller tile), from 24 slabs of K
    on.  (A larger remainder - 68 tiles of 4608^2 - stays one persistent launch.)  The seam between the two row
    ranges, the first and the last rows are compared with the oracle."""
    m, n = shape
    k = 24 * 128 // np.dtype(O.IN_DTYPE[types]).itemsize
    short = G.capi.plan(types, m, n, k - 128, O.ROW, lb)
    assert short.tail_rows == 0, "a short K is one launch"
    assert G.capi.plan(types, 4608, 4608, k, O.ROW, lb).tail_rows == 0, "68 remaining tiles are one launch"
    p = G.capi.plan(types, m, n, k, O.ROW, lb)
    assert p.rung == 4 and (p.tile_m, p.tile_n) == (256, 256) and 0 < p.tail_rows < m and p.tail_tile_m in (64, 128, 256)
    main_tiles = (m - p.tail_rows) // 256 * -(-n // 256)   # past one round of the compute units one work-group per CU walks them
    assert (m - p.tail_rows) % 256 == 0 and p.grid == min(main_tiles, G.capi.device_props()[0]) and p.tail_grid > 0
    # an explicit variant is one launch
    assert G.capi.plan(types, m, n, k, O.ROW, lb, 4, 6).tail_rows == 0
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT
    a, b, ha, hb = device_inputs(G, types, m, n, k, kind, 51)
    hc = O.fill(m * n, O.OUT_DT[types], kind, 1.0, 53)
    got = G.run_gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, -1)
    seam = m - p.tail_rows
    for rows in ((0, 8), (seam - 16, seam + 16), (m - 24, m)):
        ref = O.gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, rows=rows)
        assert np.array_equal(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]), (types, shape, lb, rows)
    # the whole result against the single launch of the same tile (on-device compare would need both; host is enough)
    one = G.run_gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, 4, 5)
    assert np.array_equal(got, one)
    # beta = 0 with no C
    got0 = G.run_gemm(types, ha, hb, None, m, n, k, O.ROW, lb, 1, 0, -1)
    ref = O.gemm(types, ha, hb, None, m, n, k, O.ROW, lb, 1, 0, rows=(seam - 4, seam + 4))
    assert np.array_equal(got0[seam - 4:seam + 4], ref[seam - 4:seam + 4])


@pytest.mark.parametrize("types", [O.S8S8S32, O.BF16BF16F32, O.F16F16F16, O.E4M3E4M3F16])
@pytest.mark.parametrize("variant", [5, 6])
@pytest.mark.parametrize("shape,lb", [((4352, 4096, 3), O.COL), ((8192, 4096, 1), O.ROW), ((4096, 6144, 6), O.COL)])
def test_more_tiles_than_compute_units_on_the_ring_kernel(G, types, variant, shape, lb):
    """272, 512 and 384 whole 256x256 tiles: past one round of the compute units the ring kernel is persistent - a
    work-group walks several tiles and asks for the next tile's first slab before it stores the current one.  K is
    1, 3 or 6 slabs, so the prefetched groups are all, most or a few of a tile's copies.  First and last rows, and
    rows of tiles that are a work-group's second or third, against the oracle; everything against the same kernel
    launched with one work-group per tile (variants 9 and 10)."""
    m, n, slabs = shape
    k = slabs * 128 // np.dtype(O.IN_DTYPE[types]).itemsize
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT
    a, b, ha, hb = device_inputs(G, types, m, n, k, kind, 71)
    hc = O.fill(m * n, O.OUT_DT[types], kind, 1.0, 73)
    print("case", types, variant, shape, lb, flush=True)
    got = G.run_gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, 4, variant)
    for rows in ((0, 4), (1020, 1028), (m // 2 - 2, m // 2 + 2), (m - 4, m)):
        ref = O.gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, rows=rows)
        assert np.array_equal(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]), (types, variant, shape, lb, rows)
    one = G.run_gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, 4, variant + 4)
    assert np.array_equal(got, one)


@pytest.mark.parametrize("types", [O.S8S8S32, O.BF16BF16F32, O.F16F16F16, O.E4M3E4M3F16, O.F32F32F32])
@pytest.mark.parametrize("variant", [5, 6])
@pytest.mark.parametrize("shape,lb", [((4360, 4096, 3), O.COL), ((8200, 4080, 1), O.ROW), ((4100, 6128, 6), O.COL),
                                      ((4112, 4336, 2), O.ROW)])
def test_more_ragged_tiles_than_compute_units_on_the_ring_kernel(G, types, variant, shape, lb):
    """288, 528, 408 and 289 tiles of 256x256 with a last row and / or column of tiles that reaches past the matrix:
    the persistent launch of the kernel's ragged instance.  A work-group's next tile may be one whose rows or columns
    are clamped while its current one is not (and the other way round), so the first copies of the next tile, asked
    for before the current one is stored, must use the next tile's offsets.  First and last rows, rows of second
    tiles and the ragged last rows against the oracle; everything against one work-group per tile (variants 9, 10)."""
    m, n, slabs = shape
    k = slabs * 128 // np.dtype(O.IN_DTYPE[types]).itemsize
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT
    ha, hb, hc = O.make_inputs(types, m, n, k, kind=kind, seed=81)
    p = G.capi.plan(types, m, n, k, O.ROW, lb, 4, variant)
    print("case", types, variant, shape, lb, p.variant, p.grid, flush=True)
    # (fp32 has the four-wave instance only: variant 6 runs the register-staged kernel, a work-group per tile)
    assert p.grid == (-(-m // 256) * -(-n // 256) if types == O.F32F32F32 and variant == 6 else 256)
    got = G.run_gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, 4, variant)
    for rows in ((0, 4), (1020, 1028), (m // 2 - 2, m // 2 + 2), (m // 256 * 256 - 4, m // 256 * 256 + 4), (m - 4, m)):
        ref = O.gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, rows=rows)
        assert np.array_equal(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]), (types, variant, shape, lb, rows)
    one = G.run_gemm(types, ha, hb, hc, m, n, k, O.ROW, lb, 2, 1, 4, variant + 4)
    assert np.array_equal(got, one)


@pytest.mark.parametrize("types", [O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16, O.F32F32F32, O.E4M3E4M3F16])
@pytest.mark.parametrize("shape", [(4096, 4097, 72), (2048, 8200, 130), (4095, 4160, 255), (4094, 4099, 1023)])
def test_columns_past_a_multiple_of_256_run_as_a_second_launch(G, types, shape):
    """N = 256 q + r with r <= 64 on a grid that the whole tiles just fill: the launcher's choice gives the last r
    columns a launch of their own, which addresses C, D and a row-major B with the pitch of the whole matrices.
    Every layout, alpha and beta at work, whole and ragged K; bit-exact on integer-valued data against the oracle
    (first and last rows, every column)."""
    m, n, k = shape
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT
    split_seen = False
    for la, lb in [(O.ROW, O.COL), (O.ROW, O.ROW), (O.COL, O.ROW), (O.COL, O.COL)]:
        p = G.capi.plan(types, m, n, k, la, lb)
        split_seen |= p.tail_cols > 0
        if p.tail_cols:
            assert p.tail_cols == n % 256 and p.tail_rows == 0
            # up to eight columns as dot products while that is the cheaper way (a short K), otherwise small tiles
            assert (p.tail_tile_m, p.tail_tile_n) in ((((16, p.tail_cols),) if p.tail_cols <= 8 else ()) + ((128, 128),))
            assert p.grid == -(-m // p.tile_m) * ((n - p.tail_cols) // p.tile_n)
        a, b, c = O.make_inputs(types, m, n, k, kind=kind, seed=5 + la + 2 * lb)
        print("case", types, shape, la, lb, p.tail_cols, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 2, -1, -1)
        for rows in ((0, 24), (m - 24, m)):
            ref = O.gemm(types, a, b, c, m, n, k, la, lb, 2, -1, rows=rows)
            assert np.array_equal(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]), (types, shape, la, lb, rows)
    # (the 8-bit floats keep a strip of more than eight columns in the one launch: on their four-wave register-staged
    # kernel the estimate prefers small tiles for everything)
    assert split_seen or (types in O.FP8_TYPES and n % 256 > 8)


@pytest.mark.parametrize("types", [O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16, O.F32F32F32, O.E4M3E4M3F16])
@pytest.mark.parametrize("shape", [(4096, 4104, 512), (2048, 8200, 256), (4000, 4160, 384)])
def test_column_major_pair_cuts_columns_before_the_transposed_launch(G, types, shape):
    """Column-major A and B with a few columns past a multiple of 256 and whole K slabs: the columns up to the
    multiple run as the transposed problem on the ring kernel, the rest as dot products or small tiles of the problem
    as given.  First and last rows, every column (the seam included), alpha and beta at work, against the oracle."""
    m, n, k = shape
    p = G.capi.plan(types, m, n, k, O.COL, O.COL)
    assert p.variant in (5, 6) and (p.tile_m, p.tile_n) == (256, 256) and p.tail_cols == n % 256 and p.tail_rows == 0
    assert p.grid == -(-m // 256) * (n // 256) and p.tail_grid > 0
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT
    a, b, c = O.make_inputs(types, m, n, k, kind=kind, seed=11)
    got = G.run_gemm(types, a, b, c, m, n, k, O.COL, O.COL, 2, -1, -1)
    for rows in ((0, 24), (m // 2 - 8, m // 2 + 8), (m - 24, m)):
        ref = O.gemm(types, a, b, c, m, n, k, O.COL, O.COL, 2, -1, rows=rows)
        assert np.array_equal(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]), (types, shape, rows)


def test_ragged_baseline_shape_is_split_by_columns(G):
    p = G.capi.plan(O.F16F16F16, 4095, 4097, 1023, O.ROW, O.ROW)
    assert (p.tile_m, p.tile_n, p.grid, p.tail_cols, p.tail_tile_m, p.tail_grid) == (256, 256, 256, 1, 16, 256)
    assert G.capi.plan(O.F16F16F16, 4096, 4096, 1024, O.ROW, O.ROW).tail_cols == 0
    assert G.capi.plan(O.F16F16F16, 4096, 4096 + 100, 1024, O.ROW, O.ROW).tail_cols == 0


def random_big_problems(capi, types, want_cut=5, want_plain=2):
    """Seeded draws of big problems with a short K; kept: the first `want_cut` that the launcher cuts in two launches
    (rows or columns) and the first `want_plain` that it does not."""
    rng = np.random.default_rng(77 + types)
    es = np.dtype(O.IN_DTYPE[types]).itemsize
    cut, plain = [], []
    for _ in range(400):
        m = int(rng.integers(2500, 7500))
        n = 256 * int(rng.integers(10, 30)) + int(rng.choice([0, 0, 1, 3, 8, 9, 40, 64, 65, 130]))
        k = (128 // es) * int(rng.integers(1, 3)) if rng.integers(0, 3) else int(rng.integers(24, 200))
        la = O.ROW if rng.integers(0, 4) else O.COL
        lb = int(rng.integers(0, 2))
        al, be = int(rng.integers(1, 3)), int(rng.integers(-1, 2))
        p = capi.plan(types, m, n, k, la, lb)
        case = (m, n, k, la, lb, al, be, p.tail_rows, p.tail_cols)
        if p.tail_rows or p.tail_cols:
            if len(cut) < want_cut:
                cut.append(case)
        elif len(plain) < want_plain:
            plain.append(case)
        if len(cut) == want_cut and len(plain) == want_plain:
            break
    return cut, plain


@pytest.mark.parametrize("types", [O.S8S8S32, O.BF16BF16F32, O.F16F16F16])
def test_launcher_choice_on_random_big_grids(G, types):
    """Seeded random problems large enough for the launcher to cut them (a mostly empty last round of tiles: the
    last rows in a second launch; a few columns past a multiple of 256: those columns in a second launch, as tiles
    or as dot products), with a short K so that the oracle can follow: any layout, alpha and beta at work,
    bit-exact on integer-valued data in the first and last rows and in a band around the cut."""
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT
    cut, plain = random_big_problems(G.capi, types)
    assert len(cut) >= 3, "the draw must exercise the cuts"
    for m, n, k, la, lb, al, be, tail_rows, tail_cols in cut + plain:
        a, b, c = O.make_inputs(types, m, n, k, kind=kind, seed=m + 3 * n + 5 * k)
        print("case", types, m, n, k, la, lb, al, be, "tail_rows", tail_rows, "tail_cols", tail_cols, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, al, be, -1)
        edge = m - tail_rows if tail_rows else m // 2
        for rows in ((0, 16), (max(edge - 8, 0), min(edge + 8, m)), (m - 16, m)):
            ref = O.gemm(types, a, b, c, m, n, k, la, lb, al, be, rows=rows)
            assert np.array_equal(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]), (types, m, n, k, la, lb, rows)
