"""GPU parity of every rung, type bundle and layout against the CPU oracle, through the C ABI."""
import itertools

import numpy as np
import pytest
import torch

import oracle_lib as O

pytestmark = pytest.mark.gpu

LAYOUTS = list(itertools.product((O.ROW, O.COL), repeat=2))
ALL_TYPES = (O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16, O.F32F32F32, O.E4M3E4M3F16, O.E5M2E5M2F16)
SKINNY_TYPES = (O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16)
VALU_RUNGS = (0, 1, 2, 3)
MFMA = 4
SKINNY = 5
# ragged, tiny, tile-multiple and "one past a tile" shapes
SHAPES = [(1, 1, 1), (3, 5, 7), (64, 64, 64), (65, 63, 33), (100, 130, 70), (256, 256, 128), (257, 129, 200),
          (31, 300, 1023)]


def exact_kind(types):
    return O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


@pytest.mark.parametrize("types", ALL_TYPES)
@pytest.mark.parametrize("rung", VALU_RUNGS + (MFMA,))
def test_bit_exact_all_layouts_and_shapes(G, types, rung):
    """int8 full range / integer-valued floats: any summation order must give the oracle's bits."""
    for (la, lb), (m, n, k), (al, be) in itertools.product(LAYOUTS, SHAPES, [(1, 0), (2, -1)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=m + 3 * n + 7 * k)
        print("case", types, rung, la, lb, m, n, k, al, be, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, al, be, rung)
        ref = O.gemm(types, a, b, c, m, n, k, la, lb, al, be)
        assert np.array_equal(got, ref), (types, rung, la, lb, m, n, k, al, be)


@pytest.mark.parametrize("types", ALL_TYPES[1:])
@pytest.mark.parametrize("rung", VALU_RUNGS)
def test_valu_rungs_sum_in_k_order(G, types, rung):
    """Rungs 0-3 add each output's products in k order (fp32 inputs: fused into the sum), so even N(0,1) data
    matches the oracle bit for bit."""
    for (la, lb), (m, n, k) in itertools.product(LAYOUTS, [(65, 63, 129), (128, 192, 257)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=11)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 1.0, 0.5, rung)
        ref = O.gemm(types, a, b, c, m, n, k, la, lb, 1.0, 0.5)
        assert np.array_equal(got, ref), (types, rung, la, lb, m, n, k)


@pytest.mark.parametrize("types", ALL_TYPES[1:])
def test_mfma_within_tolerance_on_normal_data(G, types):
    """Blocked fp32 accumulation differs from the sequential sum only by rounding: <= 1e-3 (fp32 out) / 1e-2 (16-bit out)."""
    for (la, lb), (m, n, k), variant in itertools.product(LAYOUTS, [(256, 256, 512), (300, 200, 1000)], (0, 1, 2)):
        kind = O.FILL_UNIFORM_PM1 if types == O.F16F16F16 else O.FILL_NORMAL
        a, b, c = O.make_inputs(types, m, n, k, kind=kind, seed=21)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 1.0, 1.0, MFMA, variant)
        truth, _ = O.gemm_f64(types, a, b, c, m, n, k, la, lb, 1.0, 1.0)
        G.assert_within(types, got, truth, f"mfma vs fp64 truth {types} {la}{lb} {m}x{n}x{k} v{variant}")
        ref = O.out_to_f64(types, O.gemm(types, a, b, c, m, n, k, la, lb, 1.0, 1.0))
        G.assert_within(types, got, ref, "mfma vs sequential fp32 oracle")


@pytest.mark.parametrize("types", ALL_TYPES)
def test_mfma_every_variant_bit_exact(G, types):
    nvar = G.capi.variant_count(types, G.capi.RUNG_MFMA)
    assert nvar >= 3
    for variant, (la, lb), (m, n, k) in itertools.product(range(1, nvar + 1), [(0, 1), (0, 0), (1, 0)],
                                                          [(512, 512, 256), (300, 520, 130)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=variant)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, la, lb, 1, 1)), (types, variant, la, lb, m, n, k)


@pytest.mark.parametrize("types", ALL_TYPES)
def test_edge_tiles_of_the_register_staged_kernel(G, types):
    """Tiles that reach past M or N, several K slabs deep, on every tile configuration of the register-staged
    kernel: lines past the matrix are read from the last line and 16-byte pieces past a line's end as they lie in
    memory, so only what is computed for rows and columns inside the matrix may reach D.  K a whole number of slabs
    and not; M / N below, at and just past a 16-byte piece; operands at odd addresses."""
    shapes = [(300, 20, 700), (20, 300, 700), (270, 15, 256), (15, 270, 256), (258, 258, 385), (129, 1, 640),
              (1, 129, 640), (17, 16, 128)]
    for variant, (la, lb), (m, n, k) in itertools.product((1, 2, 3, 4), LAYOUTS, shapes):
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=variant + m)
        print("case", types, variant, la, lb, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 1, 1, MFMA, variant, misalign=(m + n) % 3)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, la, lb, 1, 1)), (types, variant, la, lb, m, n, k)


@pytest.mark.parametrize("types", (O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16, O.E4M3E4M3F16, O.E5M2E5M2F16,
                                   O.F32F32F32))
def test_whole_line_pipeline_every_slab_count(G, types):
    """Whole 256x256 tiles, row-major A, column-major B, K = 1..12 slabs of 128 bytes: the kernel whose ring of five
    buffers is filled by whole-line copies (variants 5 and 6; 9 and 10 launch one work-group per tile), through a full
    turn of the ring and past it."""
    slab = 128 // np.dtype(O.IN_DTYPE[types]).itemsize
    # (variant 11: the same kernel on 128 x 128 tiles; the 8-bit floats have no such instance and run the tile's
    # register-staged kernel; fp32 has the four-wave 256 x 256 instances only - v_mfma_f32_16x16x4_f32, four per block)
    for variant, slabs, (m, n) in itertools.product((5, 6, 9, 10, 11), (1, 2, 3, 4, 5, 6, 7, 9, 10, 11, 12), [(256, 512), (512, 256)]):
        k = slab * slabs
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs)
        print("case", types, variant, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)), (types, variant, m, n, k)
    # ragged M and N with whole slabs (rows clamped at the edges)
    for variant, slabs, (m, n) in itertools.product((5, 6), (1, 4, 7), [(300, 520), (257, 255), (511, 1)]):
        k = slab * slabs
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs + 50)
        print("ragged case", types, variant, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)), (types, variant, m, n, k)
    # a row-major B: whole K rows per copy, transposing LDS reads; whole tiles, and ragged M and N with rows of whole
    # 16-byte pieces
    for variant, slabs, (m, n) in itertools.product((5, 6, 11), (1, 2, 5, 6, 11), [(256, 512), (512, 256), (128, 384)]):
        k = slab * slabs
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs + 90)
        print("row/row case", types, variant, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.ROW, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.ROW, 1, 1)), (types, variant, m, n, k)
    for variant, slabs, (m, n) in itertools.product((5, 6), (1, 4, 7), [(300, 528), (257, 240), (511, 16)]):
        k = slab * slabs
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs + 70)
        print("ragged row/row case", types, variant, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.ROW, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.ROW, 1, 1)), (types, variant, m, n, k)


@pytest.mark.parametrize("types", (O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16, O.E4M3E4M3F16, O.E5M2E5M2F16,
                                   O.F32F32F32))
def test_whole_line_pipeline_on_the_transposed_problem(G, types):
    """Column-major A and B: the same kernel runs D^T = B^T A^T (a row-major pair of operands) and writes the
    row-major D.  Whole tiles on every variant of that kernel, the launcher's own choice, M and N ragged (M in whole
    16-byte pieces), alpha and beta at work; shapes the kernel cannot take (M = 300) run the kernels of the problem
    as given.  Bit-exact."""
    slab = 128 // np.dtype(O.IN_DTYPE[types]).itemsize
    for variant, slabs, (m, n) in itertools.product((0, 5, 6, 9, 10, 11), (1, 2, 5, 6, 11), [(256, 512), (512, 256), (128, 384)]):
        k = slab * slabs
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs + 30)
        print("col/col case", types, variant, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.COL, O.COL, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.COL, O.COL, 1, 1)), (types, variant, m, n, k)
    for variant, slabs, (m, n) in itertools.product((0, 5, 6), (1, 4, 7), [(528, 300), (240, 257), (16, 511), (300, 528)]):
        k = slab * slabs
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs + 10)
        print("ragged col/col case", types, variant, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.COL, O.COL, 2, -1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.COL, O.COL, 2, -1)), (types, variant, m, n, k)
    # sub-matrix views: leading dimensions of whole 16-byte pieces stay on this path, odd ones leave it
    piece_in = 16 // np.dtype(O.IN_DTYPE[types]).itemsize
    piece_out = 16 // np.dtype(O.OUT_DTYPE[types]).itemsize
    for variant, (m, n), pads in itertools.product((5, 6, 11), [(512, 256), (528, 300)],
                                                   [(2 * piece_in, piece_in, piece_out, 2 * piece_out), (piece_in, piece_in, 1, 1),
                                                    (1, 3, piece_out, piece_out)]):
        k = 3 * slab
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=variant + 3)
        print("col/col ld case", types, variant, m, n, k, pads, flush=True)
        got = G.run_gemm_ld(types, a, b, c, m, n, k, O.COL, O.COL, 1, 1, MFMA, variant, pads)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.COL, O.COL, 1, 1)), (types, variant, m, n, k, pads)


@pytest.mark.parametrize("types", (O.S8S8S32, O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16, O.E4M3E4M3F16))
def test_whole_line_pipeline_column_major_a_with_row_major_b(G, types):
    """Neither operand K-contiguous: both go into LDS as whole K rows and come out through the transposing reads
    (int8 and the 16-bit types; the 8-bit floats run the register-staged kernel on the same calls).  Whole tiles on
    every variant of the kernel and the launcher's own choice, M and N ragged in whole 16-byte pieces, shapes it
    cannot take (M = 300), sub-matrix views.  Bit-exact."""
    slab = 128 // np.dtype(O.IN_DTYPE[types]).itemsize
    for variant, slabs, (m, n) in itertools.product((0, 5, 6, 9, 10, 11), (1, 2, 5, 6, 11), [(256, 512), (512, 256), (128, 384)]):
        k = slab * slabs
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs + 40)
        print("col/row case", types, variant, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.COL, O.ROW, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.COL, O.ROW, 1, 1)), (types, variant, m, n, k)
    for variant, slabs, (m, n) in itertools.product((0, 5, 6), (1, 4, 7), [(528, 304), (240, 272), (16, 512), (300, 528)]):
        k = slab * slabs
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=slabs + 20)
        print("ragged col/row case", types, variant, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.COL, O.ROW, 2, -1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.COL, O.ROW, 2, -1)), (types, variant, m, n, k)
    piece_in = 16 // np.dtype(O.IN_DTYPE[types]).itemsize
    piece_out = 16 // np.dtype(O.OUT_DTYPE[types]).itemsize
    for variant, (m, n), pads in itertools.product((5, 6, 11), [(512, 256), (528, 304)],
                                                   [(2 * piece_in, piece_in, piece_out, 2 * piece_out), (piece_in, piece_in, 1, 1),
                                                    (1, 3, piece_out, piece_out)]):
        k = 3 * slab
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=variant + 5)
        print("col/row ld case", types, variant, m, n, k, pads, flush=True)
        got = G.run_gemm_ld(types, a, b, c, m, n, k, O.COL, O.ROW, 1, 1, MFMA, variant, pads)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.COL, O.ROW, 1, 1)), (types, variant, m, n, k, pads)


@pytest.mark.parametrize("types", (O.E4M3E4M3F16, O.E5M2E5M2F16))
def test_whole_line_pipeline_8bit_floats_on_normal_data(G, types):
    """The 16x16x128 kernel (variants 5 and 6) on N(0,1) data, where every bit of the operands matters: a long K
    on whole and ragged grids, both layouts of B, against the fp64 truth within the type's tolerance."""
    for variant, lb, (m, n, k) in itertools.product((5, 6), (O.COL, O.ROW), [(512, 256, 2048), (300, 528, 1152)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=variant + lb)
        print("case", types, variant, lb, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, lb, 1.0, 1.0, MFMA, variant)
        truth, _ = O.gemm_f64(types, a, b, c, m, n, k, O.ROW, lb, 1.0, 1.0)
        G.assert_within(types, got, truth, f"16x16x128 vs fp64 truth {types} {lb} {m}x{n}x{k} v{variant}")


@pytest.mark.parametrize("types", ALL_TYPES)
def test_a_few_columns_past_a_tile_multiple(G, types):
    """N one, seven or thirty-two columns past a multiple of the tile width (the last tile column is almost empty),
    and N below 32 altogether: every variant, every layout, whole and ragged M and K; bit-exact on integer-valued
    data, within tolerance on N(0,1) data."""
    nvar = G.capi.variant_count(types, G.capi.RUNG_MFMA)
    shapes = [(256, 257, 128), (300, 288, 200), (512, 513, 1024), (130, 160, 95), (257, 7, 333), (64, 32, 64)]
    for variant, (la, lb), (m, n, k) in itertools.product(range(0, nvar + 1), LAYOUTS, shapes):
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=variant + n)
        print("case", types, variant, la, lb, m, n, k, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 1, 1, MFMA, variant)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, la, lb, 1, 1)), (types, variant, la, lb, m, n, k)
    if types == O.S8S8S32:
        return
    for (la, lb), (m, n, k) in itertools.product(LAYOUTS, [(512, 513, 1024), (300, 288, 1000)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=23)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 1.0, 0.5, MFMA)
        truth, _ = O.gemm_f64(types, a, b, c, m, n, k, la, lb, 1.0, 0.5)
        G.assert_within(types, got, truth, f"types {types} layouts {la}{lb} {m}x{n}x{k}")


@pytest.mark.parametrize("types", SKINNY_TYPES)
def test_skinny_rung(G, types):
    # three kernels: M <= 16 with K % 128 == 0 (direct-to-LDS), M <= 16 otherwise (registers), 16 < M <= 128 (tile)
    for (m, n, k), (al, be) in itertools.product([(1, 16, 64), (1, 1000, 256), (8, 14336, 512), (16, 250, 128),
                                                  (13, 37, 384), (17, 33, 192), (32, 512, 4096), (33, 100, 64),
                                                  (64, 3000, 1024), (100, 9, 128), (128, 7170, 576)],
                                                 [(1, 0), (0.5, 2)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=5)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, al, be, SKINNY)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, al, be)), (types, m, n, k)
        # decode-like data: activations N(0,1), weights N(0, 0.02)
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=6, scale_b=0.02)
        got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 0, G.capi.RUNG_AUTO)  # AUTO picks the same kernel
        assert G.capi.plan(types, m, n, k, O.ROW, O.COL).rung == SKINNY
        truth, _ = O.gemm_f64(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 0)
        G.assert_within(types, got, truth, f"skinny {types} {m}x{n}x{k}")


@pytest.mark.parametrize("types", SKINNY_TYPES)
def test_skinny_rung_long_k_wide_column_blocks(G, types):
    """65 ... 128 rows with K >= 8192: column blocks of 128 ... 256 columns, K split in two or four parts, partial sums
    through the workspace and a second launch that adds them in order.  Column counts that fill, nearly fill and
    barely touch the blocks, K parts of unequal length, alpha / beta, sub-matrix views; M = 64 and K = 4096 beside
    them stay on the one-launch kernel.  Integer-valued data: every partial sum is exact, so bit-exact."""
    cases = [(128, 14336, 8192), (100, 8192 + 4, 8192), (65, 12000, 8192 + 64), (128, 4100, 14336), (127, 28672, 8192),
             (64, 14336, 8192), (128, 14336, 4096)]
    for (m, n, k), (al, be) in itertools.product(cases, [(1, 0), (0.5, 2)]):
        plan = G.capi.plan(types, m, n, k, O.ROW, O.COL, SKINNY)
        assert (plan.split_k > 1) == (m > 64 and k >= 8192), (m, n, k, plan.split_k)
        assert (plan.workspace_bytes > 0) == (plan.split_k > 1)
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=m + 1)
        print("case", types, m, n, k, al, be, plan.split_k, plan.tile_n, flush=True)
        ref = O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, al, be)
        for rung in (SKINNY, -1):
            got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, al, be, rung)
            assert np.array_equal(got, ref), (types, m, n, k, al, be, rung)
    m, n, k = 96, 9000, 8192
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=3)
    ref = O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)
    for pads in [(8, 16, 4, 8), (16, 8, 1, 3)]:
        assert np.array_equal(G.run_gemm_ld(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, SKINNY, 0, pads), ref), pads
    # N(0,1) activations against weights of N(0, 0.02): within the type's tolerance of the fp64 truth
    m, n, k = 128, 14336, 8192
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_NORMAL, seed=9, scale_b=0.02)
    got = G.run_gemm(types, a, b, None, m, n, k, O.ROW, O.COL, 1, 0, -1)
    truth, _ = O.gemm_f64(types, a, b, None, m, n, k, O.ROW, O.COL, 1, 0)
    G.assert_within(types, got, truth, f"skinny long K {types}")


def test_skinny_rung_refuses_what_it_cannot_do(G):
    a = torch.zeros(129 * 64, dtype=torch.int16, device="cuda")
    for kw in (dict(m=129), dict(lb=O.ROW), dict(k=96), dict(types=O.S8S8S32), dict(types=O.F32F32F32),
               dict(types=O.E4M3E4M3F16)):
        args = dict(types=O.BF16BF16BF16, m=8, n=64, k=64, la=O.ROW, lb=O.COL)
        args.update(kw)
        with pytest.raises(G.capi.GzError) as e:
            G.capi.gemm(args["types"], a, a, None, a, args["m"], args["n"], args["k"], args["la"], args["lb"], 1, 0, SKINNY)
        assert e.value.status == G.capi.ERR_UNSUPPORTED


@pytest.mark.parametrize("types", ALL_TYPES)
@pytest.mark.parametrize("rung", VALU_RUNGS + (MFMA,))
def test_degenerate_and_unaligned(G, types, rung):
    # K = 0: D = beta * C
    m, n = 5, 9
    a, b, c = O.make_inputs(types, m, n, 4, kind=exact_kind(types), seed=2)
    got = G.run_gemm(types, a, b, c, m, n, 0, O.ROW, O.COL, 3, 2, rung)
    assert np.array_equal(got, O.gemm(types, a, b, c, m, n, 0, O.ROW, O.COL, 3, 2))
    # operands that start 1 element (not 16 bytes) into an allocation, tile-multiple shape
    m, n, k = 256, 256, 256
    a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=3)
    for la, lb in LAYOUTS:
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, 1, 1, rung, misalign=1)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, la, lb, 1, 1)), (types, rung, la, lb)
    # D alone off by one element (operands aligned): the element-wise epilogue of the MFMA rung
    got = G.run_gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, rung, guard=65)
    assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)), (types, rung, "D + 1 element")


@pytest.mark.parametrize("types", ALL_TYPES)
def test_beta_zero_never_reads_c(G, types):
    m, n, k = 130, 70, 96
    a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=4)
    ref = O.gemm(types, a, b, None, m, n, k, O.ROW, O.COL, 1, 0)
    poison = np.full(m * n, 0xFF, np.uint8).repeat(c.dtype.itemsize).view(c.dtype)  # NaN pattern for floats, -1 for int32
    for rung in VALU_RUNGS + (MFMA,):
        assert np.array_equal(G.run_gemm(types, a, b, None, m, n, k, O.ROW, O.COL, 1, 0, rung), ref)
        assert np.array_equal(G.run_gemm(types, a, b, poison, m, n, k, O.ROW, O.COL, 1, 0, rung), ref)


def test_int32_epilogue_wraps(G):
    m = n = 64; k = 256
    a = np.full(m * k, 127, np.int8); b = np.full(k * n, 127, np.int8); c = np.full(m * n, 2 ** 31 - 1, np.int32)
    ref = O.gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.COL, 70000, 3)
    for rung in VALU_RUNGS + (MFMA,):
        assert np.array_equal(G.run_gemm(O.S8S8S32, a, b, c, m, n, k, O.ROW, O.COL, 70000, 3, rung), ref)


def test_16bit_epilogue_rounding_order(G):
    """The hand-built cases that pin the oracle's rounding order, on every rung."""
    bf = lambda v: (np.asarray(v, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    k = 257
    a = bf([1.0] * k); b = bf([1.0] * k)
    for rung in VALU_RUNGS + (MFMA,):
        d = G.run_gemm(O.BF16BF16BF16, a, b, None, 1, 1, k, O.ROW, O.COL, 1.5, 0.0, rung)
        assert O.bf16_to_f32(d)[0, 0] == 384.0
        d = G.run_gemm(O.BF16BF16BF16, bf([0.0]), bf([0.0]), bf([1.0078125]), 1, 1, 1, O.ROW, O.COL, 1.0, 1.0078125, rung)
        assert O.bf16_to_f32(d)[0, 0] == 1.015625


@pytest.mark.parametrize("types", ALL_TYPES)
def test_launcher_choice_on_random_problems(G, types):
    """GZ_RUNG_AUTO on seeded random shapes, layouts and scalars (integer-valued data: bit-exact): whatever kernel
    the launcher picks - streaming, direct-to-LDS, ragged, predicated - must give the oracle's bits."""
    rng = np.random.default_rng(1000 + types)
    es = np.dtype(O.IN_DTYPE[types]).itemsize
    cases = []
    for _ in range(14):
        m, n, k = (int(rng.integers(1, 700)) for _ in range(3))
        cases.append((m, n, k))
    for _ in range(8):   # whole 16-byte rows and K slabs: the direct-to-LDS kernels, ragged or not
        m, n = int(rng.integers(1, 5)) * 128 + int(rng.integers(0, 2)) * int(rng.integers(1, 128)), \
            int(rng.integers(1, 5)) * 128 + int(rng.integers(0, 2)) * (16 // es) * int(rng.integers(1, 8))
        cases.append((m, n, (128 // es) * int(rng.integers(1, 9))))
    for _ in range(4):   # decode shapes
        cases.append((int(rng.integers(1, 129)), int(rng.integers(1, 40)) * 16, 64 * int(rng.integers(1, 12))))
    for m, n, k in cases:
        la, lb = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        al, be = int(rng.integers(-2, 3)), int(rng.integers(-1, 2))
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=m * 7 + n * 3 + k)
        print("case", types, m, n, k, la, lb, al, be, flush=True)
        got = G.run_gemm(types, a, b, c, m, n, k, la, lb, al, be, G.capi.RUNG_AUTO)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, la, lb, al, be)), (types, m, n, k, la, lb, al, be)


@pytest.mark.parametrize("types", [O.BF16BF16F32, O.BF16BF16BF16, O.F16F16F16, O.F32F32F32, O.E4M3E4M3F16])
def test_sign_of_zero_survives_the_epilogue(G, types):
    """alpha = 0 on negative sums and alpha < 0 on zero sums give -0 in IEEE arithmetic; a multiply fused with the
    conversion to fp16 (fma with a +0 addend) would lose it."""
    m, n, k = 64, 48, 40
    a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=5)
    for (al, be), rung in itertools.product([(0, 0), (-2, 0), (0, 1), (-1, -1)], VALU_RUNGS + (MFMA,)):
        ref = O.gemm(types, a, b, c, m, n, k, O.COL, O.ROW, al, be)
        got = G.run_gemm(types, a, b, c, m, n, k, O.COL, O.ROW, al, be, rung)
        assert np.array_equal(got, ref), (types, al, be, rung)
    # an all-zero product with a negative alpha
    z = np.zeros_like(a)
    ref = O.gemm(types, z, b, c, m, n, k, O.ROW, O.COL, -1, 0)
    assert (ref.view(np.uint8).reshape(m * n, -1)[:, -1] == 0x80).all()
    for rung in VALU_RUNGS + (MFMA,):
        assert np.array_equal(G.run_gemm(types, z, b, c, m, n, k, O.ROW, O.COL, -1, 0, rung), ref), (types, rung)


def ld_pads(types):
    """Leading-dimension paddings in elements: whole 16-byte pieces on every operand (the direct-to-LDS kernels keep
    working), odd ones (every kernel that needs aligned lines has to step aside), and a mix."""
    piece_in = 16 // np.dtype(O.IN_DTYPE[types]).itemsize
    piece_out = 16 // np.dtype(O.OUT_DTYPE[types]).itemsize
    return [(piece_in, 2 * piece_in, piece_out, 3 * piece_out), (3, 1, 5, 7), (piece_in, 0, 1, piece_out)]


@pytest.mark.parametrize("types", ALL_TYPES)
@pytest.mark.parametrize("rung", (-1,) + VALU_RUNGS + (MFMA,))
def test_leading_dimensions_every_rung(G, types, rung):
    """gz_gemm_ld on sub-matrix views (nvidia/kernels/generic_gemm.cuh:6-8 takes lda, ldb, ldc, ldd): A, B, C and D
    each inside a wider allocation, paddings aligned and not, every layout pair; bit-exact against the oracle on the
    packed copies of the same sub-matrices, the paddings of D untouched."""
    shapes = [(65, 63, 33), (256, 256, 256), (300, 200, 128)]
    for (la, lb), (m, n, k), pads in itertools.product(LAYOUTS, shapes, ld_pads(types)):
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=m + n + k + pads[0])
        print("case", types, rung, la, lb, m, n, k, pads, flush=True)
        got = G.run_gemm_ld(types, a, b, c, m, n, k, la, lb, 2, -1, rung, 0, pads)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, la, lb, 2, -1)), (types, rung, la, lb, m, n, k, pads)


@pytest.mark.parametrize("types", (O.S8S8S32, O.BF16BF16F32, O.F16F16F16, O.E4M3E4M3F16))
def test_leading_dimensions_on_the_direct_kernels(G, types):
    """Whole 256 x 256 tiles with leading dimensions of whole 16-byte pieces stay on the ring kernel (variants 5, 6:
    both layouts of B, stream-K with variant 7) and on the compiler-scheduled direct-to-LDS kernels (variants 2, 3);
    ragged M and N with them on the ring kernel's ragged instance; odd paddings send the same calls to the
    register-staged kernel.  Bit-exact either way."""
    slab = 128 // np.dtype(O.IN_DTYPE[types]).itemsize
    piece_in = 16 // np.dtype(O.IN_DTYPE[types]).itemsize
    piece_out = 16 // np.dtype(O.OUT_DTYPE[types]).itemsize
    cases = [(512, 256, 6 * slab), (300, 520, 3 * slab)]
    pad_sets = [(2 * piece_in, piece_in, piece_out, 2 * piece_out), (piece_in, piece_in, 1, 1), (1, 3, piece_out, piece_out)]
    variants = (2, 3, 5, 6) + ((7,) if types in (O.S8S8S32, O.BF16BF16F32, O.F16F16F16) else ())
    for variant, lb, (m, n, k), pads in itertools.product(variants, (O.COL, O.ROW), cases, pad_sets):
        a, b, c = O.make_inputs(types, m, n, k, kind=exact_kind(types), seed=variant + k)
        print("case", types, variant, lb, m, n, k, pads, flush=True)
        got = G.run_gemm_ld(types, a, b, c, m, n, k, O.ROW, lb, 1, 1, MFMA, variant, pads)
        assert np.array_equal(got, O.gemm(types, a, b, c, m, n, k, O.ROW, lb, 1, 1)), (types, variant, lb, m, n, k, pads)


@pytest.mark.parametrize("types", SKINNY_TYPES)
def test_leading_dimensions_on_the_streaming_rung(G, types):
    """The weight-streaming kernels take leading dimensions of whole 16-byte pieces; others are refused by the rung
    itself and served by the tiled rung under the launcher's choice."""
    for (m, n, k), pads in itertools.product([(1, 520, 256), (8, 512, 192), (24, 300, 512), (100, 448, 1024)],
                                             [(8, 16, 4, 8), (16, 8, 1, 3)]):
        a, b, c = O.make_inputs(types, m, n, k, kind=O.FILL_SMALL_INT, seed=m + n)
        ref = O.gemm(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1)
        for rung in (SKINNY, -1):
            print("case", types, rung, m, n, k, pads, flush=True)
            assert np.array_equal(G.run_gemm_ld(types, a, b, c, m, n, k, O.ROW, O.COL, 1, 1, rung, 0, pads), ref), (m, n, k, pads, rung)
    a, b, c = O.make_inputs(types, 8, 512, 256, kind=O.FILL_SMALL_INT, seed=1)
    with pytest.raises(G.capi.GzError) as e:
        G.run_gemm_ld(types, a, b, c, 8, 512, 256, O.ROW, O.COL, 1, 1, SKINNY, 0, (3, 8, 0, 0))
    assert e.value.status == G.capi.ERR_UNSUPPORTED
    assert np.array_equal(G.run_gemm_ld(types, a, b, c, 8, 512, 256, O.ROW, O.COL, 1, 1, -1, 0, (3, 8, 0, 0)),
                          O.gemm(types, a, b, c, 8, 512, 256, O.ROW, O.COL, 1, 1))
