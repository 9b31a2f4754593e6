"""Host-side checks of the C ABI that need no GPU: the library loads, exports what the header
declares, validates arguments before touching the device, and plans launches sensibly."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "gemm_zoo.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gz_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(capi):
    names = declared_symbols()
    assert len(names) >= 13 and set(names) == set(capi.EXPORTS)
    raw = ctypes.CDLL(str(capi.LIB_PATH))
    for n in names:
        assert hasattr(raw, n), n


def test_version_and_names(capi):
    assert capi.lib.gz_version() >= 1
    assert [capi.rung_name(r) for r in range(capi.NUM_RUNGS)] == [
        "naive", "coalesced", "lds_tiled", "double_buffered", "mfma", "skinny"]
    assert capi.lib.gz_types_name(capi.S8S8S32) == b"s8s8s32"
    assert capi.variant_count(capi.BF16BF16F32, capi.RUNG_MFMA) >= 3
    assert capi.variant_count(capi.S8S8S32, capi.RUNG_SKINNY) == 0
    assert capi.lib.gz_types_name(capi.F32F32F32) == b"f32f32f32"
    assert capi.variant_count(capi.F32F32F32, capi.RUNG_SKINNY) == 0 and capi.variant_count(capi.F32F32F32, capi.RUNG_MFMA) >= 3


@pytest.mark.parametrize("kwargs,status", [
    (dict(types=9), 1), (dict(m=-1), 1), (dict(k=-5), 1), (dict(layout_a=2), 1), (dict(layout_b=-1), 1),
    (dict(rung=6), 1), (dict(rung=-2), 1), (dict(variant=-1), 1),
    (dict(m=1 << 31), 2),                       # an extent of 2^31 (2^40 elements with smaller extents are fine)
    (dict(rung=4, variant=99), 2),
    (dict(rung=0, variant=1), 2),
    (dict(types=0, rung=5), 2),                 # no int8 streaming kernel
    (dict(types=4, rung=5, m=8, layout_b=1), 2),  # no fp32 streaming kernel
    (dict(rung=5, m=129, layout_b=1), 2),       # M too large for the streaming kernels
    (dict(rung=5, m=8, layout_b=0), 2),         # needs column-major weights
    (dict(rung=5, m=8, layout_b=1, k=100), 2),  # K not a whole number of super-steps
])
def test_plan_rejects_bad_requests(capi, kwargs, status):
    args = dict(types=1, m=128, n=128, k=128, layout_a=0, layout_b=0, rung=-1, variant=0)
    args.update(kwargs)
    with pytest.raises(capi.GzError) as e:
        capi.plan(**args)
    assert e.value.status == status and str(e.value)


def test_gemm_entry_points_validate_before_any_device_work(capi):
    """Bad arguments must come back as status codes without a GPU being present."""
    for types in range(4):
        with pytest.raises(capi.GzError) as e:
            capi.gemm(types, 0, 0, 0, 0, 16, 16, 16)  # NULL operands
        assert e.value.status == capi.ERR_BAD_ARG
        with pytest.raises(capi.GzError) as e:
            capi.gemm(types, 64, 64, 0, 64, 16, 16, 16, beta=1)  # beta != 0 needs C
        assert e.value.status == capi.ERR_BAD_ARG and "C is NULL" in str(e.value)
        with pytest.raises(capi.GzError) as e:
            capi.gemm(types, 64, 64, 64, 64, -1, 16, 16)
        assert e.value.status == capi.ERR_BAD_ARG
        with pytest.raises(capi.GzError) as e:
            capi.gemm(types, 64, 64, 64, 64, 16, 16, 16, layout_a=7)
        assert e.value.status == capi.ERR_BAD_ARG
        # empty outputs are a no-op, whatever the pointers
        capi.gemm(types, 0, 0, 0, 0, 0, 16, 16)
        capi.gemm(types, 0, 0, 0, 0, 16, 0, 16)
    st = capi.lib.gz_gemm(0, 64, 64, 64, 64, 4, 4, 4, 0, 0, 1.5, 0.0, -1, 0, None)
    assert st == capi.ERR_BAD_ARG and "integral" in capi.last_error()
    assert capi.lib.gz_gemm(17, 64, 64, 64, 64, 4, 4, 4, 0, 0, 1.0, 0.0, -1, 0, None) == capi.ERR_BAD_ARG
    assert capi.lib.gz_fill(None, 10, 0, 0, 1.0, 1, None) == capi.ERR_BAD_ARG
    assert capi.lib.gz_fill(None, 0, 0, 0, 1.0, 1, None) == capi.OK
    assert capi.lib.gz_fill(64, 10, 9, 0, 1.0, 1, None) == capi.ERR_BAD_ARG
    assert capi.lib.gz_compare(None, None, 10, 0, 0.0, None, None) == capi.ERR_BAD_ARG
    assert capi.lib.gz_compare(None, None, 0, 0, 0.0, None, None) == capi.OK


def test_plan_headline_configs(capi):
    # bf16 4096^3: 256 tiles of 256x256 = one per compute unit
    p = capi.plan(capi.BF16BF16F32, 4096, 4096, 4096, 0, 1)
    assert (p.rung, p.tile_m, p.tile_n, p.tile_k, p.grid) == (capi.RUNG_MFMA, 256, 256, 64, 256)
    assert p.lds_bytes <= 160 * 1024 and p.vector_bytes_a == 16 and p.vector_bytes_b == 16
    # int8 consumes 128 k per slab
    p = capi.plan(capi.S8S8S32, 8192, 8192, 8192, 0, 1)
    assert (p.rung, p.tile_k, p.grid) == (capi.RUNG_MFMA, 128, 256)   # 1024 tiles, one persistent work-group per CU
    # ragged M and N on the same kernel: persistent too (32 x 32 tiles, the last row and column of them clamped), and
    # the wave estimate decides as for whole tiles (a K-contiguous B and a long K: four waves)
    p = capi.plan(capi.S8S8S32, 8000, 8000, 8192, 0, 1)
    assert (p.variant, p.tile_m, p.tile_n, p.threads, p.grid) == (5, 256, 256, 256, 256)
    assert capi.plan(capi.S8S8S32, 8000, 8000, 8192, 0, 1, capi.RUNG_MFMA, 9).grid == 1024   # one work-group per tile
    # ragged fp16 problem: ceil-div grid, only 2-byte aligned lines
    p = capi.plan(capi.F16F16F16, 4095, 4097, 1023, 0, 0)
    # the one column past 4096 runs as a second launch: dot products, one wave per row, sixteen rows per work-group
    assert (p.tail_cols, p.tail_tile_m, p.tail_tile_n, p.tail_grid) == (1, 16, 1, 256)
    assert p.grid == -(-4095 // p.tile_m) * (4096 // p.tile_n)
    assert p.vector_bytes_a == 2 and p.vector_bytes_b == 2
    # decode shapes go to the streaming kernel under AUTO, big M does not
    for m in (1, 8, 32, 128):
        p = capi.plan(capi.BF16BF16BF16, m, 14336, 4096, 0, 1)
        assert p.rung == capi.RUNG_SKINNY and p.grid * p.tile_n >= 14336 and p.tile_m >= m
        # equal column groups: one or two per compute unit, 4-column granular
        assert p.grid % 256 == 0 and p.tile_n % 4 == 0 and p.lds_bytes <= 160 * 1024
    # the LDS-shared tile kernel is chosen only while the tiled rung cannot give every compute unit its own tile
    assert capi.plan(capi.BF16BF16BF16, 128, 65536, 4096, 0, 1).rung == capi.RUNG_MFMA
    assert capi.plan(capi.BF16BF16BF16, 32, 65536, 4096, 0, 1).rung == capi.RUNG_SKINNY
    assert capi.plan(capi.BF16BF16BF16, 129, 14336, 4096, 0, 1).rung == capi.RUNG_MFMA
    # K that is a multiple of 64 but not of 128 takes the register-streaming kernel for M <= 16
    assert capi.plan(capi.BF16BF16BF16, 8, 4096, 192, 0, 1).tile_k == 64
    assert capi.plan(capi.BF16BF16BF16, 8, 4096, 256, 0, 1).tile_k == 128
    assert capi.plan(capi.BF16BF16BF16, 24, 4096, 192, 0, 1).tile_k == 64
    # a small problem shrinks the tile so that more work-groups exist
    small = capi.plan(capi.BF16BF16F32, 1024, 1024, 1024, 0, 1)
    assert small.tile_m * small.tile_n < 256 * 256
    # an explicit variant is honoured; a device with little LDS refuses the big tile
    assert capi.plan(capi.BF16BF16F32, 1024, 1024, 1024, 0, 1, capi.RUNG_MFMA, 1).tile_m == 256
    with pytest.raises(capi.GzError) as e:
        capi.plan(capi.BF16BF16F32, 4096, 4096, 4096, 0, 1, capi.RUNG_MFMA, 1, num_cus=256, lds_per_cu=64 * 1024)
    assert e.value.status == capi.ERR_UNSUPPORTED


def test_plan_split_launch_and_offset_limits(capi):
    # 272 tiles of 256x256 on 256 compute units, row-major B (no stream-K): whole rounds first, the remaining rows
    # as a second launch
    p = capi.plan(capi.BF16BF16F32, 4352, 4096, 4096, 0, 0)
    assert (p.tile_m, p.tile_n, p.grid) == (256, 256, 256) and p.tail_rows == 256 and p.tail_grid > 0
    # column-major A and B: the same cut on the transposed problem, i.e. over columns of the real one
    p = capi.plan(capi.BF16BF16F32, 4096, 4352, 4096, 1, 1)
    assert (p.tile_m, p.tile_n, p.grid) == (256, 256, 256) and p.tail_rows == 0 and p.tail_cols == 256 and p.tail_grid > 0
    # 324 tiles: 68 remain, which the persistent launch carries better than a second launch
    p = capi.plan(capi.BF16BF16F32, 4608, 4608, 4608, 0, 0)
    assert p.tail_rows == 0 and p.grid == 256
    assert capi.plan(capi.BF16BF16F32, 4352, 4096, 4096, 0, 0, capi.RUNG_MFMA, 6).tail_rows == 0
    assert capi.plan(capi.BF16BF16F32, 4096, 4096, 4096, 0, 1).tail_rows == 0      # exactly one round
    # the streaming kernels address rows with 32-bit byte offsets: a K of 20 million goes to the tiled rung
    assert capi.plan(capi.BF16BF16BF16, 64, 64, 20_000_000, 0, 1).rung == capi.RUNG_MFMA
    assert capi.plan(capi.BF16BF16BF16, 64, 64, 8_000_000, 0, 1).rung == capi.RUNG_SKINNY


def test_plan_every_rung_and_type(capi):
    for types in range(capi.NUM_TYPES):
        for rung in range(5):
            p = capi.plan(types, 300, 500, 700, 0, 0, rung)
            assert p.rung == rung and p.grid >= 1 and p.threads in (128, 256, 512, 1024)
            assert p.grid * p.tile_m * p.tile_n >= 300 * 500


def test_plan_streamk(capi):
    """Host-only planning of the stream-K decomposition (nothing is launched)."""
    MF = capi.RUNG_MFMA
    # 272 tiles on 256 compute units: a whole round, and 16 tiles whose slabs are dealt to further work-groups
    # (from a long K on: at K = 4096 the remaining rows as a launch of 64 x 64 tiles cost the same or less)
    p = capi.plan(capi.BF16BF16F32, 4352, 4096, 8192, 0, 1)
    assert p.variant in (7, 8) and p.streamk_tiles == 16 and p.streamk_blocks % 8 == 0 and p.streamk_blocks > 16
    assert p.grid == 256 + p.streamk_blocks and p.tail_rows == 0 and p.tail_cols == 0
    assert p.workspace_bytes == (p.streamk_blocks + 16 - 1) * 256 * 256 * 4
    # a small grid and a long K: every tile is cut
    p = capi.plan(capi.BF16BF16F32, 1024, 1024, 16384, 0, 1)
    assert p.streamk_tiles == 16 and p.grid == p.streamk_blocks == 256
    # exactly one round, most of a round left over, a short K: plain launches
    for m, n, k in [(4096, 4096, 4096), (5120, 5120, 5120), (5120, 5120, 1024), (512, 512, 512)]:
        assert capi.plan(capi.BF16BF16F32, m, n, k, 0, 1).streamk_tiles == 0
    # an explicit stream-K variant is taken wherever it can run and is a plain variant elsewhere
    p = capi.plan(capi.S8S8S32, 5120, 5120, 5120, 0, 1, MF, 7)
    assert p.variant == 7 and p.streamk_tiles == 144 and p.streamk_blocks == 256 and p.threads == 256
    assert capi.plan(capi.F16F16F16, 5120, 5120, 5120, 0, 1, MF, 8).threads == 512
    # (a row-major B as well: its copies carry whole K rows, and a run starts at a K row of its own)
    assert capi.plan(capi.BF16BF16F32, 5120, 5120, 5120, 0, 0, MF, 7).streamk_tiles == 144
    for args in [(capi.BF16BF16F32, 5120, 5120, 5120, 1, 0), (capi.BF16BF16F32, 5120, 5120, 5120, 1, 1),
                 (capi.F32F32F32, 5120, 5120, 5120, 0, 1), (capi.E4M3E4M3F16, 5120, 5120, 5120, 0, 1),
                 (capi.BF16BF16F32, 5120, 5120, 5100, 0, 1), (capi.BF16BF16F32, 256, 256, 64, 0, 1)]:
        p = capi.plan(*args, MF, 7)
        assert p.streamk_tiles == 0 and p.workspace_bytes == 0 and (p.tile_m, p.tile_n) == (256, 256)
    # fewer compute units, fewer work-groups
    p = capi.plan(capi.BF16BF16F32, 1024, 1024, 16384, 0, 1, MF, 0, 64)
    assert p.streamk_blocks <= 64


def test_column_cut_weighs_k(capi):
    """A few columns past a multiple of 256: dot products while K is short, 128 x 128 tiles once K makes them cheaper."""
    p = capi.plan(capi.F16F16F16, 4096, 4097, 1024, 0, 1)
    assert (p.tail_cols, p.tail_tile_m, p.tail_tile_n) == (1, 16, 1)
    # (row-major A and B with rows of B that are not whole 16-byte pieces: no ring kernel, no row cut that pays)
    p = capi.plan(capi.F16F16F16, 4096, 4099, 4096, 0, 0)
    assert (p.tail_cols, p.tail_tile_m, p.tail_tile_n) == (3, 16, 3)
    # a K-contiguous B: the last rows as a launch of 64 x 64 tiles beside a first launch of 255 tiles of 256 x 256
    p = capi.plan(capi.F16F16F16, 4096, 4099, 4096, 0, 1)
    assert (p.tail_rows, p.tail_cols, p.tail_tile_m, p.tail_tile_n, p.grid) == (256, 0, 64, 64, 255)
    # a column-major A makes the dot products expensive: tiles from a shorter K on
    p = capi.plan(capi.F16F16F16, 4096, 4099, 4096, 1, 1)
    assert (p.tail_cols, p.tail_tile_m, p.tail_tile_n) == (3, 128, 128)
    p = capi.plan(capi.F16F16F16, 4096, 4104, 4096, 1, 0)
    assert (p.tail_cols, p.tail_tile_m, p.tail_tile_n) == (8, 128, 128)
    # row-major A and B: a column range of a row-major B keeps the pitch of the whole matrix, which the ring kernel
    # takes as a leading dimension while its rows are whole 16-byte pieces (4104 fp16 are); with N = 4100 they are not,
    # a column cut would put the first launch on the register-staged kernel, and the rows are cut instead
    p = capi.plan(capi.F16F16F16, 2048, 8200, 4096, 0, 0)
    assert (p.tail_cols, p.tail_tile_m, p.tail_tile_n) == (8, 128, 128) and (p.tile_m, p.tile_n) == (256, 256) and p.variant in (5, 6)
    # (4096 x 4104: the last 256 rows as a launch of 64 x 64 tiles cost less than the strip of eight columns)
    p = capi.plan(capi.F16F16F16, 4096, 4104, 4096, 0, 0)
    assert (p.tail_rows, p.tail_cols, p.tail_tile_m, p.variant) == (256, 0, 64, 6)
    p = capi.plan(capi.F16F16F16, 4096, 4100, 4096, 0, 0)
    assert p.tail_cols == 4 and p.variant == 2
    # with a K-contiguous B and a long K the sixteen tiles of that seventeenth tile column are cut along K instead
    # (stream-K)
    p = capi.plan(capi.F16F16F16, 4096, 4104, 8192, 0, 1)
    assert p.tail_cols == 0 and p.streamk_tiles == 16


def test_tile_choice_on_the_register_staged_kernel(capi):
    """Problems that cannot run a direct-to-LDS kernel (ragged K, column-major A, fp32): the estimate was fitted to
    timings on the device, and these are the choices that were fastest there (a mostly empty last round of 256 x 256
    tiles costs less than a whole one; 128 x 128 tiles cost more per round beyond four; the four-wave kernel of
    the 8-bit floats has a large fixed part per tile, so a short K sends them to small tiles; fp32 is charged by
    its products)."""
    tile = lambda *a: (lambda p: (p.tile_m, p.tile_n, p.threads))(capi.plan(*a))
    for types in (capi.BF16BF16F32, capi.S8S8S32):
        for la, lb in ((0, 1), (0, 0), (1, 1)):
            assert tile(types, 6000, 6000, 3000, la, lb) == (256, 256, 512)   # 2.25 rounds, eight waves
            assert tile(types, 5000, 5000, 5000, la, lb) == (256, 256, 512)
            assert tile(types, 2000, 2000, 2000, la, lb)[:2] == (128, 128)
            assert tile(types, 3000, 3000, 1000, la, lb) == (256, 256, 512)
    assert tile(capi.E4M3E4M3F16, 4096, 4096, 4000, 0, 1) == (256, 256, 256)      # four waves for the 8-bit floats
    assert tile(capi.E4M3E4M3F16, 5000, 5000, 5000, 0, 1) == (256, 256, 256)
    assert tile(capi.E4M3E4M3F16, 8000, 8000, 1000, 0, 1)[:2] == (128, 128)
    assert tile(capi.E4M3E4M3F16, 6000, 6000, 3000, 0, 1)[:2] == (128, 128)
    assert tile(capi.F32F32F32, 6000, 6000, 3000, 0, 1)[:2] == (128, 128)
    assert tile(capi.F32F32F32, 3000, 3000, 1000, 0, 0)[:2] == (128, 128)
    assert tile(capi.F32F32F32, 4096, 4096, 4000, 0, 1)[:2] == (256, 256)
    assert tile(capi.F32F32F32, 1000, 8000, 4000, 0, 1)[:2] == (256, 128)


def test_leading_dimension_arguments(capi):
    """gz_gemm_ld checks its leading dimensions before anything touches a device: each at least the extent of a line,
    none negative, none of 2^31 or more; and extents of 2^31 are refused while element counts beyond 2^31 are not an
    argument error."""
    ld = capi.lib.gz_gemm_ld
    base = dict(types=1, a=64, lda=0, b=64, ldb=0, c=0, ldc=0, d=64, ldd=0, m=4, n=6, k=8, la=0, lb=1, alpha=1.0, beta=0.0,
                rung=-1, variant=0, stream=None)

    def call(**kw):
        v = dict(base, **kw)
        return ld(v["types"], v["a"], v["lda"], v["b"], v["ldb"], v["c"], v["ldc"], v["d"], v["ldd"], v["m"], v["n"], v["k"],
                  v["la"], v["lb"], v["alpha"], v["beta"], v["rung"], v["variant"], v["stream"])
    assert call(lda=7) == capi.ERR_BAD_ARG and "lda" in capi.last_error()            # row-major A: at least K
    assert call(la=1, lda=3) == capi.ERR_BAD_ARG                                      # column-major A: at least M
    assert call(ldb=7) == capi.ERR_BAD_ARG and call(lb=0, ldb=5) == capi.ERR_BAD_ARG  # column-major B: K; row-major: N
    assert call(ldc=5) == capi.ERR_BAD_ARG and call(ldd=5) == capi.ERR_BAD_ARG
    assert call(lda=-1) == capi.ERR_BAD_ARG
    assert call(lda=1 << 31) == capi.ERR_UNSUPPORTED
    assert call(m=1 << 31) == capi.ERR_UNSUPPORTED
    # 65536 x 65536 x 32768 holds 2^31 and 2^32 elements per matrix: planned like any other problem
    p = capi.plan(capi.S8S8S32, 65536, 65536, 32768, 0, 1)
    assert p.rung == capi.RUNG_MFMA and (p.tile_m, p.tile_n) == (256, 256)


def test_plan_skinny_split_k(capi):
    """The weight-streaming rung splits K for 65 ... 128 rows from K = 8192 on, with column blocks of up to 256
    columns, and says so in the plan (gz_skinny_cfg.hpp: skinny_resolve_wide)."""
    p = capi.plan(capi.BF16BF16F32, 128, 14336, 8192, capi.ROW_MAJOR, capi.COL_MAJOR, capi.RUNG_SKINNY, 0, 256, 160 * 1024)
    assert (p.split_k, p.tile_m, p.tile_n, p.threads) == (4, 128, 224, 512)
    assert p.grid == 256 and p.workspace_bytes == 256 * 4 * 2 * 4 * 4 * 1024 and p.lds_bytes == 3 * (128 + 256) * 128
    p = capi.plan(capi.BF16BF16F32, 100, 28672, 8192, capi.ROW_MAJOR, capi.COL_MAJOR, capi.RUNG_SKINNY, 0, 256, 160 * 1024)
    assert (p.split_k, p.tile_n) == (2, 224)
    p = capi.plan(capi.BF16BF16F32, 128, 8192, 16384, capi.ROW_MAJOR, capi.COL_MAJOR, capi.RUNG_SKINNY, 0, 256, 160 * 1024)
    assert (p.split_k, p.tile_n, p.lds_bytes) == (4, 128, 4 * (128 + 128) * 128)
    for m, n, k in [(64, 14336, 8192), (128, 14336, 4096), (128, 4096, 8192), (128, 65536, 8192)]:
        p = capi.plan(capi.BF16BF16F32, m, n, k, capi.ROW_MAJOR, capi.COL_MAJOR, capi.RUNG_SKINNY, 0, 256, 160 * 1024)
        assert p.split_k == 1 and p.workspace_bytes == 0, (m, n, k)
    # the entry point that allocates nothing: the split only while its partial sums fit the static buffer
    p = capi.plan_static_scratch(capi.BF16BF16F32, 128, 14336, 8192, capi.ROW_MAJOR, capi.COL_MAJOR, capi.RUNG_SKINNY, 0, 256, 160 * 1024)
    assert p.split_k == 4 and p.workspace_bytes <= capi.STATIC_SCRATCH_BYTES
