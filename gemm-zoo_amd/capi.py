"""ctypes binding of ``lib/libgemmzoo.so`` (the C ABI declared in ``include/gemm_zoo.h``).

The library is the only compute path: if it is missing this module raises at import
time instead of falling back to anything else.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

_HERE = Path(__file__).resolve().parent
LIB_PATH = _HERE / "lib" / "libgemmzoo.so"

# enums of include/gemm_zoo.h
OK, ERR_BAD_ARG, ERR_UNSUPPORTED, ERR_HIP, ERR_MISMATCH = 0, 1, 2, 3, 4
ROW_MAJOR, COL_MAJOR = 0, 1
S8S8S32, BF16BF16F32, BF16BF16BF16, F16F16F16, F32F32F32, E4M3E4M3F16, E5M2E5M2F16 = 0, 1, 2, 3, 4, 5, 6
BF16BF16BF16_ACC16, F16F16F16_ACC16 = 7, 8   # opt-in: the reference kernels' 16-bit running sums
NUM_TYPES = 9
RUNG_AUTO, RUNG_NAIVE, RUNG_COALESCED, RUNG_LDS_TILED, RUNG_DOUBLE_BUFFERED, RUNG_MFMA, RUNG_SKINNY = -1, 0, 1, 2, 3, 4, 5
NUM_RUNGS = 6
DT_INT8, DT_BF16, DT_F16, DT_F32, DT_INT32, DT_E4M3, DT_E5M2 = 0, 1, 2, 3, 4, 5, 6
FILL_INT8_UNIFORM, FILL_NORMAL, FILL_UNIFORM_PM1, FILL_SMALL_INT = 0, 1, 2, 3
# tile configurations of the MFMA rung (variant ids; 0 = the launcher chooses): the register-staged / compiler-scheduled
# kernels on four tiles, the hand-scheduled ring kernel on four and eight waves, the same with the stream-K
# decomposition, and the ring kernel with one work-group per tile instead of one per compute unit
MFMA_256_W4, MFMA_256_W8, MFMA_128, MFMA_256X128 = 1, 2, 3, 4
MFMA_RING_W4, MFMA_RING_W8, MFMA_STREAMK_W4, MFMA_STREAMK_W8, MFMA_RING_W4_PER_TILE, MFMA_RING_W8_PER_TILE = 5, 6, 7, 8, 9, 10
MFMA_RING_128 = 11

TYPES_NAMES = {S8S8S32: "s8s8s32", BF16BF16F32: "bf16bf16f32", BF16BF16BF16: "bf16bf16bf16", F16F16F16: "f16f16f16",
               F32F32F32: "f32f32f32", E4M3E4M3F16: "e4m3e4m3f16", E5M2E5M2F16: "e5m2e5m2f16",
               BF16BF16BF16_ACC16: "bf16bf16bf16_acc16", F16F16F16_ACC16: "f16f16f16_acc16"}
IN_SIZE = {S8S8S32: 1, BF16BF16F32: 2, BF16BF16BF16: 2, F16F16F16: 2, F32F32F32: 4, E4M3E4M3F16: 1, E5M2E5M2F16: 1,
           BF16BF16BF16_ACC16: 2, F16F16F16_ACC16: 2}
OUT_SIZE = {S8S8S32: 4, BF16BF16F32: 4, BF16BF16BF16: 2, F16F16F16: 2, F32F32F32: 4, E4M3E4M3F16: 2, E5M2E5M2F16: 2,
            BF16BF16BF16_ACC16: 2, F16F16F16_ACC16: 2}

EXPORTS = [
    "gz_gemm_s8s8s32", "gz_gemm_bf16bf16f32", "gz_gemm_bf16bf16bf16", "gz_gemm_f16f16f16", "gz_gemm_f32f32f32",
    "gz_gemm_e4m3e4m3f16", "gz_gemm_e5m2e5m2f16", "gz_gemm_bf16bf16bf16_acc16", "gz_gemm_f16f16f16_acc16", "gz_gemm",
    "gz_plan", "gz_variant_count", "gz_rung_name", "gz_types_name", "gz_fill", "gz_compare", "gz_compare_rel",
    "gz_last_error", "gz_version", "gz_device_props", "gz_gemm_static_scratch", "gz_plan_static_scratch", "gz_gemm_ld",
]


class GzError(RuntimeError):
    """A non-zero gz_status; ``status`` holds the code, the text is gz_last_error()."""

    def __init__(self, status: int, message: str):
        super().__init__(f"gz status {status}: {message}")
        self.status = status


class Plan(C.Structure):
    _fields_ = [
        ("rung", C.c_int32), ("variant", C.c_int32),
        ("tile_m", C.c_int32), ("tile_n", C.c_int32), ("tile_k", C.c_int32),
        ("wave_m", C.c_int32), ("wave_n", C.c_int32),
        ("threads", C.c_int32), ("lds_bytes", C.c_int32),
        ("grid", C.c_int64), ("split_k", C.c_int32),
        ("vector_bytes_a", C.c_int32), ("vector_bytes_b", C.c_int32),
        ("tail_rows", C.c_int32), ("tail_tile_m", C.c_int32), ("tail_tile_n", C.c_int32), ("tail_grid", C.c_int64),
        ("tail_cols", C.c_int32),
        ("streamk_tiles", C.c_int32), ("streamk_blocks", C.c_int32), ("workspace_bytes", C.c_int64),
    ]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


def _load():
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python gemm-zoo_amd/build.py` "
            "(there is no fallback path)")
    lib = C.CDLL(str(LIB_PATH))
    vp, i64, i32, f32, f64 = C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_double
    common = [vp, vp, vp, vp, i64, i64, i64, i32, i32]
    lib.gz_gemm_s8s8s32.argtypes = common + [C.c_int32, C.c_int32, i32, i32, vp]
    for name in ("gz_gemm_bf16bf16f32", "gz_gemm_bf16bf16bf16", "gz_gemm_f16f16f16", "gz_gemm_f32f32f32",
                 "gz_gemm_e4m3e4m3f16", "gz_gemm_e5m2e5m2f16", "gz_gemm_bf16bf16bf16_acc16",
                 "gz_gemm_f16f16f16_acc16"):
        getattr(lib, name).argtypes = common + [f32, f32, i32, i32, vp]
    lib.gz_gemm.argtypes = [i32] + common + [f64, f64, i32, i32, vp]
    lib.gz_gemm_static_scratch.argtypes = [i32] + common + [f64, f64, i32, i32, vp]
    lib.gz_gemm_ld.argtypes = [i32, vp, i64, vp, i64, vp, i64, vp, i64, i64, i64, i64, i32, i32, f64, f64, i32, i32, vp]
    lib.gz_plan.argtypes = [i32, i64, i64, i64, i32, i32, i32, i32, i32, i32, C.POINTER(Plan)]
    lib.gz_plan_static_scratch.argtypes = lib.gz_plan.argtypes
    lib.gz_variant_count.argtypes = [i32, i32]
    lib.gz_rung_name.argtypes = [i32]
    lib.gz_rung_name.restype = C.c_char_p
    lib.gz_types_name.argtypes = [i32]
    lib.gz_types_name.restype = C.c_char_p
    lib.gz_fill.argtypes = [vp, i64, i32, i32, f32, C.c_uint64, vp]
    lib.gz_compare.argtypes = [vp, vp, i64, i32, f32, C.POINTER(C.c_int64), vp]
    lib.gz_compare_rel.argtypes = [vp, vp, i64, i32, f32, f32, C.POINTER(C.c_int64), vp]
    lib.gz_last_error.restype = C.c_char_p
    lib.gz_device_props.argtypes = [C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    for name in EXPORTS:
        fn = getattr(lib, name)
        if fn.restype is C.c_int or fn.restype is None:
            fn.restype = C.c_int
    return lib


lib = _load()


def last_error() -> str:
    return lib.gz_last_error().decode()


def check(status: int) -> None:
    if status != OK:
        raise GzError(status, last_error())


def _ptr(x) -> int:
    """Device pointer of a torch tensor, an int, or None."""
    if x is None:
        return 0
    if isinstance(x, int):
        return x
    return x.data_ptr()


def gemm(types: int, a, b, c, d, m: int, n: int, k: int, layout_a: int = ROW_MAJOR, layout_b: int = ROW_MAJOR,
         alpha=1, beta=0, rung: int = RUNG_AUTO, variant: int = 0, stream: int = 0) -> None:
    """Typed entry point dispatch (raises GzError on a non-zero status)."""
    fn = {S8S8S32: lib.gz_gemm_s8s8s32, BF16BF16F32: lib.gz_gemm_bf16bf16f32,
          BF16BF16BF16: lib.gz_gemm_bf16bf16bf16, F16F16F16: lib.gz_gemm_f16f16f16,
          F32F32F32: lib.gz_gemm_f32f32f32, E4M3E4M3F16: lib.gz_gemm_e4m3e4m3f16,
          E5M2E5M2F16: lib.gz_gemm_e5m2e5m2f16, BF16BF16BF16_ACC16: lib.gz_gemm_bf16bf16bf16_acc16,
          F16F16F16_ACC16: lib.gz_gemm_f16f16f16_acc16}.get(types)
    if fn is None:
        raise GzError(ERR_BAD_ARG, f"unknown type bundle {types}")
    if types == S8S8S32:
        alpha, beta = int(alpha), int(beta)
    check(fn(_ptr(a), _ptr(b), _ptr(c), _ptr(d), m, n, k, layout_a, layout_b, alpha, beta, rung, variant, stream))


def gemm_ld(types: int, a, lda: int, b, ldb: int, c, ldc: int, d, ldd: int, m: int, n: int, k: int,
            layout_a: int = ROW_MAJOR, layout_b: int = ROW_MAJOR, alpha=1, beta=0, rung: int = RUNG_AUTO, variant: int = 0,
            stream: int = 0) -> None:
    """gz_gemm_ld: matrices with leading dimensions in elements, 0 = packed (raises GzError on a non-zero status)."""
    check(lib.gz_gemm_ld(types, _ptr(a), lda, _ptr(b), ldb, _ptr(c), ldc, _ptr(d), ldd, m, n, k, layout_a, layout_b,
                         float(alpha), float(beta), rung, variant, stream))


STATIC_SCRATCH_BYTES = 96 << 20


def gemm_static_scratch(types: int, a, b, c, d, m: int, n: int, k: int, layout_a: int = ROW_MAJOR,
                        layout_b: int = ROW_MAJOR, alpha=1, beta=0, rung: int = RUNG_AUTO, variant: int = 0,
                        stream: int = 0) -> None:
    """gz_gemm_static_scratch: gz_gemm for callers that cannot allocate (raises GzError on a non-zero status)."""
    check(lib.gz_gemm_static_scratch(types, _ptr(a), _ptr(b), _ptr(c), _ptr(d), m, n, k, layout_a, layout_b,
                                     float(alpha), float(beta), rung, variant, stream))


def plan(types: int, m: int, n: int, k: int, layout_a: int = ROW_MAJOR, layout_b: int = ROW_MAJOR,
         rung: int = RUNG_AUTO, variant: int = 0, num_cus: int = 0, lds_per_cu: int = 0) -> Plan:
    p = Plan()
    check(lib.gz_plan(types, m, n, k, layout_a, layout_b, rung, variant, num_cus, lds_per_cu, C.byref(p)))
    return p


def plan_static_scratch(types: int, m: int, n: int, k: int, layout_a: int = ROW_MAJOR, layout_b: int = ROW_MAJOR,
                        rung: int = RUNG_AUTO, variant: int = 0, num_cus: int = 0, lds_per_cu: int = 0) -> Plan:
    """The plan gz_gemm_static_scratch takes: gz_plan within the static scratch buffer."""
    p = Plan()
    check(lib.gz_plan_static_scratch(types, m, n, k, layout_a, layout_b, rung, variant, num_cus, lds_per_cu, C.byref(p)))
    return p


def fill(dst, count: int, dtype: int, kind: int, scale: float = 1.0, seed: int = 2025, stream: int = 0) -> None:
    check(lib.gz_fill(_ptr(dst), count, dtype, kind, scale, seed, stream))


def compare(out, ref, count: int, dtype: int, abs_threshold: float = 0.0, stream: int = 0,
            rel_threshold: float = 0.0) -> int:
    """Returns the number of differing elements (0 = equal); raises only on API errors."""
    nd = C.c_int64(0)
    st = lib.gz_compare_rel(_ptr(out), _ptr(ref), count, dtype, abs_threshold, rel_threshold, C.byref(nd), stream)
    if st not in (OK, ERR_MISMATCH):
        raise GzError(st, last_error())
    return nd.value


def device_props() -> tuple[int, int]:
    """(compute units, LDS bytes per compute unit) of the current device, as the C++ functors read them."""
    cus, lds = C.c_int32(0), C.c_int32(0)
    check(lib.gz_device_props(C.byref(cus), C.byref(lds)))
    return cus.value, lds.value


def variant_count(types: int, rung: int) -> int:
    return lib.gz_variant_count(types, rung)


def rung_name(rung: int) -> str:
    return lib.gz_rung_name(rung).decode()
