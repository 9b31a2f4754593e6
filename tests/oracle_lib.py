"""ctypes wrapper of the CPU checker in ``oracle/`` (test infrastructure only)."""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
ORACLE_DIR = ROOT / "oracle"
LIB = ORACLE_DIR / "liboracle.so"

S8S8S32, BF16BF16F32, BF16BF16BF16, F16F16F16, F32F32F32, E4M3E4M3F16, E5M2E5M2F16 = 0, 1, 2, 3, 4, 5, 6
BF16BF16BF16_ACC16, F16F16F16_ACC16 = 7, 8   # the reference kernels' 16-bit running sums (chunks of 16 / 8 k)
FP8_TYPES = (E4M3E4M3F16, E5M2E5M2F16)
ACC16_TYPES = (BF16BF16BF16_ACC16, F16F16F16_ACC16)
ACC16_CHUNK = {BF16BF16BF16_ACC16: 16, F16F16F16_ACC16: 8}
ROW, COL = 0, 1
IN_DTYPE = {0: np.int8, 1: np.uint16, 2: np.uint16, 3: np.uint16, 4: np.float32, 5: np.uint8, 6: np.uint8, 7: np.uint16,
            8: np.uint16}
OUT_DTYPE = {0: np.int32, 1: np.float32, 2: np.uint16, 3: np.uint16, 4: np.float32, 5: np.uint16, 6: np.uint16,
             7: np.uint16, 8: np.uint16}
# gz_fill / oracle_fill codes
DT_INT8, DT_BF16, DT_F16, DT_F32, DT_INT32, DT_E4M3, DT_E5M2 = 0, 1, 2, 3, 4, 5, 6
NP_OF_DT = {0: np.int8, 1: np.uint16, 2: np.uint16, 3: np.float32, 4: np.int32, 5: np.uint8, 6: np.uint8}
FILL_INT8_UNIFORM, FILL_NORMAL, FILL_UNIFORM_PM1, FILL_SMALL_INT = 0, 1, 2, 3
IN_DT = {0: DT_INT8, 1: DT_BF16, 2: DT_BF16, 3: DT_F16, 4: DT_F32, 5: DT_E4M3, 6: DT_E5M2, 7: DT_BF16, 8: DT_F16}
OUT_DT = {0: DT_INT32, 1: DT_F32, 2: DT_BF16, 3: DT_F16, 4: DT_F32, 5: DT_F16, 6: DT_F16, 7: DT_BF16, 8: DT_F16}


def _load():
    src = ORACLE_DIR / "gz_oracle.c"
    if not LIB.exists() or LIB.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(["make", "-C", str(ORACLE_DIR)], check=True, capture_output=True)
    lib = C.CDLL(str(LIB))
    vp, i64, i32, f64 = C.c_void_p, C.c_int64, C.c_int, C.c_double
    lib.oracle_gemm.argtypes = [i32, vp, vp, vp, vp, i64, i64, i64, i32, i32, f64, f64, i32]
    lib.oracle_gemm_rows.argtypes = [i32, vp, vp, vp, vp, i64, i64, i64, i32, i32, f64, f64, i64, i64, i32]
    lib.oracle_gemm_naive_rows.argtypes = lib.oracle_gemm_rows.argtypes
    lib.oracle_gemm_f64.argtypes = [i32, vp, vp, vp, vp, vp, i64, i64, i64, i32, i32, f64, f64, i64, i64, i32]
    lib.oracle_literal_s8s32.argtypes = [vp, vp, vp, vp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int32, C.c_int32]
    lib.oracle_literal_f32.argtypes = [vp, vp, vp, vp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float, C.c_float]
    lib.oracle_fill.argtypes = [vp, i64, i32, i32, C.c_float, C.c_uint64, i32]
    lib.oracle_philox4x32_10.argtypes = [C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
    lib.oracle_bf16_to_f32.argtypes = [C.c_uint16]
    lib.oracle_bf16_to_f32.restype = C.c_float
    lib.oracle_f16_to_f32.argtypes = [C.c_uint16]
    lib.oracle_f16_to_f32.restype = C.c_float
    lib.oracle_f32_to_bf16.argtypes = [C.c_float]
    lib.oracle_f32_to_bf16.restype = C.c_uint16
    lib.oracle_f32_to_f16.argtypes = [C.c_float]
    lib.oracle_f32_to_f16.restype = C.c_uint16
    lib.oracle_fp8_to_f32.argtypes = [i32, C.c_uint8]
    lib.oracle_fp8_to_f32.restype = C.c_float
    lib.oracle_f32_to_fp8.argtypes = [i32, C.c_float]
    lib.oracle_f32_to_fp8.restype = C.c_uint8
    lib.oracle_f64_to_f16.argtypes = [C.c_double]
    lib.oracle_f64_to_f16.restype = C.c_uint16
    lib.oracle_fma_f16.argtypes = [C.c_float, C.c_float, C.c_float]
    lib.oracle_fma_f16.restype = C.c_uint16
    lib.oracle_normal_from_words.argtypes = [C.c_uint32, C.c_uint32]
    lib.oracle_normal_from_words.restype = C.c_float
    lib.oracle_num_threads.restype = i32
    return lib


lib = _load()


def _p(a):
    return None if a is None else a.ctypes.data


def gemm(types, a, b, c, m, n, k, la=ROW, lb=ROW, alpha=1.0, beta=0.0, threads=0, rows=None, naive=False):
    """D (or rows [r0,r1) of it, other rows left zero) from the CPU oracle."""
    d = np.zeros((m, n), dtype=OUT_DTYPE[types])
    r0, r1 = (0, m) if rows is None else rows
    fn = lib.oracle_gemm_naive_rows if naive else lib.oracle_gemm_rows
    st = fn(types, _p(a), _p(b), _p(c), _p(d), m, n, k, la, lb, float(alpha), float(beta), r0, r1, threads)
    if st != 0:
        raise RuntimeError(f"oracle status {st}")
    return d


def gemm_f64(types, a, b, c, m, n, k, la=ROW, lb=ROW, alpha=1.0, beta=0.0, rows=None, threads=0):
    """(truth, sum|a||b|) for rows [r0,r1) in float64."""
    r0, r1 = (0, m) if rows is None else rows
    out = np.zeros((r1 - r0, n), dtype=np.float64)
    ab = np.zeros((r1 - r0, n), dtype=np.float64)
    st = lib.oracle_gemm_f64(types, _p(a), _p(b), _p(c), _p(out), _p(ab), m, n, k, la, lb, float(alpha), float(beta),
                             r0, r1, threads)
    if st != 0:
        raise RuntimeError(f"oracle status {st}")
    return out, ab


def fill(count, dtype, kind, scale=1.0, seed=2025, threads=0):
    out = np.empty(count, dtype=NP_OF_DT[dtype])
    st = lib.oracle_fill(_p(out), count, dtype, kind, scale, seed, threads)
    if st != 0:
        raise RuntimeError(f"oracle status {st}")
    return out


def philox(ctr, key):
    c = (C.c_uint32 * 4)(*ctr)
    k = (C.c_uint32 * 2)(*key)
    o = (C.c_uint32 * 4)()
    lib.oracle_philox4x32_10(c, k, o)
    return list(o)


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f16_to_f32(bits: np.ndarray) -> np.ndarray:
    return bits.view(np.float16).astype(np.float32)


def out_to_f64(types, d: np.ndarray) -> np.ndarray:
    if types in (BF16BF16BF16, BF16BF16BF16_ACC16):
        return bf16_to_f32(d).astype(np.float64)
    if types in (F16F16F16, F16F16F16_ACC16) or types in FP8_TYPES:
        return f16_to_f32(d).astype(np.float64)
    return d.astype(np.float64)


def make_inputs(types, m, n, k, kind=None, seed=2025, scale_a=1.0, scale_b=1.0, with_c=True):
    """Seeded operands as flat host arrays (the layout is only an interpretation)."""
    if kind is None:
        kind = FILL_INT8_UNIFORM if types == S8S8S32 else FILL_NORMAL
    a = fill(m * k, IN_DT[types], kind, scale_a, seed)
    b = fill(k * n, IN_DT[types], kind, scale_b, seed + 1)
    c = None
    if with_c:
        ckind = kind if types != S8S8S32 else FILL_INT8_UNIFORM
        c = fill(m * n, OUT_DT[types], ckind, 1.0, seed + 2)
    return a, b, c
