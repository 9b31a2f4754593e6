"""Helpers shared by the GPU parity tests: device buffers via torch, calls through the C ABI."""
from __future__ import annotations

import importlib

import numpy as np
import torch

import oracle_lib as O

capi = importlib.import_module("gemm-zoo_amd.capi")

TOL = {O.BF16BF16F32: 1e-3, O.BF16BF16BF16: 1e-2, O.F16F16F16: 1e-2,  # max relative error allowed for fp32 / 16-bit outputs
       O.F32F32F32: 1e-4,  # fp32 inputs: only the summation order differs
       O.E4M3E4M3F16: 1e-2, O.E5M2E5M2F16: 1e-2}  # fp16 output, exact products: the 16-bit-output bound


def dev():
    return torch.device("cuda:0")


def up(x: np.ndarray | None, misalign_elems: int = 0):
    """Host array -> device tensor (16-bit patterns travel as int16).  misalign_elems > 0 returns a view
    that starts that many elements into a larger allocation (an operand that is not 16-byte aligned)."""
    if x is None:
        return None
    h = x.view(np.int16) if x.dtype == np.uint16 else x.view(np.int8) if x.dtype == np.uint8 else x
    t = torch.from_numpy(np.ascontiguousarray(h))
    if misalign_elems:
        big = torch.zeros(t.numel() + misalign_elems + 64, dtype=t.dtype, device=dev())
        big[misalign_elems:misalign_elems + t.numel()] = t.to(dev())
        return big[misalign_elems:misalign_elems + t.numel()]
    return t.to(dev())


def down(t: torch.Tensor, types: int, m: int, n: int) -> np.ndarray:
    return t.cpu().numpy().view(O.OUT_DTYPE[types]).reshape(m, n)


def out_torch_dtype(types):
    return {O.S8S8S32: torch.int32, O.BF16BF16F32: torch.float32, O.F32F32F32: torch.float32}.get(types, torch.int16)


def run_gemm(types, a, b, c, m, n, k, la, lb, alpha, beta, rung, variant=0, misalign=0, guard=64):
    """Runs the HIP path on host arrays; returns D (m x n) and checks nothing was written around it."""
    da, db = up(a, misalign), up(b, misalign)
    dc = up(c, misalign) if c is not None else None
    sentinel = 0x5A5A if O.OUT_DTYPE[types] == np.uint16 else 0x5A5A5A5A
    full = torch.full((m * n + 2 * guard,), sentinel, dtype=out_torch_dtype(types), device=dev())
    dd = full[guard:guard + m * n]
    capi.gemm(types, da, db, dc, dd, m, n, k, la, lb, alpha, beta, rung, variant,
              torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    host = full.cpu()
    assert (host[:guard] == sentinel).all() and (host[guard + m * n:] == sentinel).all(), "wrote outside D"
    return host[guard:guard + m * n].numpy().view(O.OUT_DTYPE[types]).reshape(m, n)


def assert_within(types, got, truth_f64, what=""):
    """|x - ref| <= tol * max(|ref_ij|, rms(ref)) element-wise; returns the worst ratio for reporting."""
    tol = TOL[types]
    g = O.out_to_f64(types, got)
    rms = float(np.sqrt((truth_f64 ** 2).mean())) if truth_f64.size else 0.0
    bound = tol * np.maximum(np.abs(truth_f64), rms)
    err = np.abs(g - truth_f64)
    worst = float((err / np.maximum(bound, 1e-300)).max()) if err.size else 0.0
    assert worst <= 1.0, f"{what}: error is {worst:.3f} x the allowed {tol} relative bound"
    return worst * tol


def run_gemm_ld(types, a, b, c, m, n, k, la, lb, alpha, beta, rung, variant=0, pads=(0, 0, 0, 0), misalign=0):
    """gz_gemm_ld on sub-matrix views: every operand sits in a wider allocation whose leading dimension is its packed
    one plus pads[i] elements, the padding filled with a pattern that is a NaN for the float types and a large value
    for int8, so that a kernel that reads across a line's end shows.  a, b, c are the packed host arrays (a: m x k or
    k x m as its layout says, flat is fine).  Returns D (m x n) and checks that neither the padding of D nor the
    words around it were written."""
    def lines(layout_rows_major, rows, cols):   # (number of lines, line length)
        return (rows, cols) if layout_rows_major else (cols, rows)

    def widen(x, nlines, length, pad):
        x = np.asarray(x).reshape(nlines, length)
        big = np.empty((nlines, length + pad), dtype=x.dtype)
        # NaN patterns of bf16 / fp16 (0x7fc1), e4m3 / e5m2 (0x7f), fp32; large values for the integer types
        big[...] = {np.dtype(np.uint16): 0x7FC1, np.dtype(np.uint8): 0x7F, np.dtype(np.int8): 127,
                    np.dtype(np.int32): 0x5A5A5A5A, np.dtype(np.float32): np.nan}[x.dtype]
        big[:, :length] = x
        return big

    an, al = lines(la == O.ROW, m, k)
    bn, bl = lines(lb == O.ROW, k, n)
    pa, pb, pc, pd = pads
    abig = widen(a, an, al, pa)
    bbig = widen(b, bn, bl, pb)
    da, db = up(abig.reshape(-1), misalign), up(bbig.reshape(-1), misalign)
    dc = None
    if c is not None:
        cbig = widen(c, m, n, pc)
        dc = up(cbig.reshape(-1), misalign)
    sentinel = 0x5A5A if O.OUT_DTYPE[types] == np.uint16 else 0x5A5A5A5A
    guard = 64
    ldd = n + pd
    full = torch.full((m * ldd + 2 * guard,), sentinel, dtype=out_torch_dtype(types), device=dev())
    dd = full[guard:guard + m * ldd]
    capi.gemm_ld(types, da, al + pa, db, bl + pb, dc, n + pc, dd, ldd, m, n, k, la, lb, alpha, beta, rung, variant,
                 torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    host = full.cpu()
    assert (host[:guard] == sentinel).all() and (host[guard + m * ldd:] == sentinel).all(), "wrote outside D"
    body = host[guard:guard + m * ldd].reshape(m, ldd)
    assert (body[:, n:] == sentinel).all(), "wrote into the padding between the rows of D"
    return np.ascontiguousarray(body[:, :n].numpy()).view(O.OUT_DTYPE[types]).reshape(m, n)
