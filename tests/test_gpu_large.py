"""Matrices of 2^31 elements and more (the reference indexes with std::size_t, nvidia/utils/benchmark.cuh:17,
nvidia/kernels/naive_gemm.cuh:8): extents stay below 2^31, every index the kernels form is 64-bit.  Operands are
filled on the device; bands of rows are checked bit for bit against the CPU oracle, and the whole product with
Freivalds' identities y (A B) = (y A) B and (A B) x = A (B x) on small integer vectors, evaluated in float64 where
every value involved is an exact integer."""
import numpy as np
import pytest
import torch

import oracle_lib as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def as_f64_matrix(t, rows, cols, types):
    """A device operand (flat, rows x cols in memory) as float64 values."""
    if types == O.S8S8S32:
        return t.view(rows, cols).double()
    return t.view(torch.bfloat16).view(rows, cols).double()


def chunked_matvec(t, rows, cols, types, x_right=None, y_left=None, chunk=2048):
    """M x (cols) or y M for a matrix too large to widen at once; float64 on the device."""
    m = t.view(rows, cols) if types == O.S8S8S32 else t.view(torch.bfloat16).view(rows, cols)
    if x_right is not None:
        return torch.cat([m[r:r + chunk].double() @ x_right for r in range(0, rows, chunk)])
    acc = torch.zeros(cols, dtype=torch.float64, device=t.device)
    for r in range(0, rows, chunk):
        acc += y_left[r:r + chunk] @ m[r:r + chunk].double()
    return acc


@pytest.mark.parametrize("types,shape,lb", [
    (O.S8S8S32, (65536, 256, 32768), O.COL),      # A: 2^31 elements; whole 256 x 256 tiles on the ring kernel
    (O.S8S8S32, (65536, 256, 32768), O.ROW),
    (O.BF16BF16F32, (40000, 512, 60000), O.COL),  # A: 2.4e9 elements; ragged M, K not a whole number of slabs
    (O.BF16BF16F32, (40000, 512, 60000), O.ROW),
    (O.BF16BF16F32, (40000, 512, 60032), O.COL),  # whole slabs: the ring kernel's ragged instance
])
def test_operands_past_two_to_the_31_elements(G, types, shape, lb):
    m, n, k = shape
    assert m * k >= 1 << 31
    capi = G.capi
    it, in_dt = (torch.int8, O.DT_INT8) if types == O.S8S8S32 else (torch.int16, O.DT_BF16)
    ot = torch.int32 if types == O.S8S8S32 else torch.float32
    kind = O.FILL_INT8_UNIFORM if types == O.S8S8S32 else O.FILL_SMALL_INT   # every partial sum exact
    a = torch.empty(m * k, dtype=it, device="cuda"); b = torch.empty(k * n, dtype=it, device="cuda")
    capi.fill(a, m * k, in_dt, kind, 1.0, 101); capi.fill(b, k * n, in_dt, kind, 1.0, 102)
    d = torch.empty(m * n, dtype=ot, device="cuda")
    print("case", types, shape, lb, flush=True)
    capi.gemm(types, a, b, None, d, m, n, k, O.ROW, lb, 1, 0)
    torch.cuda.synchronize()
    # bands of rows against the oracle: the first rows, rows whose offset in A straddles 2^31 elements, the last rows
    hb = b.cpu().numpy()
    if types != O.S8S8S32:
        hb = hb.view(np.uint16)
    edge = (1 << 31) // k
    for r0 in (0, min(max(edge - 4, 0), m - 8), m - 8):
        band = a[r0 * k:(r0 + 8) * k].cpu().numpy()
        if types != O.S8S8S32:
            band = band.view(np.uint16)
        ref = O.gemm(types, band, hb, None, 8, n, k, O.ROW, lb, 1, 0)
        got = d[r0 * n:(r0 + 8) * n].cpu().numpy().reshape(8, n)
        assert np.array_equal(got, ref), (types, shape, lb, r0)
    # the whole product: Freivalds
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randint(-3, 4, (n,), generator=gen, device="cuda").double()
    y = torch.randint(-3, 4, (m,), generator=gen, device="cuda").double()
    bm = as_f64_matrix(b, k, n, types) if lb == O.ROW else as_f64_matrix(b, n, k, types).t()
    dm = d.view(m, n).double()
    assert torch.equal(dm @ x, chunked_matvec(a, m, k, types, x_right=bm @ x))
    assert torch.equal(y @ dm, chunked_matvec(a, m, k, types, y_left=y) @ bm)
    del dm, bm
    # the LDS-tiled rung on the same operands (its own 64-bit indexing), compared on the device
    d2 = torch.empty(m * n, dtype=ot, device="cuda")
    capi.gemm(types, a, b, None, d2, m, n, k, O.ROW, lb, 1, 0, capi.RUNG_LDS_TILED)
    torch.cuda.synchronize()
    assert capi.compare(d, d2, m * n, O.DT_INT32 if types == O.S8S8S32 else O.DT_F32, 0.0) == 0


def test_output_past_two_to_the_31_elements(G):
    """D with 2^31 elements: int8 46400 x 46400 x 128 (one slab), whole-tile and ragged epilogues at large offsets."""
    capi = G.capi
    types, (m, n, k) = O.S8S8S32, (46400, 46400, 128)
    assert m * n >= 1 << 31
    a = torch.empty(m * k, dtype=torch.int8, device="cuda"); b = torch.empty(k * n, dtype=torch.int8, device="cuda")
    capi.fill(a, m * k, O.DT_INT8, O.FILL_INT8_UNIFORM, 1.0, 7); capi.fill(b, k * n, O.DT_INT8, O.FILL_INT8_UNIFORM, 1.0, 8)
    d = torch.empty(m * n, dtype=torch.int32, device="cuda")
    capi.gemm(types, a, b, None, d, m, n, k, O.ROW, O.COL, 1, 0)
    torch.cuda.synchronize()
    ha, hb = a.cpu().numpy(), b.cpu().numpy()
    for r0 in (0, (1 << 31) // n - 4, m - 8):
        ref = O.gemm(types, ha[r0 * k:(r0 + 8) * k], hb, None, 8, n, k, O.ROW, O.COL, 1, 0)
        assert np.array_equal(d[r0 * n:(r0 + 8) * n].cpu().numpy().reshape(8, n), ref), r0
    gen = torch.Generator(device="cuda").manual_seed(6)
    x = torch.randint(-3, 4, (n,), generator=gen, device="cuda").double()
    am, bm = a.view(m, k).double(), b.view(n, k).double()
    lhs = torch.cat([d.view(m, n)[r:r + 1024].double() @ x for r in range(0, m, 1024)])
    assert torch.equal(lhs, am @ (bm.t() @ x))
