"""Device fill == CPU fill bit for bit; compare kernel semantics (harness rows of the hot path)."""
import numpy as np
import pytest
import torch

import oracle_lib as O

pytestmark = pytest.mark.gpu

TORCH_OF_DT = {O.DT_INT8: torch.int8, O.DT_BF16: torch.int16, O.DT_F16: torch.int16, O.DT_F32: torch.float32,
               O.DT_INT32: torch.int32, O.DT_E4M3: torch.uint8, O.DT_E5M2: torch.uint8}


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


@pytest.mark.parametrize("dtype", [O.DT_INT8, O.DT_BF16, O.DT_F16, O.DT_F32, O.DT_INT32, O.DT_E4M3, O.DT_E5M2])
@pytest.mark.parametrize("kind", [O.FILL_INT8_UNIFORM, O.FILL_NORMAL, O.FILL_UNIFORM_PM1, O.FILL_SMALL_INT])
def test_device_fill_matches_cpu_fill_bit_for_bit(G, dtype, kind):
    if dtype in (O.DT_INT8, O.DT_INT32) and kind in (O.FILL_NORMAL, O.FILL_UNIFORM_PM1):
        pytest.skip("real-valued kinds are for float destinations")
    cases = [(1, 1, 1.0), (1000003, 2025, 1.0), (70000, (5 << 32) | 17, 0.02)]
    if dtype in (O.DT_E4M3, O.DT_E5M2):  # 8-bit floats: also the subnormal range and saturation at the top
        cases += [(50000, 3, 2.0 ** -8), (50000, 4, 2.0 ** -15), (50000, 5, 300.0), (50000, 6, 1e6)]
    for count, seed, scale in cases:
        t = torch.zeros(count + 8, dtype=TORCH_OF_DT[dtype], device="cuda")
        G.capi.fill(t, count, dtype, kind, scale, seed, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        got = t.cpu().numpy()
        assert not got[count:].any(), "fill wrote past count"
        want = O.fill(count, dtype, kind, scale, seed)
        assert np.array_equal(got[:count].view(want.dtype), want), (dtype, kind, count, seed)


def test_compare_exact_and_threshold(G):
    n = 100000
    a = torch.arange(n, dtype=torch.float32, device="cuda")
    b = a.clone()
    assert G.capi.compare(a, b, n, O.DT_F32, 0.0) == 0
    b[17] += 0.25; b[99999] -= 1.0
    assert G.capi.compare(a, b, n, O.DT_F32, 0.0) == 2          # exact: intel/test/utils.hpp:57
    assert G.capi.compare(a, b, n, O.DT_F32, 0.5) == 1          # abs threshold: nvidia/utils/compare.cuh:19
    assert G.capi.compare(a, b, n, O.DT_F32, 0.0, rel_threshold=1e-4) == 1   # 0.25 at 17 is out, 1.0 at 99999 is in
    assert G.capi.compare(a, b, n, O.DT_F32, 0.2, rel_threshold=1e-2) == 0
    st = G.capi.lib.gz_compare(a.data_ptr(), b.data_ptr(), n, O.DT_F32, 0.0, None, None)
    assert st == G.capi.ERR_MISMATCH and "verification failed" in G.capi.last_error()
    i = torch.arange(n, dtype=torch.int32, device="cuda"); j = i.clone(); j[5] += 1
    assert G.capi.compare(i, j, n, O.DT_INT32, 0.0) == 1
    h = torch.from_numpy(np.array([0x3C00, 0x8000, 0x7E00], np.uint16).view(np.int16)).cuda()
    g = torch.from_numpy(np.array([0x3C00, 0x0000, 0x7E00], np.uint16).view(np.int16)).cuda()
    assert G.capi.compare(h, g, 3, O.DT_F16, 0.0) == 1          # -0 == +0, NaN != NaN (value compare)
    assert G.capi.compare(h, g, 0, O.DT_F16, 0.0) == 0
