"""The C++ surface on the GPU: the reference's bench mains, compiled unchanged against the functor and harness
headers (nvidia/bench/bench_bf16_mma_gemm.cu:9-28, nvidia/bench/bench_fp16_mma_gemm.cu,
bench/bench_xe_gemm_s8_s8_s32_m8k16.cpp:10-18), run as child processes.  The harness verifies every size against
hipBLASLt (or the any-shape kernel) before it times it and throws on a mismatch, so rc 0 plus one "GEMM Problem:"
line per size means: the functor constructors planned with the device's real properties, the launches went through
the C ABI, and the results agreed."""
from __future__ import annotations

import importlib
import os
import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent
BIN = ROOT / "gemm-zoo_amd" / "bench" / "bin"

# driver -> (lines expected, largest dimension let through)
DRIVERS = {
    # 256 .. 4096 of the reference's list (row-major B, alpha = beta = 1) and the 4096^3 headline (column-major B):
    # the functor constructors plan, launch and verify the 256 x 256 ring kernel from C++; 8192^3 is cut
    "bench_bf16_mma_gemm": (6, 4096),
    "bench_fp16_mma_gemm": (6, 4097),            # the same list and the ragged 4095 x 4097 x 1023
    "bench_xe_gemm_s8_s8_s32_m8k16": (3, 4096),  # 1024, 2048, 4096
    "bench_ladder": (18, 2048),                  # three type bundles x six rungs at 2048^3
    "bench_fp8_mma_gemm": (10, 4096),            # e4m3 and e5m2, 256 .. 4096
}


@pytest.mark.parametrize("driver", sorted(DRIVERS))
def test_cpp_driver_runs_and_verifies(driver):
    exe = BIN / driver
    if not exe.exists():
        pytest.fail(f"{exe} is not built (python gemm-zoo_amd/build.py builds the drivers)")
    want, max_dim = DRIVERS[driver]
    env = dict(os.environ, GZ_BENCH_MAX_DIM=str(max_dim), GZ_BENCH_REPS="2")
    print("running", driver, flush=True)
    proc = subprocess.run([str(exe)], env=env, capture_output=True, text=True, timeout=240)
    out = proc.stdout + proc.stderr
    assert proc.returncode == 0, out[-2000:]
    assert "verification failed" not in out and "HIP error" not in out, out[-2000:]
    lines = [l for l in proc.stdout.splitlines() if "GEMM Problem:" in l]
    assert len(lines) == want, out[-2000:]
    for l in lines:   # a time and a rate were measured
        ms = float(l.split("Time in ms:")[1].split("|")[0])
        assert 0.0 < ms < 1e4, l


def test_device_properties_give_a_plan():
    """What the C++ functor constructors do: plan with hipDeviceProp_t's compute-unit count and LDS size.  The
    256 x 256 MFMA tiles need all 160 KiB; a runtime that reported less would make every such constructor throw."""
    capi = importlib.import_module("gemm-zoo_amd.capi")
    F = importlib.import_module("gemm-zoo_amd.functors")
    cus, lds = capi.device_props()
    assert cus > 0 and lds >= 160 * 1024, (cus, lds)
    props = F.DeviceProps.current()
    assert (props.multiProcessorCount, props.maxSharedMemoryPerMultiProcessor) == (cus, lds)
    for types in (capi.S8S8S32, capi.BF16BF16F32, capi.BF16BF16BF16, capi.F16F16F16, capi.E4M3E4M3F16):
        p = capi.plan(types, 4096, 4096, 4096, capi.ROW_MAJOR, capi.COL_MAJOR, capi.RUNG_MFMA, 0, cus, lds)
        assert (p.tile_m, p.tile_n) == (256, 256) and p.lds_bytes <= lds
    k = F.functor("bf16_mma_gemm", "bf16", "f32", layout_b=capi.COL_MAJOR)(4096, 4096, 4096, props)
    assert k.plan.tile_m == 256
