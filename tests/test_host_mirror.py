"""Host-side mirror of the reference's functor surface: instantiation, planning, rejection (no GPU needed)."""
import importlib

import pytest


@pytest.fixture(scope="module")
def F(gz):
    return importlib.import_module("gemm-zoo_amd.functors")


def test_functor_instantiation_follows_the_reference_names(F, capi):
    names = ["naive_gemm", "generic_gemm", "smem_tiled_gemm", "rmem_tiled_gemm", "double_buffered_gemm",
             "async_buffered_gemm", "bf16_mma_gemm", "gemm_bf16_bf16_f32_m8k16"]
    for name in names:
        K = F.functor(name, "bf16", "f32", 128, 128, 32)
        k = K(1024, 1024, 1024, F.DeviceProps())
        assert k.plan.grid >= 1 and K.types == capi.BF16BF16F32 and name in K.__name__
    assert F.functor("fp16_mma_gemm", "f16", "f16", 256, 256, 32).types == capi.F16F16F16
    assert F.functor("gemm_s8_s8_s32_m8k16", "s8", "s32").types == capi.S8S8S32
    assert F.functor("gemm_bf16_bf16_bf16_m8k16", "bf16", "bf16").types == capi.BF16BF16BF16
    # the reference's own ladder drivers are fp32 (nvidia/bench/bench_naive.cu:9-17, bench_tf32_mma_gemm.cu:9-26)
    assert F.functor("tf32_mma_gemm", "f32", "f32", 128, 128, 32).types == capi.F32F32F32
    assert F.functor("naive_gemm", "f32", "f32")(128, 128, 128).plan.rung == capi.RUNG_NAIVE
    with pytest.raises(KeyError):
        F.functor("fp4_mma_gemm", "f32", "f32")        # no such functor
    with pytest.raises(KeyError):
        F.functor("naive_gemm", "bf16", "s32")


def test_constructor_plans_like_the_reference_constructors(F, capi):
    # the tile integers of the reference's drivers are a hint: the launcher picks the gfx950 tile
    k = F.functor("bf16_mma_gemm", "bf16", "f32", 128, 128, 32, layout_b=F.COL)(4096, 4096, 4096)
    assert (k.plan.rung, k.plan.tile_m, k.plan.tile_n, k.plan.grid) == (capi.RUNG_MFMA, 256, 256, 256)
    # a pinned variant is honoured
    k = F.functor("bf16_mma_gemm", "bf16", "f32", variant=3)(4096, 4096, 4096)
    assert (k.plan.tile_m, k.plan.tile_n) == (128, 128)
    # generic_gemm is the any-shape fallback: 64x64 tiles, ceil-div grid
    k = F.functor("generic_gemm", "f16", "f16")(100, 130, 7)
    assert k.plan.rung == capi.RUNG_LDS_TILED and k.plan.grid == 2 * 3
    # the typed entry point routes decode shapes to the streaming kernel
    k = F.functor("gemm_bf16_bf16_bf16_m8k16", "bf16", "bf16", layout_b=F.COL)(8, 14336, 4096)
    assert k.plan.rung == capi.RUNG_SKINNY
    # fewer compute units: the big tile is kept only while it still covers the device
    small = F.functor("bf16_mma_gemm", "bf16", "f32")(1024, 1024, 1024, F.DeviceProps(multiProcessorCount=16))
    assert small.plan.tile_m == 256


def test_constructor_rejects_what_the_rung_cannot_run(F, capi):
    with pytest.raises(capi.GzError) as e:
        F.functor("skinny_gemm", "bf16", "bf16", layout_b=F.COL)(129, 128, 128)
    assert e.value.status == capi.ERR_UNSUPPORTED
    with pytest.raises(capi.GzError):
        F.functor("naive_gemm", "bf16", "f32")(-1, 4, 4)
    with pytest.raises(capi.GzError):
        F.functor("bf16_mma_gemm", "bf16", "f32", variant=99)(256, 256, 256)
    # a failing call surfaces the C ABI's status (NULL operands here) without touching a device
    k = F.functor("naive_gemm", "bf16", "f32")(4, 4, 4)
    with pytest.raises(capi.GzError) as e:
        k(0, 0, 0, 0, 1.0, 0.0)
    assert e.value.status == capi.ERR_BAD_ARG


def test_comparator_library_exports(F):
    import ctypes
    import re
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    text = re.sub(r"/\*.*?\*/", "", (root / "include" / "gemm_zoo_hipblaslt.h").read_text(), flags=re.S)
    names = sorted(set(re.findall(r"\b(gz_hipblaslt_[a-z_]+)\s*\(", text)))
    assert names == ["gz_hipblaslt_create", "gz_hipblaslt_destroy", "gz_hipblaslt_last_error", "gz_hipblaslt_run"]
    lib = F.HipblasLtGemm.lib()
    for n in names:
        assert hasattr(lib, n)
    plan = ctypes.c_void_p()
    assert lib.gz_hipblaslt_create(9, 4, 4, 4, 0, 0, ctypes.byref(plan)) == 1  # bad type bundle, no device touched
    assert lib.gz_hipblaslt_create(7, 4, 4, 4, 0, 0, ctypes.byref(plan)) == 2  # 16-bit running sums: not in the library
