"""MI355X (gfx950) GEMM kernel ladder behind gemm-zoo's kernel-functor surface.

``capi``      ctypes binding of the C ABI (``include/gemm_zoo.h``)
``functors``  host-side mirror of gemm-zoo's kernel functors
``harness``   host-side mirror of gemm-zoo's benchmark/verify harness
"""
from . import capi  # noqa: F401  (raises ImportError when the HIP library is not built)
