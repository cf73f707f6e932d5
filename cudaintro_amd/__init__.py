"""MI355X (gfx950) quantization-GEMM library: Python bindings over the C ABI.

The product is ``libcigemm.so`` (hand-written HIP kernels behind ``include/cigemm.h``) and
the C++ suite driver ``gemm_suite``.  This package only binds the C ABI with ctypes so that
tests and the benchmark can call it; PyTorch supplies device memory and streams.
There is no CPU fallback: importing works anywhere, but creating a handle needs the built
library and a gfx950 device.
"""
from .cigemm import (  # noqa: F401
    ACT_NONE,
    ACT_RELU,
    ALGO_DEFAULT,
    ALGO_GENERIC,
    ALGO_SKINNY,
    ALGO_SMALL,
    ALGO_TILE,
    ALGO_MFMA_ANY,
    B_KN,
    B_NK,
    OUT_BF16,
    OUT_F32,
    SCALE_TENSOR,
    SCALE_VECTOR,
    CigemmError,
    Handle,
    Status,
    build_library,
    gemm_bf16_static,
    library_path,
    load_library,
    suite_path,
)
