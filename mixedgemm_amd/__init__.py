"""MI355X-native reorder-quantize + mixed MXFP4/6/8 GEMM.

`mixedgemm_amd.abi` binds the C-ABI of lib/libmixedgemm_hip.so with ctypes;
`build/mixedgemm.so` (see mixedgemm_amd.build) is the torch extension with the
reference's operator surface.
"""
from . import abi  # noqa: F401
from .abi import (  # noqa: F401
    MixedGemmError, fused_linear, matmul, reorder_quantize_w, reorder_quantize_x, sf_bytes,
)
