"""MI355X-native dequantize-GEMM kernels behind the call surface of TileLang's examples.

Hand-written gfx950 HIP kernels in ``libdqgemm.so`` (C-ABI: ``include/dqgemm.h``), a thin
ctypes adapter with the reference adapter's call contract, and factories named after the
examples' kernels.  PyTorch is used for tensors and streams only.
"""

from . import quantize  # noqa: F401
from .adapter import KernelAdapter, KernelParam  # noqa: F401
from .kernels import (  # noqa: F401
    bitlinear_int8xint2,
    bitnet_158_int8xint2_decode,
    bitnet_activation_quant,
    bitnet_158_int8xint2_prefill,
    dequantize_gemv,
    dequantize_w4,
    matmul_bf16_fp4,
    matmul_bf16_mxfp4,
    matmul_mxfp4_mxfp4,
    matmul_fp16_fp4,
    matmul_int8xint4,
    matmul,
    matmul_nt_int4,
    matmul_nt_int4xint2,
    matmul_w4_fine_grained,
    matmul_w4a16,
    quantize_bf16_mxfp4,
)
from .bitlinear import BitLinear  # noqa: F401
from .w4linear import W4A16Linear  # noqa: F401
from .profiler import Profiler, TensorSupplyType, do_bench  # noqa: F401

__version__ = "0.1.0"
