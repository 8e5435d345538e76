"""MI355X-native (gfx950) implementation of candle's GGUF quantized-matmul path.

Public surface (mirrors candle-core/src/quantized/mod.rs and candle-nn/src/moe.rs):
``GgmlDType``, ``QStorage``, ``QTensor``, ``QMatMul``, ``moe_gemm_gguf``; ``gguf_file`` mirrors
candle-core/src/quantized/gguf_file.rs.
"""
from . import gguf_file  # noqa: F401
from .quantized import GgmlDType, QMatMul, QStorage, QTensor, check_shape, moe_gemm_gguf  # noqa: F401

__all__ = ["GgmlDType", "QStorage", "QTensor", "QMatMul", "moe_gemm_gguf", "check_shape", "gguf_file"]
