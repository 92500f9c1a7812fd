"""hecbench_amd — MI355X-native weight-only quantized-inference kernels.

Host-side mirror of the HeCBench launch wrappers (quant3MatMul, lut-gemm,
quantAQLM, quantBnB) on top of the C-ABI library libhq.so.  Tensors are
torch CUDA(HIP) tensors used purely as device buffers; all arithmetic happens in
the hand-written HIP kernels behind the ABI.
"""
from . import _lib
from ._lib import HqError, EXPORTED_SYMBOLS, LIB_PATH
from .ops import (
    NF4, FP4,
    vecquant3matmul, vecquant3matmul_faster, q3_matvec, q3_gemm,
    dequant_4bit, quantize_dynamic8, dynamic_map, lut_matmul, code1x16_matvec,
    device_info, init, q3_pack, bcq_pack, quantize_4bit,
    static_scaled_int8_quant, dynamic_scaled_int8_quant,
    gemv_fp16, gemv_int8, gemv_int4, mxfp4_qdq,
)

__all__ = [
    "HqError", "EXPORTED_SYMBOLS", "LIB_PATH", "NF4", "FP4",
    "vecquant3matmul", "vecquant3matmul_faster", "q3_matvec", "q3_gemm",
    "dequant_4bit", "quantize_dynamic8", "dynamic_map", "lut_matmul", "code1x16_matvec",
    "device_info", "init", "q3_pack", "bcq_pack", "quantize_4bit",
    "static_scaled_int8_quant", "dynamic_scaled_int8_quant",
    "gemv_fp16", "gemv_int8", "gemv_int4", "mxfp4_qdq",
]
