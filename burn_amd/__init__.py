"""burn_amd: burn's quantized-tensor hot path (quantize / quantize_dynamic / dequantize / q_matmul)
as hand-written gfx950 HIP kernels behind a C ABI (include/burnq.h, libburnq_mi355.so).

The Python layer is a thin ctypes mirror of the reference's operator interface:

    from burn_amd import Device, FloatOps, QTensorOps, QuantScheme, QuantValue, QuantStore

Importing the package does not load the library; the first operation does, and fails loudly if
the shared object has not been built (`python -m burn_amd.build`).
"""
from ._lib import BF16, F32, I32, I64, QFLOAT, BurnqError
from .ops import (Device, FloatOps, IntOps, ModuleOps, PackReader, PackWriter, QTensorOps, Tensor, TensorData, bf16_bits_from_f32,
                  f32_from_bf16_bits)
from .quantization import QuantScheme, QuantStore, QuantValue, ScaleDtype, params_shape

__all__ = [
    "BF16", "F32", "I32", "I64", "QFLOAT", "BurnqError", "Device", "FloatOps", "IntOps", "ModuleOps", "PackReader", "PackWriter", "QTensorOps", "Tensor",
    "TensorData", "QuantScheme", "QuantStore", "QuantValue", "ScaleDtype", "params_shape",
    "bf16_bits_from_f32", "f32_from_bf16_bits",
]
