"""kvmix_amd: the KVmix KV-cache hot path (group quantize + bit-pack on append, fused
dequantize-GEMV for q.K^T and p.V) as hand-written gfx950 HIP kernels behind a C ABI."""
from .ops import (process_key_quantization_cuda, process_value_quantization_cuda,
                  quantize_pack_last_dim_cuda, quantized_gemm)

from .cache import PackedKVCache  # noqa: E402

__all__ = [
    "PackedKVCache",
    "quantize_pack_last_dim_cuda",
    "quantized_gemm",
    "process_key_quantization_cuda",
    "process_value_quantization_cuda",
]
