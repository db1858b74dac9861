"""Drop-in for the reference's compiled extension module `KVmix`
(quant_cuda/csrc/pybind.cpp:6-15): `import KVmix` in models/modeling_llama_KVmix.py:9 and
models/modeling_mistral_KVmix.py:37 resolves here when the repository root is on sys.path."""
from kvmix_amd.ops import (process_key_quantization_cuda, process_value_quantization_cuda,
                           quantize_pack_last_dim_cuda, quantized_gemm)

__all__ = [
    "quantized_gemm",
    "quantize_pack_last_dim_cuda",
    "process_value_quantization_cuda",
    "process_key_quantization_cuda",
]
