// Version and error text of the C ABI.  The argument-error texts are the ones the
// reference raises through TORCH_CHECK for the same condition
// (quant_cuda/csrc/quantization_cuda.cu:318-321,433-436,638,644,649,652,687;
//  quant_cuda/csrc/dequantization_gemv_cuda.cu:136,174-178,203).
#include "kvmix_common.h"

extern "C" int kvmix_version(void) { return 100; }

extern "C" const char *kvmix_strerror(int code)
{
    switch (code) {
    case KVMIX_OK: return "ok";
    case KVMIX_ERR_BITS: return "Supported quantization bits: 1, 2, 3, 4";
    case KVMIX_ERR_GROUP3: return "For 3-bit quantization, group_length must be 11";
    case KVMIX_ERR_STEPS_GROUP: return "steps must be divisible by group_length";
    case KVMIX_ERR_STEPS_WORD: return "steps must be divisible by (32 / quant_bits)";
    case KVMIX_ERR_HEADS: return "Total heads must be divisible by KV heads";
    case KVMIX_ERR_DTYPE: return "unsupported dtype: expected float16 or float32";
    case KVMIX_ERR_NULL: return "null pointer argument";
    case KVMIX_ERR_SHAPE: return "negative size, or a stride smaller than the row it spans";
    case KVMIX_ERR_UNSUPPORTED: return "group size and codes-per-word combination is not expressible in the packed layout";
    case KVMIX_ERR_FORMAT: return "unknown packed format or scale mode";
    case KVMIX_ERR_WORKSPACE: return "workspace is smaller than kvmix_gemv_workspace_bytes()";
    case KVMIX_ERR_LAUNCH: return "kernel launch failed";
    case KVMIX_ERR_STATIC_SCRATCH:
        return "problem needs more split-K scratch than kvmix_quantized_gemv_static's built-in buffer holds "
               "(KVMIX_GEMV_STATIC_SCRATCH_BYTES): use kvmix_quantized_gemv with a caller-owned workspace";
    case KVMIX_ERR_STATIC_LOOKUP:
        return "the address of kvmix_quantized_gemv_static's built-in buffer could not be obtained on this device "
               "(hipGetSymbolAddress failed): use kvmix_quantized_gemv with a caller-owned workspace";
    default: return "unknown kvmix error";
    }
}
