// Shared host/device helpers for the gfx950 KVmix kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kvmix_hip.h"

namespace kvmix {

constexpr int kWave = 64;  // CDNA wavefront width

__host__ __device__ constexpr int values_per_word(int bits) { return bits == 3 ? 11 : 32 / bits; }

// float -> fp16 bits, round to nearest even (v_cvt_f16_f32)
__device__ __forceinline__ uint16_t f32_to_h16(float v)
{
    return __half_as_ushort(__float2half_rn(v));
}

__device__ __forceinline__ float h16_to_f32(uint16_t h)
{
    return __half2float(__ushort_as_half(h));
}

// clamp(roundf((x - mn) / scale), 0, hi) with IEEE fp32 division.  A NaN quotient
// (constant group: 0/0) converts to 0, like the reference's float->int conversion.
__device__ __forceinline__ uint32_t quantize_code(float x, float mn, float scale, int hi)
{
    float normalized = (x - mn) / scale;
    float r = roundf(normalized);  // ties away from zero
    int q = (r != r) ? 0 : (r >= 2147483648.0f ? 0x7fffffff : (r <= -2147483648.0f ? (int)0x80000000 : (int)r));
    q = q > hi ? hi : q;
    q = q < 0 ? 0 : q;
    return (uint32_t)q;
}

// scale returned to the caller; the codes always use the true division.
__device__ __forceinline__ float scale_for_output(float range, float scale_div, float inv_qmax, int scale_mode)
{
    return scale_mode == KVMIX_SCALE_RECIPROCAL ? range * inv_qmax : scale_div;
}

inline int launch_status()
{
    return hipGetLastError() == hipSuccess ? KVMIX_OK : KVMIX_ERR_LAUNCH;
}

}  // namespace kvmix
