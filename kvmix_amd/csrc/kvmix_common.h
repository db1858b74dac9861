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

// The same code without a division per element.  rcp approximates 1/scale (v_rcp_f32, 1 ulp), so
// t = (x - mn) * rcp is within a few ulp of the true quotient -- for quotients up to 15 that is
// below 1e-5 -- and the IEEE quotient rounds to the same integer as t unless t lies within that
// distance of a tie k + 0.5.  Only then (margin 2^-12), or when t is not an ordinary number
// (constant group: 0 * inf), the exact path runs.  Bit-identical to quantize_code.
// rcp for the division-free quantize_code below; NaN (= always take the exact path) when the
// scale is so small or large that the reciprocal leaves the range where v_rcp_f32 is 1 ulp
__device__ __forceinline__ float quantize_rcp(float scale)
{
    return (scale > 1e-30f && scale < 1e30f) ? __builtin_amdgcn_rcpf(scale) : __builtin_nanf("");
}

__device__ __forceinline__ uint32_t quantize_code(float x, float mn, float scale, float rcp, int hi)
{
    const float t = (x - mn) * rcp;
    const float fl = floorf(t);
    const float fr = t - fl;
    if (__builtin_expect(!(fabsf(fr - 0.5f) >= 0.000244140625f) || !(fabsf(t) < 1024.0f), 0))
        return quantize_code(x, mn, scale, hi);
    int q = (int)fl + (fr > 0.5f ? 1 : 0);
    q = q > hi ? hi : q;
    q = q < 0 ? 0 : q;
    return (uint32_t)q;
}

// The cheapest form, for the quantizers' inner loops: u = (x - mn) * rcp + 0.5 and the code is min(trunc(u), hi)
// (x >= mn inside its own group, so u >= 0.5; the conversion saturates).  u is within 3e-6 of the true
// quotient + 0.5 for quotients up to 15 (reciprocal 1 ulp, one rounding of the fused multiply-add), so the
// truncation is the division's rounding unless u lies within 2^-15 of an integer or is not a number (constant
// group, infinities, NaN): then `near` is raised and quantize_codes below redoes its values with the division.
__device__ __forceinline__ uint32_t quantize_code_fast(float x, float mn, float rcp, int hi, bool &near)
{
    const float u = fmaf(x - mn, rcp, 0.5f);
    const float f = __builtin_amdgcn_fractf(u);
    near |= !(fabsf(f - 0.5f) <= 0.5f - 0.000030517578125f);
    const uint32_t q = (uint32_t)u;
    return q > (uint32_t)hi ? (uint32_t)hi : q;
}

// codes of N values of one group (hi(t): the largest code of value t): seven vector instructions per value and
// one branch per call, bit-identical to quantize_code(x, mn, scale, hi)
template <int N, typename Hi>
__device__ __forceinline__ void quantize_codes(const float *v, float mn, float scale, float rcp, Hi hi, uint32_t *q)
{
    bool near = false;
#pragma unroll
    for (int t = 0; t < N; t++) q[t] = quantize_code_fast(v[t], mn, rcp, hi(t), near);
    if (__builtin_expect(near, 0)) {
#pragma unroll
        for (int t = 0; t < N; t++) q[t] = quantize_code(v[t], mn, scale, hi(t));
    }
}

// scale returned to the caller; the codes always use the true division.
__device__ __forceinline__ float scale_for_output(float range, float scale_div, float inv_qmax, int scale_mode)
{
    return scale_mode == KVMIX_SCALE_RECIPROCAL ? range * inv_qmax : scale_div;
}

// Halving butterfly over lanes.  v[0..NV) of every lane are summed across the lanes whose
// indices differ in the bits {FIRST, 2*FIRST, ...} (UP = 1: up to bit 32; UP = 0: FIRST, FIRST/2,
// ... down to bit 1).  A step halves what a lane holds: the lane with the step's bit clear
// keeps the lower half, its partner the upper half.  Returns the index (in the original
// numbering) of the value left in v[0]; the lane's remaining values follow it in order.
template <int NV, int FIRST, int UP>
__device__ __forceinline__ int scatter_reduce(float *v, int lane)
{
    if constexpr (NV <= 1 || FIRST < 1 || FIRST >= kWave) {
        return 0;
    } else {
        constexpr int H = NV / 2;
        const bool up = (lane & FIRST) != 0;
#pragma unroll
        for (int i = 0; i < H; i++) {
            const float keep = up ? v[H + i] : v[i];
            const float send = up ? v[i] : v[H + i];
            v[i] = keep + __shfl_xor(send, FIRST);
        }
        return (up ? H : 0) + scatter_reduce<H, UP ? FIRST * 2 : FIRST / 2, UP>(v, lane);
    }
}

// The matrix-core tiles of the single-pass decode step (attn_step_mfma in dequant_gemv.hip, launched for
// kvmix_decode_attention_fused in fused_attn.hip): the quantized positions [0, tokens) of keys and values alike.
struct AttnSlabArgs {
    const uint16_t *q;        // [samples, 128] fp16
    int64_t q_bs;
    const uint32_t *k_code;   // [kv samples, 128, words], groups of 32 positions
    const uint16_t *k_scale, *k_zero;
    int64_t kc_bs, kc_rs, ksz_bs, ksz_rs;
    const uint32_t *v_code;   // [kv samples, tokens, 128 * bits / 32], dense rows
    const uint16_t *v_scale, *v_zero;
    int64_t vc_bs, vsz_bs;
    const float *mask;        // optional [batch, width]
    int64_t mask_bs;
    float *ws_o, *ws_ml;      // [samples, slabs, 128] partial outputs, [samples, slabs, 2] slab maximum and sum
    int64_t tokens;           // a multiple of 32, at least 1024
    int heads_per_kv, heads;  // query heads per kv head; query heads per batch entry (for the mask row)
    int slabs;                // slabs of a row in the workspace (these tiles first, the tail's slabs after them)
    float inv_sqrt_d;
};
inline int launch_status()
{
    return hipGetLastError() == hipSuccess ? KVMIX_OK : KVMIX_ERR_LAUNCH;
}

}  // namespace kvmix
