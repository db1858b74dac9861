// One decode step of attention over the packed cache and its fp16 residual tails, as a handful of
// launches on one stream:
//
//   1. logits over the quantized keys          kvmix_quantized_gemv (q.K^T), fp16 into the probability row
//   2. attn_tail_softmax                        logits over the fp16 key tail, then the softmax of the whole row
//   3. output over the quantized values         kvmix_quantized_gemv (p.V)
//   4. attn_tail_output                         p.V over the fp16 value tail, added to the result of 3
//
// The arithmetic follows the reference's decode branch (models/modeling_llama_KVmix.py:68-75,180-211):
// GEMV results and tail products are rounded to fp16 where the reference holds them in fp16 tensors,
// the row is scaled by 1/sqrt(D), an optional additive mask is applied and clamped to the lowest
// finite fp32, the softmax runs in fp32, probabilities are rounded to fp16, and the two halves of
// the output are added as fp16 values.
//
// The tails are windows of `*_tail_slots` tokens of which the first `len` hold tokens; `len` comes
// from the host or, for a step replayed from a captured graph, from device memory.  Slots past
// `len` get probability zero and are not read on the value side.
#include "kvmix_common.h"

namespace kvmix {

struct AttnArgs {
    const uint16_t *q;       // [samples, D]
    const uint16_t *k_tail;  // [samples / heads_per_kv, slots, D]
    const uint16_t *v_tail;
    uint16_t *probs;         // [samples, width]: logits of the quantized keys on entry to attn_tail_softmax
    uint16_t *out;           // [samples, D]
    const float *mask;       // optional [batch, width] additive mask, broadcast over heads
    const int64_t *k_len_dev, *v_len_dev;
    int64_t q_bs, kt_bs, kt_ts, vt_bs, vt_ts, p_bs, o_bs, mask_bs;
    int64_t k_tokens, v_tokens;  // quantized tokens
    int64_t k_slots, v_slots;    // tail window sizes
    int64_t k_len, v_len;        // live tail tokens (when the device pointers are null)
    int64_t width;               // entries of a probability row that take part in the softmax
    int heads_per_kv, heads, D;
    float inv_sqrt_d;
};

struct __attribute__((packed, aligned(2))) H8 {
    uint16_t v[8];
};

// One block per (batch, head).  The kernels are chains of short latency-bound phases, so with at
// most one row per CU the block is as wide as it can be (16 waves) to shorten each phase; with more
// rows than CUs, 8-wave blocks let two rows share a CU instead of queueing behind each other.
constexpr int kAttnThreadsWide = 1024;
constexpr int kAttnThreadsNarrow = 512;
constexpr int kAttnRowEntries = 16384;  // longest row the softmax keeps in registers

template <int THREADS>
__device__ __forceinline__ float block_reduce(float v, bool is_max, float *scratch)
{
    // THREADS / 64 waves; xor-shuffles inside the wave, then one value per wave through LDS
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float other = __shfl_xor(v, o);
        v = is_max ? fmaxf(v, other) : v + other;
    }
    const int wave = threadIdx.x / kWave;
    __syncthreads();  // (scratch may still be read from an earlier reduction)
    if (threadIdx.x % kWave == 0) scratch[wave] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < THREADS / kWave; w++) r = is_max ? fmaxf(r, scratch[w]) : r + scratch[w];
    return r;
}

// grid = samples.  Sixteen lanes share a tail token (eight head dimensions each) and every lane group
// has two tokens in flight, so a block covers 128 tail tokens per step.  The softmax keeps a row of up
// to 16384 entries in registers (two or four 8-entry vectors per thread): one read, one write.
constexpr int kTailUnroll = 2;

template <int THREADS>
__global__ void __launch_bounds__(THREADS) attn_tail_softmax(AttnArgs a)
{
    constexpr int kAttnThreads = THREADS, kAttnGroups = THREADS / 16, kRowVecs = kAttnRowEntries / (THREADS * 8);
    __shared__ float scratch[kAttnThreads / kWave];
    const int64_t sample = blockIdx.x;
    const int64_t kv = sample / a.heads_per_kv;
    const int tid = threadIdx.x;
    uint16_t *row = a.probs + sample * a.p_bs;
    // (a device-side counter that ran past the window is cut to it: nothing is read out of bounds)
    int64_t k_len = a.k_len_dev ? *a.k_len_dev : a.k_len;
    k_len = k_len < 0 ? 0 : (k_len > a.k_slots ? a.k_slots : k_len);
    const int D = a.D;

    // 1. logits of the tail window: row[k_tokens + j] = fp16(q . k_tail[j]) or -inf past the live tokens
    const int sub = tid % 16;
    const uint16_t *qp = a.q + sample * a.q_bs;
    const uint16_t *kt = a.k_tail + kv * a.kt_bs;
    for (int64_t j0 = 0; j0 < a.k_slots; j0 += kAttnGroups * kTailUnroll) {
        float dot[kTailUnroll] = {};
        for (int d = sub * 8; d < D; d += 128) {
            const H8 qq = *reinterpret_cast<const H8 *>(qp + d);
            H8 kk[kTailUnroll];
#pragma unroll
            for (int t = 0; t < kTailUnroll; t++) {
                const int64_t j = j0 + kAttnGroups * t + tid / 16;
                kk[t] = *reinterpret_cast<const H8 *>(kt + (j < k_len ? j : 0) * a.kt_ts + d);  // (slot 0 stands in past the end)
            }
#pragma unroll
            for (int t = 0; t < kTailUnroll; t++) {
#pragma unroll
                for (int i = 0; i < 8; i++) dot[t] = fmaf(h16_to_f32(qq.v[i]), h16_to_f32(kk[t].v[i]), dot[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < kTailUnroll; t++) {
#pragma unroll
            for (int o = 8; o >= 1; o >>= 1) dot[t] += __shfl_xor(dot[t], o);
            const int64_t j = j0 + kAttnGroups * t + tid / 16;
            if (sub == 0 && j < a.k_slots) row[a.k_tokens + j] = j < k_len ? f32_to_h16(dot[t]) : (uint16_t)0xfc00u;  // -inf
        }
    }
    // entries between the key window and the row's width (a value window that reaches further)
    for (int64_t i = a.k_tokens + a.k_slots + tid; i < a.width; i += kAttnThreads) row[i] = (uint16_t)0xfc00u;
    __syncthreads();

    // 2. softmax of the row in fp32: x = fp32(logit) / sqrt(D) (+ mask, clamped to the lowest finite value)
    const float *mrow = a.mask ? a.mask + (sample / a.heads) * a.mask_bs : nullptr;
    auto value = [&](int64_t i, uint16_t h) {
        float x = h16_to_f32(h) * a.inv_sqrt_d;
        if (mrow) x = fmaxf(x + mrow[i], -3.4028234663852886e38f);
        return x;
    };
    if (a.width <= (int64_t)kAttnThreads * 8 * kRowVecs) {
        // thread t holds entries 8*(kAttnThreads*v + t) .. +7 of vector round v; a ragged end is read entry by entry
        float x[kRowVecs][8];
#pragma unroll
        for (int v = 0; v < kRowVecs; v++) {
            const int64_t i0 = ((int64_t)v * kAttnThreads + tid) * 8;
            if (i0 + 8 <= a.width) {
                const H8 h = *reinterpret_cast<const H8 *>(row + i0);
#pragma unroll
                for (int i = 0; i < 8; i++) x[v][i] = value(i0 + i, h.v[i]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) x[v][i] = i0 + i < a.width ? value(i0 + i, row[i0 + i]) : -INFINITY;
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < kRowVecs; v++) {
#pragma unroll
            for (int i = 0; i < 8; i++) mx = fmaxf(mx, x[v][i]);
        }
        mx = block_reduce<THREADS>(mx, true, scratch);
        float sum = 0.f;
#pragma unroll
        for (int v = 0; v < kRowVecs; v++) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                x[v][i] = expf(x[v][i] - mx);
                sum += x[v][i];
            }
        }
        sum = block_reduce<THREADS>(sum, false, scratch);
#pragma unroll
        for (int v = 0; v < kRowVecs; v++) {
            const int64_t i0 = ((int64_t)v * kAttnThreads + tid) * 8;
            if (i0 + 8 <= a.width) {
                H8 h;
#pragma unroll
                for (int i = 0; i < 8; i++) h.v[i] = f32_to_h16(x[v][i] / sum);
                *reinterpret_cast<H8 *>(row + i0) = h;
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    if (i0 + i < a.width) row[i0 + i] = f32_to_h16(x[v][i] / sum);
                }
            }
        }
        return;
    }
    // longer rows: three passes over the row (it stays in L2)
    float mx = -INFINITY;
    for (int64_t i = tid; i < a.width; i += kAttnThreads) mx = fmaxf(mx, value(i, row[i]));
    mx = block_reduce<THREADS>(mx, true, scratch);
    float sum = 0.f;
    for (int64_t i = tid; i < a.width; i += kAttnThreads) sum += expf(value(i, row[i]) - mx);
    sum = block_reduce<THREADS>(sum, false, scratch);
    for (int64_t i = tid; i < a.width; i += kAttnThreads) row[i] = f32_to_h16(expf(value(i, row[i]) - mx) / sum);
}

// grid = samples: thread t owns head dimensions 8*(t%16).. of the tokens t/16, t/16 + 64, ...
// out = fp16( fp16(out from the quantized values) + fp16(sum_j p[v_tokens + j] * v_tail[j]) )
template <int THREADS>
__global__ void __launch_bounds__(THREADS) attn_tail_output(AttnArgs a)
{
    constexpr int kAttnGroups = THREADS / 16;
    __shared__ float part[kAttnGroups][129];
    const int64_t sample = blockIdx.x;
    const int64_t kv = sample / a.heads_per_kv;
    const int tid = threadIdx.x;
    const int sub = tid % 16, grp = tid / 16;
    int64_t v_len = a.v_len_dev ? *a.v_len_dev : a.v_len;
    v_len = v_len < 0 ? 0 : (v_len > a.v_slots ? a.v_slots : v_len);
    const uint16_t *prow = a.probs + sample * a.p_bs + a.v_tokens;
    const uint16_t *vt = a.v_tail + kv * a.vt_bs;
    uint16_t *op = a.out + sample * a.o_bs;
    for (int d0 = 0; d0 < a.D; d0 += 128) {
        const int d = d0 + sub * 8;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (d < a.D) {
            for (int64_t j0 = grp; j0 < v_len; j0 += kAttnGroups * kTailUnroll) {
                float p[kTailUnroll];
                H8 vv[kTailUnroll];
#pragma unroll
                for (int t = 0; t < kTailUnroll; t++) {
                    const int64_t j = j0 + kAttnGroups * t;
                    const bool in = j < v_len;
                    p[t] = in ? h16_to_f32(prow[j]) : 0.f;
                    vv[t] = *reinterpret_cast<const H8 *>(vt + (in ? j : j0) * a.vt_ts + d);
                }
#pragma unroll
                for (int t = 0; t < kTailUnroll; t++) {
#pragma unroll
                    for (int i = 0; i < 8; i++) acc[i] = fmaf(p[t], h16_to_f32(vv[t].v[i]), acc[i]);
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; i++) part[grp][sub * 8 + i] = acc[i];
        __syncthreads();
        if (tid < 128 && d0 + tid < a.D) {
            float s = 0.f;
#pragma unroll
            for (int g = 0; g < kAttnGroups; g++) s += part[g][tid];
            const float tail = h16_to_f32(f32_to_h16(s));
            const float quant = a.v_tokens > 0 ? h16_to_f32(op[d0 + tid]) : 0.f;
            op[d0 + tid] = f32_to_h16(quant + tail);
        }
    }
}

}  // namespace kvmix

using namespace kvmix;

static int64_t attn_width(const kvmix_decode_attn_t *p)
{
    const int64_t a = p->k_tokens + p->k_tail_slots, b = p->v_tokens + p->v_tail_slots;
    return a > b ? a : b;
}

extern "C" size_t kvmix_decode_attention_workspace_bytes(const kvmix_decode_attn_t *p)
{
    if (!p || p->v_tokens <= 0) return 0;
    return kvmix_gemv_workspace_bytes(p->samples, 1, p->v_tokens, p->D);
}

extern "C" int kvmix_decode_attention(const kvmix_decode_attn_t *p, void *workspace, size_t workspace_bytes,
                                      kvmix_stream_t stream)
{
    if (!p) return KVMIX_ERR_NULL;
    if (p->samples < 0 || p->D <= 0 || p->k_tokens < 0 || p->v_tokens < 0 || p->k_tail_slots < 0 || p->v_tail_slots < 0 ||
        p->k_tail_len < 0 || p->v_tail_len < 0 || p->k_tail_len > p->k_tail_slots || p->v_tail_len > p->v_tail_slots)
        return KVMIX_ERR_SHAPE;
    if (p->heads_per_kv <= 0 || p->samples % p->heads_per_kv != 0) return KVMIX_ERR_HEADS;
    if (p->heads <= 0 || p->samples % p->heads != 0) return KVMIX_ERR_HEADS;
    if (p->D % 8 != 0) return KVMIX_ERR_UNSUPPORTED;
    if (p->samples == 0) return KVMIX_OK;
    const int64_t width = attn_width(p);
    if (width == 0) return KVMIX_ERR_SHAPE;  // nothing to attend to
    if (!p->k_tail_len_dev && !p->v_tail_len_dev && p->k_tokens + p->k_tail_len != p->v_tokens + p->v_tail_len)
        return KVMIX_ERR_SHAPE;  // keys and values must cover the same positions
    if (!p->q || !p->probs || !p->out) return KVMIX_ERR_NULL;
    if ((p->k_tail_slots > 0 && !p->k_tail) || (p->v_tail_slots > 0 && !p->v_tail)) return KVMIX_ERR_NULL;
    if (p->probs_stride < width || p->out_stride < p->D || p->q_stride < p->D || (p->mask && p->mask_stride < width))
        return KVMIX_ERR_SHAPE;
    if ((p->k_tail_slots > 0 && p->k_tail_token_stride < p->D) || (p->v_tail_slots > 0 && p->v_tail_token_stride < p->D))
        return KVMIX_ERR_SHAPE;

    if (p->k_tokens > 0) {
        const int rc = kvmix_quantized_gemv(p->k_group, p->q, p->q_stride, p->q_stride, p->k_code, p->k_code_batch_stride,
                                            p->k_code_row_stride, p->k_scale, p->k_zero, p->k_sz_batch_stride,
                                            p->k_sz_row_stride, p->k_bits, p->k_fmt, p->samples, p->heads_per_kv, 1, p->D,
                                            p->k_tokens, p->probs, p->probs_stride, p->probs_stride, nullptr, 0, stream);
        if (rc != KVMIX_OK) return rc;
    }
    AttnArgs a;
    a.q = (const uint16_t *)p->q;
    a.k_tail = (const uint16_t *)p->k_tail;
    a.v_tail = (const uint16_t *)p->v_tail;
    a.probs = (uint16_t *)p->probs;
    a.out = (uint16_t *)p->out;
    a.mask = p->mask;
    a.k_len_dev = p->k_tail_len_dev;
    a.v_len_dev = p->v_tail_len_dev;
    a.q_bs = p->q_stride;
    a.kt_bs = p->k_tail_batch_stride;
    a.kt_ts = p->k_tail_token_stride;
    a.vt_bs = p->v_tail_batch_stride;
    a.vt_ts = p->v_tail_token_stride;
    a.p_bs = p->probs_stride;
    a.o_bs = p->out_stride;
    a.mask_bs = p->mask_stride;
    a.k_tokens = p->k_tokens;
    a.v_tokens = p->v_tokens;
    a.k_slots = p->k_tail_slots;
    a.v_slots = p->v_tail_slots;
    a.k_len = p->k_tail_len;
    a.v_len = p->v_tail_len;
    a.width = width;
    a.heads_per_kv = p->heads_per_kv;
    a.heads = p->heads;
    a.D = (int)p->D;
    a.inv_sqrt_d = 1.0f / sqrtf((float)p->D);
    hipStream_t st = (hipStream_t)stream;
    if (p->samples > 0x7fffffff) return KVMIX_ERR_SHAPE;
    const bool narrow = p->samples > 256;  // more rows than CUs
    if (narrow) hipLaunchKernelGGL(attn_tail_softmax<kAttnThreadsNarrow>, dim3((unsigned)p->samples), dim3(kAttnThreadsNarrow), 0, st, a);
    else hipLaunchKernelGGL(attn_tail_softmax<kAttnThreadsWide>, dim3((unsigned)p->samples), dim3(kAttnThreadsWide), 0, st, a);
    int rc = launch_status();
    if (rc != KVMIX_OK) return rc;
    if (p->v_tokens > 0) {
        rc = kvmix_quantized_gemv(p->v_group, p->probs, p->probs_stride, p->probs_stride, p->v_code, p->v_code_batch_stride,
                                  p->v_code_row_stride, p->v_scale, p->v_zero, p->v_sz_batch_stride, p->v_sz_row_stride,
                                  p->v_bits, p->v_fmt, p->samples, p->heads_per_kv, 1, p->v_tokens, p->D, p->out,
                                  p->out_stride, p->out_stride, workspace, workspace_bytes, stream);
        if (rc != KVMIX_OK) return rc;
    }
    if (narrow) hipLaunchKernelGGL(attn_tail_output<kAttnThreadsNarrow>, dim3((unsigned)p->samples), dim3(kAttnThreadsNarrow), 0, st, a);
    else hipLaunchKernelGGL(attn_tail_output<kAttnThreadsWide>, dim3((unsigned)p->samples), dim3(kAttnThreadsWide), 0, st, a);
    return launch_status();
}
