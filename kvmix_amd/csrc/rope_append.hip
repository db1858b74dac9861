// The tail append of a decode step, fused with the rotary embedding that precedes it: one launch
// takes the fused q/k/v projection of the new token, rotates the query and key heads, writes the
// query heads to their own tensor and the key and value heads straight into the next free slot of
// the fp16 tail windows of the cache.  It replaces what models/modeling_llama_KVmix.py:102-112 does
// with apply_rotary_pos_emb (five elementwise kernels) and two torch.cat calls.
//
// Arithmetic: x * cos + rotate_half(x) * sin evaluated as the fp16 tensor expression evaluates it --
// each product rounded to fp16, then the sum rounded to fp16 -- so the result is bit-identical to
// the torch composition.
#include "kvmix_common.h"

namespace kvmix {

struct RopeArgs {
    const uint16_t *qkv;   // [batch, heads + 2 * kv_heads, D]
    const uint16_t *cos, *sin;  // [D]
    uint16_t *q_out;       // [batch, heads, D]
    uint16_t *k_tail, *v_tail;  // [batch, kv_heads, slots, D]
    const int64_t *k_slot_dev, *v_slot_dev;
    int64_t qkv_bs, q_bs, kt_bs, kt_hs, kt_ts, vt_bs, vt_hs, vt_ts;
    int64_t k_slots, v_slots, k_slot, v_slot;
    int64_t rows;          // batch * (heads + 2 * kv_heads)
    int heads, kv_heads, D;
};

struct __attribute__((packed, aligned(2))) R8 {
    uint16_t v[8];
};

constexpr int kRopeThreads = 256;

// The products are pinned in registers as fp16 bit patterns before they are added: left to itself
// the compiler contracts fp16 product + sum into one mixed-precision fma, and the product's rounding
// to fp16 -- which the tensor expression has -- is lost.
__device__ __forceinline__ float rounded_product(float a, float b)
{
    uint32_t bits = f32_to_h16(a * b);
    asm volatile("" : "+v"(bits));
    return h16_to_f32((uint16_t)bits);
}

__device__ __forceinline__ uint16_t rope_one(uint16_t x, uint16_t other, uint16_t c, uint16_t s, bool negate_other)
{
    const float a = rounded_product(h16_to_f32(x), h16_to_f32(c));
    const float o = negate_other ? -h16_to_f32(other) : h16_to_f32(other);
    const float b = rounded_product(o, h16_to_f32(s));
    return f32_to_h16(a + b);
}

// D / 16 threads per (batch, head) row: a thread owns eight elements of the first half of the head
// dimension and the eight that rotate_half pairs them with.
__global__ void __launch_bounds__(kRopeThreads) rope_append(RopeArgs a)
{
    const int per_row = a.D / 16;
    const int64_t t = (int64_t)blockIdx.x * kRopeThreads + threadIdx.x;
    const int64_t row = t / per_row;
    const int part = (int)(t % per_row);
    if (row >= a.rows) return;
    const int total = a.heads + 2 * a.kv_heads;
    const int64_t b = row / total;
    const int h = (int)(row % total);
    const int half = a.D / 2;
    const uint16_t *src = a.qkv + b * a.qkv_bs + (int64_t)h * a.D + part * 8;
    const R8 x1 = *reinterpret_cast<const R8 *>(src);
    const R8 x2 = *reinterpret_cast<const R8 *>(src + half);
    uint16_t *dst;
    bool rotate = true;
    if (h < a.heads) {
        dst = a.q_out + b * a.q_bs + (int64_t)h * a.D;
    } else if (h < a.heads + a.kv_heads) {
        const int64_t slot = a.k_slot_dev ? *a.k_slot_dev : a.k_slot;
        if (slot < 0 || slot >= a.k_slots) return;  // a slot from device memory never leads out of the window
        dst = a.k_tail + b * a.kt_bs + (int64_t)(h - a.heads) * a.kt_hs + slot * a.kt_ts;
    } else {
        const int64_t slot = a.v_slot_dev ? *a.v_slot_dev : a.v_slot;
        if (slot < 0 || slot >= a.v_slots) return;
        dst = a.v_tail + b * a.vt_bs + (int64_t)(h - a.heads - a.kv_heads) * a.vt_hs + slot * a.vt_ts;
        rotate = false;
    }
    R8 o1 = x1, o2 = x2;
    if (rotate) {
        const R8 c1 = *reinterpret_cast<const R8 *>(a.cos + part * 8), c2 = *reinterpret_cast<const R8 *>(a.cos + half + part * 8);
        const R8 s1 = *reinterpret_cast<const R8 *>(a.sin + part * 8), s2 = *reinterpret_cast<const R8 *>(a.sin + half + part * 8);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            o1.v[i] = rope_one(x1.v[i], x2.v[i], c1.v[i], s1.v[i], true);   // x1 cos + (-x2) sin
            o2.v[i] = rope_one(x2.v[i], x1.v[i], c2.v[i], s2.v[i], false);  // x2 cos + x1 sin
        }
    }
    *reinterpret_cast<R8 *>(dst + part * 8) = o1;
    *reinterpret_cast<R8 *>(dst + half + part * 8) = o2;
}

}  // namespace kvmix

using namespace kvmix;

extern "C" int kvmix_rope_append(const kvmix_rope_append_t *p, kvmix_stream_t stream)
{
    if (!p) return KVMIX_ERR_NULL;
    if (p->batch < 0 || p->heads <= 0 || p->kv_heads <= 0 || p->D <= 0 || p->k_tail_slots < 0 || p->v_tail_slots < 0)
        return KVMIX_ERR_SHAPE;
    if (p->heads % p->kv_heads != 0) return KVMIX_ERR_HEADS;
    if (p->D % 16 != 0) return KVMIX_ERR_UNSUPPORTED;
    if (p->batch == 0) return KVMIX_OK;
    if (!p->qkv || !p->cos || !p->sin || !p->q_out || !p->k_tail || !p->v_tail) return KVMIX_ERR_NULL;
    const int64_t total = (int64_t)p->heads + 2 * (int64_t)p->kv_heads;
    if (p->qkv_batch_stride < total * p->D || p->q_batch_stride < (int64_t)p->heads * p->D) return KVMIX_ERR_SHAPE;
    if (p->k_tail_token_stride < p->D || p->v_tail_token_stride < p->D) return KVMIX_ERR_SHAPE;
    if (!p->k_slot_dev && (p->k_slot < 0 || p->k_slot >= p->k_tail_slots)) return KVMIX_ERR_SHAPE;
    if (!p->v_slot_dev && (p->v_slot < 0 || p->v_slot >= p->v_tail_slots)) return KVMIX_ERR_SHAPE;
    RopeArgs a;
    a.qkv = (const uint16_t *)p->qkv;
    a.cos = (const uint16_t *)p->cos;
    a.sin = (const uint16_t *)p->sin;
    a.q_out = (uint16_t *)p->q_out;
    a.k_tail = (uint16_t *)p->k_tail;
    a.v_tail = (uint16_t *)p->v_tail;
    a.k_slot_dev = p->k_slot_dev;
    a.v_slot_dev = p->v_slot_dev;
    a.qkv_bs = p->qkv_batch_stride;
    a.q_bs = p->q_batch_stride;
    a.kt_bs = p->k_tail_batch_stride;
    a.kt_hs = p->k_tail_head_stride;
    a.kt_ts = p->k_tail_token_stride;
    a.vt_bs = p->v_tail_batch_stride;
    a.vt_hs = p->v_tail_head_stride;
    a.vt_ts = p->v_tail_token_stride;
    a.k_slots = p->k_tail_slots;
    a.v_slots = p->v_tail_slots;
    a.k_slot = p->k_slot;
    a.v_slot = p->v_slot;
    a.rows = p->batch * total;
    a.heads = p->heads;
    a.kv_heads = p->kv_heads;
    a.D = (int)p->D;
    const int64_t threads = a.rows * (p->D / 16);
    const int64_t blocks = (threads + kRopeThreads - 1) / kRopeThreads;
    if (blocks > 0x7fffffff) return KVMIX_ERR_SHAPE;
    hipLaunchKernelGGL(rope_append, dim3((unsigned)blocks), dim3(kRopeThreads), 0, (hipStream_t)stream, a);
    return launch_status();
}
