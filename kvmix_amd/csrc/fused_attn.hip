// One decode step of attention over the packed cache and its fp16 tails in a single pass over the
// positions: every block takes one slab of consecutive positions of one (batch, kv head), computes
// that slab's logits from the packed keys (and the fp16 key tail where the slab reaches it), turns
// them into unnormalised probabilities exp(l - m_slab) kept in LDS, multiplies them into the packed
// values (and the fp16 value tail) of the same positions, and writes (m_slab, sum_slab, partial
// out[D]) per head; a second small kernel merges the slabs (a row that fits one slab is finished
// by the first kernel).  Logits and probabilities never go to memory.
//
// Arithmetic against the reference's decode branch (models/modeling_llama_KVmix.py:68-75,180-211):
// logits are rounded to fp16 before the 1/sqrt(D) scaling exactly as there (its GEMV and its tail
// matmul both return fp16), mask and clamp are the same; what is NOT reproduced are the reference's
// roundings after the softmax: it rounds every normalised probability to fp16 and adds the two
// halves of the output as fp16 values, here the probabilities stay fp32 and the sum is rounded
// once.  The result therefore differs from the four-launch step of decode_attn.hip by up to about
// 2^-10 of the largest value magnitude.
//
// Layout handled: D = 128; keys with 1/2/4 bits or dense 3 bits in groups of 32 tokens or the
// reference's 3-bit words (11 codes, own scale and zero); values with 1/2/4 bits or dense 3 bits in
// groups of 32 head dimensions; up to eight query heads per kv head (one block each; they share the
// slab through L2).
#include "kvmix_common.h"

namespace kvmix {

struct FusedArgs {
    const uint16_t *q;        // [samples, D]
    const uint32_t *k_code;   // [kv samples, D, words]
    const uint16_t *k_scale, *k_zero;
    const uint32_t *v_code;   // [kv samples, tokens, D / vpw]
    const uint16_t *v_scale, *v_zero;
    const uint16_t *k_tail, *v_tail;  // [kv samples, slots, D]
    const float *mask;        // optional [batch, width]
    const int64_t *k_len_dev, *v_len_dev;
    uint16_t *out;            // [samples, D]: written by the slab kernel itself when there is one slab
    int64_t o_bs;
    float *ws_o;              // [samples, slabs, D]
    float *ws_ml;             // [samples, slabs, 2]: slab maximum, slab sum
    int64_t q_bs, kc_bs, kc_rs, ksz_bs, ksz_rs, vc_bs, vc_rs, vsz_bs, vsz_rs;
    int64_t kt_bs, kt_ts, vt_bs, vt_ts, mask_bs;
    int64_t k_tokens, v_tokens, k_slots, v_slots, k_len, v_len;
    int k_mode, v_mode;       // 1, 2, 4 = bits; 3 = the reference's 3-bit words (keys) / dense 3-bit (values); 30 = dense 3-bit keys
    int slab;                 // positions per block
    int slabs;                // slabs of a row in the workspace
    int launch_slabs;         // slabs this launch works on: workspace slabs slab0 .., positions from t_begin on
    int slab0;
    int64_t t_begin;
    int head_groups;          // blocks per kv head and slab (query heads of a kv head / heads per block)
    int heads_per_kv, heads;
    float inv_sqrt_d;
};

struct __attribute__((packed, aligned(2))) F8 {
    uint16_t v[8];
};

template <int N>
struct __attribute__((packed, aligned(4))) Words {
    uint32_t v[N];
};

struct __attribute__((packed, aligned(2))) H4 {
    uint16_t v[4];
};

// Lanes that share a key row.  A lane owns 32 positions (one quantization group) or four of the
// reference's 3-bit words, so this sets the slab; the block has 32 key rows in flight per step.
#ifndef KVMIX_FUSED_KEY_LANES
#define KVMIX_FUSED_KEY_LANES 16
#endif
constexpr int kKeyLanes = KVMIX_FUSED_KEY_LANES;
constexpr int kFusedThreads = 32 * kKeyLanes;
constexpr int kFusedWaves = kFusedThreads / kWave;
constexpr int kFusedD = 128;
constexpr int kSlabG32 = kKeyLanes * 32;
constexpr int kSlabRef3 = kKeyLanes * 44;
constexpr int kRedStride = kKeyLanes * 45;  // floats per (wave, head) in `red`: lanes x (44 + 1 pad)
constexpr float kLowest = -3.4028234663852886e38f;
constexpr float kPatternUp = 1237940039285380274899124224.0f;  // 2^90

// A masked field of a word, read as an fp32 bit pattern below 2^24, is code * 2^(offset - 149)
// (subnormals and the first binade share one ulp), so one v_and + one v_fmac per code replaces
// shift, mask, convert, multiply-add.  Fields that end above bit 24 are taken from word >> 24.
// The multiplier carries 2^90; field_unscale(offset) = 2^(59 - offset) takes the rest out at the
// end -- powers of two, nothing is rounded differently.
__device__ __forceinline__ constexpr int field_offset(int bits, int i)
{
    return i * bits + bits <= 24 ? i * bits : i * bits - 24;
}

__device__ __forceinline__ constexpr float field_unscale(int offset)
{
    float v = 576460752303423488.0f;  // 2^59
    for (int k = 0; k < offset; k++) v *= 0.5f;
    return v;
}

// acc[i] += m * field i of w, i < 32 / BITS (BITS = 1, 2, 4), fields scaled as described above
template <int BITS>
__device__ __forceinline__ void fma_fields(uint32_t w, float m, float *acc)
{
    constexpr uint32_t M = (1u << BITS) - 1u;
    const uint32_t hi = w >> 24;
#pragma unroll
    for (int i = 0; i < 32 / BITS; i++) {
        const int off = field_offset(BITS, i);
        const uint32_t f = (i * BITS + BITS <= 24 ? w : hi) & (M << off);
        acc[i] = fmaf(m, __uint_as_float(f), acc[i]);
    }
}

// the reference's 3-bit word: codes 0..9 of three bits, code 10 of two bits at bit 30
__device__ __forceinline__ void fma_fields_ref3(uint32_t w, float m, float *acc)
{
    const uint32_t hi = w >> 24;
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = fmaf(m, __uint_as_float(w & (7u << (3 * i))), acc[i]);
    acc[8] = fmaf(m, __uint_as_float(hi & 0x07u), acc[8]);
    acc[9] = fmaf(m, __uint_as_float(hi & 0x38u), acc[9]);
    acc[10] = fmaf(m, __uint_as_float(hi & 0xC0u), acc[10]);
}

__device__ __forceinline__ constexpr float ref3_unscale(int i) { return field_unscale(3 * (i < 8 ? i : i - 8)); }

// Sum v[0..NV) over the lanes whose indices differ in the bits FIRST, 2 FIRST, .. LAST.  While the
// count is even a step halves what a lane holds (the lane with the bit clear keeps the lower half,
// its partner the upper half); once it is odd the remaining steps are plain exchanges and the
// lanes that differ only in those bits end with the same sums.  Returns the index, in the original
// numbering, of what is left in v[0]; `left` = how many values are left.
template <int NV, int FIRST, int LAST>
__device__ __forceinline__ int fold_lanes(float *v, int lane, int &left)
{
    if constexpr (FIRST > LAST) {
        left = NV;
        return 0;
    } else if constexpr (NV % 2 == 0) {
        constexpr int H = NV / 2;
        const bool up = (lane & FIRST) != 0;
#pragma unroll
        for (int i = 0; i < H; i++) {
            const float keep = up ? v[H + i] : v[i];
            const float send = up ? v[i] : v[H + i];
            v[i] = keep + __shfl_xor(send, FIRST);
        }
        return (up ? H : 0) + fold_lanes<H, FIRST * 2, LAST>(v, lane, left);
    } else {
#pragma unroll
        for (int i = 0; i < NV; i++) v[i] += __shfl_xor(v[i], FIRST);
        return fold_lanes<NV, FIRST * 2, LAST>(v, lane, left);
    }
}

// 32 codes of one quantization group of a value row -> acc[i] += m * code i (pattern-scaled)
template <int MODE>
__device__ __forceinline__ void fma_value_group(const Words<(MODE == 3 ? 3 : MODE)> &g, float m, float *acc)
{
    if (MODE == 3) {
        // dense 3-bit: 32 codes in three consecutive words; four runs of 24 bits hold eight codes each
        const uint32_t r[4] = {g.v[0] & 0xffffffu, ((g.v[0] >> 24) | (g.v[1] << 8)) & 0xffffffu,
                               ((g.v[1] >> 16) | (g.v[2] << 16)) & 0xffffffu, g.v[2] >> 8};
#pragma unroll
        for (int k = 0; k < 4; k++) {
#pragma unroll
            for (int i = 0; i < 8; i++) acc[8 * k + i] = fmaf(m, __uint_as_float(r[k] & (7u << (3 * i))), acc[8 * k + i]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < MODE; j++) fma_fields<MODE>(g.v[j], m, &acc[j * (32 / MODE)]);
    }
}

template <int MODE>
__device__ __forceinline__ constexpr float value_unscale(int i)
{
    return MODE == 3 ? field_unscale(3 * (i % 8)) : field_unscale(field_offset(MODE, i % (32 / MODE)));
}

// Logits of the slab's quantized positions.  kKeyLanes lanes share a key row (one head dimension):
// a lane owns 32 consecutive positions = one quantization group (16 / 8 / 4 bytes of codes, one
// scale, one zero), or four of the reference's 3-bit words; a block covers 32 head dimensions per
// step.  The sums of the lanes that share positions meet in `red`
// ([wave][head][lane * (LPP + 1) + position]).
template <int MODE, int NREP>
__device__ __forceinline__ void slab_key_partials(const FusedArgs &a, int64_t kv, int64_t t0, const float *qs, float *red)
{
    constexpr int WORDS = MODE == 3 ? 4 : (MODE == 30 ? 3 : MODE);  // (30: dense 3-bit, three words per group of 32)
    constexpr int LPP = MODE == 3 ? 44 : 32;
    constexpr int UNIT = MODE == 3 ? 11 : 32;          // positions per (scale, zero)
    constexpr int NSZ = MODE == 3 ? 4 : 1;
    const int tid = threadIdx.x;
    const int sub = tid % kKeyLanes, dg = tid / kKeyLanes;
    const int lane = tid % kWave, wave = tid / kWave;
    const int64_t first = t0 + (int64_t)sub * LPP;       // first position of this lane
    const int64_t left = a.k_tokens - first;               // quantized positions from there on (a multiple of UNIT)
    const int units = left >= LPP ? NSZ : (left > 0 ? (int)(left / UNIT) : 0);
    float acc[NREP][LPP];
    float zacc[NREP][NSZ];
#pragma unroll
    for (int h = 0; h < NREP; h++) {
#pragma unroll
        for (int j = 0; j < NSZ; j++) zacc[h][j] = 0.f;
#pragma unroll
        for (int i = 0; i < LPP; i++) acc[h][i] = 0.f;
    }
    if (units > 0) {
        const int64_t word0 = MODE == 3 ? first / 11 : (MODE == 30 ? first / 32 * 3 : first * MODE / 32);
        const uint32_t *codes = a.k_code + kv * a.kc_bs + word0;
        const int64_t sz0 = kv * a.ksz_bs + first / UNIT;
#pragma unroll
        for (int d = dg; d < kFusedD; d += kFusedThreads / kKeyLanes) {
            Words<WORDS> w;
            uint16_t sc[NSZ], zr[NSZ];
            const uint32_t *cp = codes + (int64_t)d * a.kc_rs;
            const uint16_t *sp = a.k_scale + sz0 + (int64_t)d * a.ksz_rs;
            const uint16_t *zp = a.k_zero + sz0 + (int64_t)d * a.ksz_rs;
            if (MODE != 3 || units == NSZ) {
                w = *reinterpret_cast<const Words<WORDS> *>(cp);
                if (MODE == 3) {
                    const H4 s4 = *reinterpret_cast<const H4 *>(sp), z4 = *reinterpret_cast<const H4 *>(zp);
#pragma unroll
                    for (int j = 0; j < NSZ; j++) {
                        sc[j] = s4.v[j];
                        zr[j] = z4.v[j];
                    }
                } else {
                    sc[0] = sp[0];
                    zr[0] = zp[0];
                }
            } else {  // the lane that holds the last, incomplete run of 3-bit words: nothing past the row's end is read
#pragma unroll
                for (int j = 0; j < NSZ; j++) {
                    const bool in = j < units;
                    w.v[j] = in ? cp[j] : 0u;
                    sc[j] = in ? sp[j] : (uint16_t)0;
                    zr[j] = in ? zp[j] : (uint16_t)0;
                }
            }
#pragma unroll
            for (int h = 0; h < NREP; h++) {
                const float x = qs[h * kFusedD + d];
                if (MODE == 3) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        fma_fields_ref3(w.v[j], x * h16_to_f32(sc[j]) * kPatternUp, &acc[h][11 * j]);
                        zacc[h][j] = fmaf(x, h16_to_f32(zr[j]), zacc[h][j]);
                    }
                } else {
                    const float m = x * h16_to_f32(sc[0]) * kPatternUp;
                    zacc[h][0] = fmaf(x, h16_to_f32(zr[0]), zacc[h][0]);
                    if constexpr (MODE == 30) {
                        fma_value_group<3>(w, m, acc[h]);
                    } else {
#pragma unroll
                        for (int j = 0; j < WORDS; j++) fma_fields<MODE>(w.v[j], m, &acc[h][j * (32 / MODE)]);
                    }
                }
            }
        }
    }
    // undo the pattern scaling, add the zero term, fold the head-dimension phases of the wave
#pragma unroll
    for (int h = 0; h < NREP; h++) {
#pragma unroll
        for (int i = 0; i < LPP; i++) {
            if (MODE == 3) acc[h][i] = fmaf(acc[h][i], ref3_unscale(i % 11), zacc[h][i / 11]);
            else if (MODE == 30) acc[h][i] = fmaf(acc[h][i], value_unscale<3>(i), zacc[h][0]);
            else acc[h][i] = fmaf(acc[h][i], field_unscale(field_offset(MODE, i % (32 / MODE))), zacc[h][0]);
        }
        int left;
        const int at = fold_lanes<LPP, kKeyLanes, 32>(acc[h], lane, left);
#pragma unroll
        for (int i = 0; i < LPP; i++) {
            if (i < left) red[(wave * NREP + h) * kRedStride + sub * (LPP + 1) + at + i] = acc[h][i];
        }
    }
}

// acc[h][i] += sum over the slab's quantized value tokens of p[h][t] * value[t][32 * grp + i]:
// four lanes share a token (one group of 32 head dimensions each), a block covers
// kFusedThreads / 4 tokens per step.  Every load is unconditional (a token past the end is
// redirected to the last one and meets p = 0), so the loads of all steps are in flight together.
template <int MODE, int NREP, int STEPS>
__device__ __forceinline__ void slab_value_quant(const FusedArgs &a, int64_t kv, int64_t t0, int64_t t_end, const float *p,
                                                 float (&acc)[NREP][32])
{
    constexpr int GW = MODE == 3 ? 3 : MODE;  // words per group of 32 codes
    const int grp = threadIdx.x % 4, tok = threadIdx.x / 4;
    const uint32_t *codes = a.v_code + kv * a.vc_bs + grp * GW;
    const int64_t sz = kv * a.vsz_bs + grp;
    float zacc[NREP];
#pragma unroll
    for (int h = 0; h < NREP; h++) zacc[h] = 0.f;
#pragma unroll
    for (int it = 0; it < STEPS; it++) {
        const int at = tok + it * (kFusedThreads / 4);
        const bool in = t0 + at < t_end;
        const int64_t t = in ? t0 + at : t_end - 1;
        const Words<GW> g = *reinterpret_cast<const Words<GW> *>(codes + t * a.vc_rs);
        const float s = h16_to_f32(a.v_scale[sz + t * a.vsz_rs]);
        const float z = h16_to_f32(a.v_zero[sz + t * a.vsz_rs]);
#pragma unroll
        for (int h = 0; h < NREP; h++) {
            const float ph = in ? p[h * a.slab + at] : 0.f;
            zacc[h] = fmaf(ph, z, zacc[h]);
            fma_value_group<MODE>(g, ph * s * kPatternUp, acc[h]);
        }
    }
#pragma unroll
    for (int h = 0; h < NREP; h++) {
#pragma unroll
        for (int i = 0; i < 32; i++) acc[h][i] = fmaf(acc[h][i], value_unscale<MODE>(i), zacc[h]);
    }
}

__device__ __forceinline__ float fused_block_reduce(float v, bool is_max, float *scratch)
{
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float other = __shfl_xor(v, o);
        v = is_max ? fmaxf(v, other) : v + other;
    }
    __syncthreads();  // (scratch may still be read from the previous reduction)
    if (threadIdx.x % kWave == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < kFusedWaves; w++) r = is_max ? fmaxf(r, scratch[w]) : r + scratch[w];
    return r;
}

// grid = (slabs, kv samples, heads_per_kv / NREP)
template <int NREP>
__global__ void __launch_bounds__(kFusedThreads) attn_fused_slab(FusedArgs a)
{
    __shared__ float red[kFusedWaves * NREP * kRedStride];  // key partials; later the value partials
    __shared__ float lg[NREP * kSlabRef3];                  // logits, then probabilities, [head][position]
    __shared__ float qs[NREP * kFusedD];
    __shared__ float scratch[kFusedWaves];

    const int tid = threadIdx.x;
    // Workgroups go to the 8 XCDs (each with its own L2) round-robin in launch order.  The launch
    // index is mapped to a logical one such that consecutive logical indices share an XCD, and the
    // logical order is slab-fastest, then query head, then kv head: the slabs of one row of scales
    // (neighbours share 128-byte lines) and the query heads of one kv head meet in one L2.
    // (the grid is one-dimensional: slabs x head groups x kv heads blocks)
    const int64_t n_blocks = gridDim.x, launch = blockIdx.x;
    const int64_t per = n_blocks / 8, rem = n_blocks % 8, xcd = launch % 8;
    const int64_t logical = xcd * per + (xcd < rem ? xcd : rem) + launch / 8;
    const int slab = (int)(logical % a.launch_slabs);
    const int head_group = (int)((logical / a.launch_slabs) % a.head_groups);
    const int64_t kv = logical / ((int64_t)a.launch_slabs * a.head_groups);
    const int64_t sample0 = kv * a.heads_per_kv + (int64_t)head_group * NREP;
    const int S = a.slab;
    const int64_t t0 = a.t_begin + (int64_t)slab * S, t1 = t0 + S;
    int64_t k_len = a.k_len_dev ? *a.k_len_dev : a.k_len;
    int64_t v_len = a.v_len_dev ? *a.v_len_dev : a.v_len;
    k_len = k_len < 0 ? 0 : (k_len > a.k_slots ? a.k_slots : k_len);  // a length from device memory never leads past the window
    v_len = v_len < 0 ? 0 : (v_len > a.v_slots ? a.v_slots : v_len);

    for (int i = tid; i < NREP * kFusedD; i += kFusedThreads)
        qs[i] = h16_to_f32(a.q[(sample0 + i / kFusedD) * a.q_bs + i % kFusedD]);
    for (int i = tid; i < NREP * S; i += kFusedThreads) lg[i] = -INFINITY;
    __syncthreads();

    const float *mrow = a.mask ? a.mask + (sample0 / a.heads) * a.mask_bs : nullptr;
    auto finish = [&](float dot, int64_t pos) {  // fp16 logit -> scaled, masked fp32 value
        float x = h16_to_f32(f32_to_h16(dot)) * a.inv_sqrt_d;
        if (mrow) x = fmaxf(x + mrow[pos], kLowest);
        return x;
    };

    // 1a. logits of the quantized keys in [t0, min(t1, k_tokens))
    if (t0 < a.k_tokens) {
        switch (a.k_mode) {
        case 4: slab_key_partials<4, NREP>(a, kv, t0, qs, red); break;
        case 2: slab_key_partials<2, NREP>(a, kv, t0, qs, red); break;
        case 1: slab_key_partials<1, NREP>(a, kv, t0, qs, red); break;
        case 30: slab_key_partials<30, NREP>(a, kv, t0, qs, red); break;
        default: slab_key_partials<3, NREP>(a, kv, t0, qs, red); break;
        }
        __syncthreads();
        const int lpp = a.k_mode == 3 ? 44 : 32;
        for (int idx = tid; idx < NREP * S; idx += kFusedThreads) {
            const int h = idx / S, pos = idx % S;
            if (t0 + pos < a.k_tokens) {
                const int at = (pos / lpp) * (lpp + 1) + pos % lpp;
                float dot = 0.f;
#pragma unroll
                for (int w = 0; w < kFusedWaves; w++) dot += red[(w * NREP + h) * kRedStride + at];
                lg[idx] = finish(dot, t0 + pos);
            }
        }
    }
    // 1b. logits of the fp16 key tail: positions k_tokens + j, j < k_len, that fall into the slab
    {
        const int sub = tid % 16, grp = tid / 16;
        const int64_t j_begin = t0 > a.k_tokens ? t0 - a.k_tokens : 0;
        const int64_t j_end = t1 - a.k_tokens < k_len ? t1 - a.k_tokens : k_len;
        const uint16_t *kt = a.k_tail + kv * a.kt_bs + sub * 8;
        for (int64_t j0 = j_begin; j0 < j_end; j0 += kFusedThreads / 16) {
            const int64_t j = j0 + grp;
            const bool in = j < j_end;
            const F8 kk = *reinterpret_cast<const F8 *>(kt + (in ? j : j_begin) * a.kt_ts);
            float dot[NREP];
#pragma unroll
            for (int h = 0; h < NREP; h++) {
                dot[h] = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) dot[h] = fmaf(qs[h * kFusedD + sub * 8 + i], h16_to_f32(kk.v[i]), dot[h]);
#pragma unroll
                for (int o = 8; o >= 1; o >>= 1) dot[h] += __shfl_xor(dot[h], o);
            }
            if (in && sub == 0) {
                const int64_t pos = a.k_tokens + j;
#pragma unroll
                for (int h = 0; h < NREP; h++) lg[h * S + (int)(pos - t0)] = finish(dot[h], pos);
            }
        }
    }
    __syncthreads();

    // 2. per head: slab maximum, unnormalised probabilities, their sum
    float m_h[NREP], l_h[NREP];
#pragma unroll
    for (int h = 0; h < NREP; h++) {
        float mx = -INFINITY;
        for (int pos = tid; pos < S; pos += kFusedThreads) mx = fmaxf(mx, lg[h * S + pos]);
        mx = fused_block_reduce(mx, true, scratch);
        float sum = 0.f;
        for (int pos = tid; pos < S; pos += kFusedThreads) {
            const float x = lg[h * S + pos];
            const float e = (x == -INFINITY) ? 0.f : expf(x - mx);
            lg[h * S + pos] = e;
            sum += e;
        }
        sum = fused_block_reduce(sum, false, scratch);
        m_h[h] = mx;
        l_h[h] = sum;
    }
    __syncthreads();

    // 3. probabilities times values of the same positions: lane = 32 head dimensions of a token
    float acc[NREP][32];
#pragma unroll
    for (int h = 0; h < NREP; h++) {
#pragma unroll
        for (int i = 0; i < 32; i++) acc[h][i] = 0.f;
    }
    if (t0 < a.v_tokens) {
        const int64_t t_end = t1 < a.v_tokens ? t1 : a.v_tokens;
        constexpr int kSteps32 = kSlabG32 / (kFusedThreads / 4), kStepsRef3 = (kSlabRef3 + kFusedThreads / 4 - 1) / (kFusedThreads / 4);
        if (S == kSlabG32) {
            switch (a.v_mode) {
            case 4: slab_value_quant<4, NREP, kSteps32>(a, kv, t0, t_end, lg, acc); break;
            case 2: slab_value_quant<2, NREP, kSteps32>(a, kv, t0, t_end, lg, acc); break;
            case 1: slab_value_quant<1, NREP, kSteps32>(a, kv, t0, t_end, lg, acc); break;
            default: slab_value_quant<3, NREP, kSteps32>(a, kv, t0, t_end, lg, acc); break;
            }
        } else {
            switch (a.v_mode) {
            case 4: slab_value_quant<4, NREP, kStepsRef3>(a, kv, t0, t_end, lg, acc); break;
            case 2: slab_value_quant<2, NREP, kStepsRef3>(a, kv, t0, t_end, lg, acc); break;
            case 1: slab_value_quant<1, NREP, kStepsRef3>(a, kv, t0, t_end, lg, acc); break;
            default: slab_value_quant<3, NREP, kStepsRef3>(a, kv, t0, t_end, lg, acc); break;
            }
        }
    }
    {
        const int grp = tid % 4, tok = tid / 4;
        const int64_t j_begin = t0 > a.v_tokens ? t0 - a.v_tokens : 0;
        const int64_t j_end = t1 - a.v_tokens < v_len ? t1 - a.v_tokens : v_len;
        const uint16_t *vt = a.v_tail + kv * a.vt_bs + grp * 32;
        for (int64_t j = j_begin + tok; j < j_end; j += kFusedThreads / 4) {
            F8 vv[4];
#pragma unroll
            for (int k = 0; k < 4; k++) vv[k] = *reinterpret_cast<const F8 *>(vt + j * a.vt_ts + 8 * k);
            const int pos = (int)(a.v_tokens + j - t0);
#pragma unroll
            for (int h = 0; h < NREP; h++) {
                const float ph = lg[h * S + pos];
#pragma unroll
                for (int i = 0; i < 32; i++) acc[h][i] = fmaf(ph, h16_to_f32(vv[i / 8].v[i % 8]), acc[h][i]);
            }
        }
    }
    // the sixteen tokens of a wave, then the four waves
    const int lane = tid % kWave, wave = tid / kWave;
    __syncthreads();  // (red still holds the key partials that step 1a read)
#pragma unroll
    for (int h = 0; h < NREP; h++) {
        const int at = scatter_reduce<32, 4, 1>(acc[h], lane);  // every lane ends with two head dimensions
        red[(wave * NREP + h) * kFusedD + (lane % 4) * 32 + at] = acc[h][0];
        red[(wave * NREP + h) * kFusedD + (lane % 4) * 32 + at + 1] = acc[h][1];
    }
    __syncthreads();
    for (int idx = tid; idx < NREP * kFusedD; idx += kFusedThreads) {
        const int h = idx / kFusedD, c = idx % kFusedD;
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < kFusedWaves; w++) o += red[(w * NREP + h) * kFusedD + c];
        if (a.slabs == 1) a.out[(sample0 + h) * a.o_bs + c] = f32_to_h16(l_h[h] > 0.f ? o / l_h[h] : 0.f);
        else a.ws_o[((sample0 + h) * a.slabs + a.slab0 + slab) * kFusedD + c] = o;
    }
    if (tid == 0 && a.slabs > 1) {
#pragma unroll
        for (int h = 0; h < NREP; h++) {
            a.ws_ml[((sample0 + h) * a.slabs + a.slab0 + slab) * 2 + 0] = m_h[h];
            a.ws_ml[((sample0 + h) * a.slabs + a.slab0 + slab) * 2 + 1] = l_h[h];
        }
    }
}

// grid = samples, one thread per head dimension: out = sum_s o_s exp(m_s - M) / sum_s l_s exp(m_s - M).
// The slab weights are computed once per block into LDS; the partial outputs are then read with
// independent loads (a slab without a live position has weight 0, nothing is skipped).
constexpr int kMergeChunk = 128;  // slabs whose weights are in LDS at a time
__global__ void __launch_bounds__(kFusedD) attn_fused_merge(const float *ws_o, const float *ws_ml, int slabs, uint16_t *out,
                                                            int64_t o_bs)
{
    __shared__ float wgt[kMergeChunk];
    __shared__ float part[kFusedD / kWave];
    const int64_t sample = blockIdx.x;
    const int c = threadIdx.x;
    const float *ml = ws_ml + sample * slabs * 2;
    // the row maximum: every thread takes a share of the slabs, then the block combines
    float M = -INFINITY;
    for (int s = c; s < slabs; s += kFusedD) M = fmaxf(M, ml[2 * s]);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
    if (c % kWave == 0) part[c / kWave] = M;
    __syncthreads();
    M = fmaxf(part[0], part[1]);
    float L = 0.f, o = 0.f;
    for (int s0 = 0; s0 < slabs; s0 += kMergeChunk) {
        const int n = slabs - s0 < kMergeChunk ? slabs - s0 : kMergeChunk;
        __syncthreads();  // (wgt may still be read from the previous chunk)
        if (c < n) {
            const float m = ml[2 * (s0 + c)];
            wgt[c] = m == -INFINITY ? 0.f : expf(m - M);
        }
        __syncthreads();
        const float *op = ws_o + (sample * slabs + s0) * kFusedD + c;
#pragma unroll 8
        for (int s = 0; s < n; s++) {
            L = fmaf(ml[2 * (s0 + s) + 1], wgt[s], L);
            o = fmaf(op[(int64_t)s * kFusedD], wgt[s], o);
        }
    }
    out[sample * o_bs + c] = f32_to_h16(L > 0.f ? o / L : 0.f);
}

}  // namespace kvmix

using namespace kvmix;

static int fused_key_mode(const kvmix_decode_attn_t *p)
{
    if (p->k_tokens == 0) return 4;  // no quantized keys: any mode, nothing is read
    if (p->k_fmt == KVMIX_FMT_DENSE3) return p->k_bits == 3 && p->k_group == 32 ? 30 : 0;
    if (p->k_fmt != KVMIX_FMT_REF) return 0;
    if (p->k_bits == 3) return p->k_group == 11 ? 3 : 0;
    return (p->k_bits == 1 || p->k_bits == 2 || p->k_bits == 4) && p->k_group == 32 ? p->k_bits : 0;
}

static int fused_value_mode(const kvmix_decode_attn_t *p)
{
    if (p->v_tokens == 0) return 4;
    if (p->v_group != 32) return 0;
    if (p->v_bits == 3) return p->v_fmt == KVMIX_FMT_DENSE3 ? 3 : 0;
    return (p->v_bits == 1 || p->v_bits == 2 || p->v_bits == 4) && p->v_fmt == KVMIX_FMT_REF ? p->v_bits : 0;
}

static int64_t fused_width(const kvmix_decode_attn_t *p)
{
    const int64_t a = p->k_tokens + p->k_tail_slots, b = p->v_tokens + p->v_tail_slots;
    return a > b ? a : b;
}

static int fused_slab(const kvmix_decode_attn_t *p) { return p->k_tokens > 0 && fused_key_mode(p) == 3 ? kSlabRef3 : kSlabG32; }

static int64_t fused_slabs(const kvmix_decode_attn_t *p)
{
    const int s = fused_slab(p);
    return (fused_width(p) + s - 1) / s;
}

// How a row's positions are divided into slabs.  Large steps whose keys and values are quantized to the same
// length take the quantized positions through the matrix-core kernel (attn_slab_mfma: tiles of 1024 positions, the
// formats of gemv_cols_mfma2 and gemv_rows_mfma) and only the fp16 tails through attn_fused_slab; everything
// else goes through attn_fused_slab from position 0.
constexpr int64_t kSlabMfmaMinWaves = 512;  // (measured: 512 waves 34 against 38 us, 256 waves 33 against 25 us)
struct FusedLayout {
    bool mfma;
    int64_t tiles;       // slabs of the matrix-core kernel (first in the workspace)
    int64_t tail_slabs;  // slabs of attn_fused_slab, from position t_begin on
    int64_t t_begin;
    int64_t slabs() const { return tiles + tail_slabs; }
};

static FusedLayout fused_layout(const kvmix_decode_attn_t *p)
{
    FusedLayout l{false, 0, fused_slabs(p), 0};
    const int km = fused_key_mode(p), vm = fused_value_mode(p);
    const int vbits = vm == 3 ? 3 : vm;
    const int64_t tiles = (p->k_tokens / 32 + 31) / 32;
    if (p->k_tokens >= 1024 && p->k_tokens == p->v_tokens && (km == 1 || km == 2 || km == 4) && vm != 0 &&
        p->v_code_row_stride == kFusedD * vbits / 32 && p->v_sz_row_stride == kFusedD / 32 && p->samples <= 65535 &&
        (kFusedD + 1) * p->k_code_row_stride < (1ll << 29) && (kFusedD + 1) * p->k_sz_row_stride < (1ll << 30) &&
        // (the value phase forms 32-bit byte offsets of code rows and 32-bit element offsets of scale rows)
        p->v_tokens * p->v_code_row_stride < (1ll << 30) && p->v_tokens * p->v_sz_row_stride < (1ll << 31) &&
        p->samples * tiles >= kSlabMfmaMinWaves) {
        l.mfma = true;
        l.tiles = tiles;
        l.t_begin = p->k_tokens;
        l.tail_slabs = (fused_width(p) - p->k_tokens + kSlabG32 - 1) / kSlabG32;
    }
    return l;
}

extern "C" int kvmix_decode_attention_fused_supported(const kvmix_decode_attn_t *p)
{
    if (!p) return 0;
    if (p->D != kFusedD || fused_key_mode(p) == 0 || fused_value_mode(p) == 0) return 0;
    if (p->heads_per_kv != 1 && p->heads_per_kv != 2 && p->heads_per_kv != 4 && p->heads_per_kv != 8) return 0;
    return 1;
}

extern "C" size_t kvmix_decode_attention_fused_workspace_bytes(const kvmix_decode_attn_t *p)
{
    if (!p || p->samples <= 0) return 0;
    if (!kvmix_decode_attention_fused_supported(p)) return 0;
    return (size_t)p->samples * (size_t)fused_layout(p).slabs() * (kFusedD + 2) * sizeof(float);
}

// the argument checks of kvmix_decode_attention_fused; `pointers`: also that the operands are there (the plan query
// passes sizes only)
static int fused_check(const kvmix_decode_attn_t *p, bool pointers)
{
    if (!p) return KVMIX_ERR_NULL;
    if (p->samples < 0 || p->D <= 0 || p->k_tokens < 0 || p->v_tokens < 0 || p->k_tail_slots < 0 || p->v_tail_slots < 0 ||
        p->k_tail_len < 0 || p->v_tail_len < 0 || p->k_tail_len > p->k_tail_slots || p->v_tail_len > p->v_tail_slots)
        return KVMIX_ERR_SHAPE;
    if (p->heads_per_kv <= 0 || p->samples % p->heads_per_kv != 0) return KVMIX_ERR_HEADS;
    if (p->heads <= 0 || p->samples % p->heads != 0 || p->heads % p->heads_per_kv != 0) return KVMIX_ERR_HEADS;
    if (!kvmix_decode_attention_fused_supported(p)) return KVMIX_ERR_UNSUPPORTED;
    if (p->samples == 0) return KVMIX_OK;
    const int64_t width = fused_width(p);
    if (width == 0) return KVMIX_ERR_SHAPE;
    if (!p->k_tail_len_dev && !p->v_tail_len_dev && p->k_tokens + p->k_tail_len != p->v_tokens + p->v_tail_len)
        return KVMIX_ERR_SHAPE;
    if (pointers) {
        if (!p->q || !p->out) return KVMIX_ERR_NULL;
        if ((p->k_tail_slots > 0 && !p->k_tail) || (p->v_tail_slots > 0 && !p->v_tail)) return KVMIX_ERR_NULL;
    }
    if (p->out_stride < p->D || p->q_stride < p->D || (p->mask && p->mask_stride < width)) return KVMIX_ERR_SHAPE;
    if ((p->k_tail_slots > 0 && p->k_tail_token_stride < p->D) || (p->v_tail_slots > 0 && p->v_tail_token_stride < p->D))
        return KVMIX_ERR_SHAPE;
    const int k_mode = fused_key_mode(p);
    if (p->k_tokens > 0) {
        if (pointers && (!p->k_code || !p->k_scale || !p->k_zero)) return KVMIX_ERR_NULL;
        const int64_t unit = k_mode == 3 ? 11 : 32;
        if (p->k_tokens % unit != 0) return KVMIX_ERR_SHAPE;
        const int64_t words = k_mode == 3 ? p->k_tokens / 11 : p->k_tokens * (k_mode == 30 ? 3 : k_mode) / 32;
        if (p->k_code_row_stride < words || p->k_sz_row_stride < p->k_tokens / unit) return KVMIX_ERR_SHAPE;
    }
    if (p->v_tokens > 0) {
        if (pointers && (!p->v_code || !p->v_scale || !p->v_zero)) return KVMIX_ERR_NULL;
        if (p->v_code_row_stride < kFusedD * p->v_bits / 32 || p->v_sz_row_stride < kFusedD / 32) return KVMIX_ERR_SHAPE;
    }
    const FusedLayout lay = fused_layout(p);
    const int64_t slabs = lay.slabs();
    if (slabs > 0x7fffffff || slabs * p->samples > 0x7fffffff) return KVMIX_ERR_SHAPE;  // (blocks of one launch)
    return KVMIX_OK;
}

extern "C" int kvmix_decode_attention_fused_plan(const kvmix_decode_attn_t *p, kvmix_attn_plan_t *plan)
{
    if (!plan) return KVMIX_ERR_NULL;
    *plan = kvmix_attn_plan_t{};
    const int rc = fused_check(p, false);
    if (rc != KVMIX_OK || p->samples == 0) return rc;
    const FusedLayout lay = fused_layout(p);
    plan->matrix = lay.mfma ? 1 : 0;
    plan->matrix_tiles = lay.tiles;
    plan->slab_positions = fused_slab(p);
    plan->slab_begin = lay.t_begin;
    plan->slabs = lay.tail_slabs;
    if (lay.mfma) {
        const int prc = plan_attn_slab_mfma(p->k_tokens, p->samples, plan->matrix_grid, plan->matrix_block);
        if (prc != KVMIX_OK) return prc;
        plan->launches++;
    }
    if (lay.tail_slabs > 0) {
        plan->slab_grid[0] = (unsigned)(lay.tail_slabs * p->samples);
        plan->slab_grid[1] = plan->slab_grid[2] = 1;
        plan->launches++;
    }
    if (!(lay.slabs() == 1 && !lay.mfma)) plan->launches++;  // the merge
    return KVMIX_OK;
}

extern "C" int kvmix_decode_attention_fused(const kvmix_decode_attn_t *p, void *workspace, size_t workspace_bytes,
                                            kvmix_stream_t stream)
{
    const int chk = fused_check(p, true);
    if (chk != KVMIX_OK || p->samples == 0) return chk;
    const int k_mode = fused_key_mode(p), v_mode = fused_value_mode(p);
    const FusedLayout lay = fused_layout(p);
    const int64_t slabs = lay.slabs();
    const int64_t kv_samples = p->samples / p->heads_per_kv;
    if (!workspace || workspace_bytes < kvmix_decode_attention_fused_workspace_bytes(p)) return KVMIX_ERR_WORKSPACE;

    FusedArgs a;
    a.q = (const uint16_t *)p->q;
    a.k_code = p->k_code;
    a.k_scale = (const uint16_t *)p->k_scale;
    a.k_zero = (const uint16_t *)p->k_zero;
    a.v_code = p->v_code;
    a.v_scale = (const uint16_t *)p->v_scale;
    a.v_zero = (const uint16_t *)p->v_zero;
    a.k_tail = (const uint16_t *)p->k_tail;
    a.v_tail = (const uint16_t *)p->v_tail;
    a.mask = p->mask;
    a.k_len_dev = p->k_tail_len_dev;
    a.v_len_dev = p->v_tail_len_dev;
    a.out = (uint16_t *)p->out;
    a.o_bs = p->out_stride;
    a.ws_o = (float *)workspace;
    a.ws_ml = a.ws_o + p->samples * slabs * kFusedD;
    a.q_bs = p->q_stride;
    a.kc_bs = p->k_code_batch_stride;
    a.kc_rs = p->k_code_row_stride;
    a.ksz_bs = p->k_sz_batch_stride;
    a.ksz_rs = p->k_sz_row_stride;
    a.vc_bs = p->v_code_batch_stride;
    a.vc_rs = p->v_code_row_stride;
    a.vsz_bs = p->v_sz_batch_stride;
    a.vsz_rs = p->v_sz_row_stride;
    a.kt_bs = p->k_tail_batch_stride;
    a.kt_ts = p->k_tail_token_stride;
    a.vt_bs = p->v_tail_batch_stride;
    a.vt_ts = p->v_tail_token_stride;
    a.mask_bs = p->mask_stride;
    a.k_tokens = p->k_tokens;
    a.v_tokens = p->v_tokens;
    a.k_slots = p->k_tail_slots;
    a.v_slots = p->v_tail_slots;
    a.k_len = p->k_tail_len;
    a.v_len = p->v_tail_len;
    a.k_mode = k_mode;
    a.v_mode = v_mode;
    a.slab = fused_slab(p);
    a.slabs = (int)slabs;
    a.launch_slabs = (int)lay.tail_slabs;
    a.slab0 = (int)lay.tiles;
    a.t_begin = lay.t_begin;
    a.heads_per_kv = p->heads_per_kv;
    a.heads = p->heads;
    a.inv_sqrt_d = 1.0f / sqrtf((float)p->D);

    hipStream_t st = (hipStream_t)stream;
    // one query head per block: the heads that share a kv head re-read its slab through L2 (two heads
    // per block need more registers than a 512-thread block has)
    a.head_groups = p->heads_per_kv;
    int rc = KVMIX_OK;
    if (lay.mfma) {
        AttnSlabArgs m;
        m.q = a.q, m.q_bs = a.q_bs;
        m.k_code = a.k_code, m.k_scale = a.k_scale, m.k_zero = a.k_zero;
        m.kc_bs = a.kc_bs, m.kc_rs = a.kc_rs, m.ksz_bs = a.ksz_bs, m.ksz_rs = a.ksz_rs;
        m.v_code = a.v_code, m.v_scale = a.v_scale, m.v_zero = a.v_zero;
        m.vc_bs = a.vc_bs, m.vsz_bs = a.vsz_bs;
        m.mask = a.mask, m.mask_bs = a.mask_bs;
        m.ws_o = a.ws_o, m.ws_ml = a.ws_ml;
        m.tokens = p->k_tokens;
        m.heads_per_kv = p->heads_per_kv, m.heads = p->heads;
        m.slabs = (int)slabs;
        m.inv_sqrt_d = a.inv_sqrt_d;
        rc = launch_attn_slab_mfma(m, k_mode, v_mode == 3 ? 30 : v_mode, p->samples, st);
        if (rc != KVMIX_OK) return rc;
    }
    if (lay.tail_slabs > 0) {
        const dim3 grid((unsigned)(lay.tail_slabs * kv_samples * p->heads_per_kv));
        hipLaunchKernelGGL(attn_fused_slab<1>, grid, dim3(kFusedThreads), 0, st, a);
        rc = launch_status();
    }
    if (rc != KVMIX_OK || (slabs == 1 && !lay.mfma)) return rc;  // a single slab of attn_fused_slab is normalised and stored by that kernel
    hipLaunchKernelGGL(attn_fused_merge, dim3((unsigned)p->samples), dim3(kFusedD), 0, st, a.ws_o, a.ws_ml, (int)slabs,
                       (uint16_t *)p->out, p->out_stride);
    return launch_status();
}
