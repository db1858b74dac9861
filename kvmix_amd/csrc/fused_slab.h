// The vector-ALU slab of the single-pass decode step (see fused_attn.hip for the arithmetic and its relation to the
// reference): device code shared by the stand-alone slab kernel (fused_attn.hip) and by the matrix-core launch, which
// runs the slabs of the positions its tiles do not cover as trailing blocks (dequant_gemv.hip).
#pragma once

#include "kvmix_common.h"

namespace kvmix {
namespace fused {

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

// Lanes that share a key row (KL, a template argument of the slab code: 16 in the stand-alone kernel, 8 where the
// slabs run as trailing blocks of the matrix-core launch).  A lane owns 32 positions (one quantization group) or
// four of the reference's 3-bit words, so this sets the slab; the block has 32 key rows in flight per step.
template <int KL>
struct SlabCfg {
    static constexpr int kThreads = 32 * KL;
    static constexpr int kWaves = kThreads / kWave;
    static constexpr int kSlabG32 = KL * 32;    // positions per slab, keys in groups of 32
    static constexpr int kSlabRef3 = KL * 44;   // ... keys in the reference's 3-bit words
    static constexpr int kRedStride = KL * 45;  // floats per (wave, head) in `red`: lanes x (44 + 1 pad)
    // floats of LDS a block of NREP heads needs: key / value partials, logits, the query, the block reductions
    static constexpr int lds_floats(int nrep) { return kWaves * nrep * kRedStride + nrep * kSlabRef3 + nrep * 128 + kWaves; }
};
constexpr int kFusedD = 128;
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

// Logits of the slab's quantized positions.  KL lanes share a key row (one head dimension):
// a lane owns 32 consecutive positions = one quantization group (16 / 8 / 4 bytes of codes, one
// scale, one zero), or four of the reference's 3-bit words; a block covers 32 head dimensions per
// step.  The sums of the lanes that share positions meet in `red`
// ([wave][head][lane * (LPP + 1) + position]).
template <int MODE, int NREP, int KL>
__device__ __forceinline__ void slab_key_partials(const FusedArgs &a, int64_t kv, int64_t t0, const float *qs, float *red, int tid)
{
    constexpr int WORDS = MODE == 3 ? 4 : (MODE == 30 ? 3 : MODE);  // (30: dense 3-bit, three words per group of 32)
    constexpr int LPP = MODE == 3 ? 44 : 32;
    constexpr int UNIT = MODE == 3 ? 11 : 32;          // positions per (scale, zero)
    constexpr int NSZ = MODE == 3 ? 4 : 1;
    const int sub = tid % KL, dg = tid / KL;
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
        for (int d = dg; d < kFusedD; d += 32) {
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
        const int at = fold_lanes<LPP, KL, 32>(acc[h], lane, left);
#pragma unroll
        for (int i = 0; i < LPP; i++) {
            if (i < left) red[(wave * NREP + h) * (SlabCfg<KL>::kRedStride) + sub * (LPP + 1) + at + i] = acc[h][i];
        }
    }
}

// acc[h][i] += sum over the slab's quantized value tokens of p[h][t] * value[t][32 * grp + i]:
// four lanes share a token (one group of 32 head dimensions each), a block covers
// (SlabCfg<KL>::kThreads) / 4 tokens per step.  Every load is unconditional (a token past the end is
// redirected to the last one and meets p = 0), so the loads of all steps are in flight together.
template <int MODE, int NREP, int STEPS, int KL>
__device__ __forceinline__ void slab_value_quant(const FusedArgs &a, int64_t kv, int64_t t0, int64_t t_end, const float *p,
                                                 float (&acc)[NREP][32], int tid)
{
    constexpr int GW = MODE == 3 ? 3 : MODE;  // words per group of 32 codes
    const int grp = tid % 4, tok = tid / 4;
    const uint32_t *codes = a.v_code + kv * a.vc_bs + grp * GW;
    const int64_t sz = kv * a.vsz_bs + grp;
    float zacc[NREP];
#pragma unroll
    for (int h = 0; h < NREP; h++) zacc[h] = 0.f;
#pragma unroll
    for (int it = 0; it < STEPS; it++) {
        const int at = tok + it * ((SlabCfg<KL>::kThreads) / 4);
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

template <int KL>
__device__ __forceinline__ float fused_block_reduce(float v, bool is_max, float *scratch, int tid)
{
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float other = __shfl_xor(v, o);
        v = is_max ? fmaxf(v, other) : v + other;
    }
    __syncthreads();  // (scratch may still be read from the previous reduction)
    if (tid % kWave == 0) scratch[tid / kWave] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < (SlabCfg<KL>::kWaves); w++) r = is_max ? fmaxf(r, scratch[w]) : r + scratch[w];
    return r;
}

// One slab: block `launch` of `n_blocks` (slabs x head groups x kv heads), (SlabCfg<KL>::kThreads) threads (numbered
// by `tid`), SlabCfg<KL>::lds_floats(NREP) floats of LDS at `smem`.  Every thread of the block must call it (block barriers).
template <int NREP, int KL>
__device__ __forceinline__ void attn_fused_slab_body(const FusedArgs &a, int64_t launch, int64_t n_blocks, int tid, float *smem)
{
    float *red = smem;                                                        // key partials; later the value partials
    float *lg = red + (SlabCfg<KL>::kWaves) * NREP * (SlabCfg<KL>::kRedStride);   // logits, then probabilities, [head][position]
    float *qs = lg + NREP * (SlabCfg<KL>::kSlabRef3);
    float *scratch = qs + NREP * kFusedD;

    // Workgroups go to the 8 XCDs (each with its own L2) round-robin in launch order.  The launch
    // index is mapped to a logical one such that consecutive logical indices share an XCD, and the
    // logical order is slab-fastest, then query head, then kv head: the slabs of one row of scales
    // (neighbours share 128-byte lines) and the query heads of one kv head meet in one L2.
    // (one-dimensional numbering: slabs x head groups x kv heads blocks)
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

    for (int i = tid; i < NREP * kFusedD; i += (SlabCfg<KL>::kThreads))
        qs[i] = h16_to_f32(a.q[(sample0 + i / kFusedD) * a.q_bs + i % kFusedD]);
    for (int i = tid; i < NREP * S; i += (SlabCfg<KL>::kThreads)) lg[i] = -INFINITY;
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
        case 4: slab_key_partials<4, NREP, KL>(a, kv, t0, qs, red, tid); break;
        case 2: slab_key_partials<2, NREP, KL>(a, kv, t0, qs, red, tid); break;
        case 1: slab_key_partials<1, NREP, KL>(a, kv, t0, qs, red, tid); break;
        case 30: slab_key_partials<30, NREP, KL>(a, kv, t0, qs, red, tid); break;
        default: slab_key_partials<3, NREP, KL>(a, kv, t0, qs, red, tid); break;
        }
        __syncthreads();
        const int lpp = a.k_mode == 3 ? 44 : 32;
        for (int idx = tid; idx < NREP * S; idx += (SlabCfg<KL>::kThreads)) {
            const int h = idx / S, pos = idx % S;
            if (t0 + pos < a.k_tokens) {
                const int at = (pos / lpp) * (lpp + 1) + pos % lpp;
                float dot = 0.f;
#pragma unroll
                for (int w = 0; w < (SlabCfg<KL>::kWaves); w++) dot += red[(w * NREP + h) * (SlabCfg<KL>::kRedStride) + at];
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
        for (int64_t j0 = j_begin; j0 < j_end; j0 += (SlabCfg<KL>::kThreads) / 16) {
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
        for (int pos = tid; pos < S; pos += (SlabCfg<KL>::kThreads)) mx = fmaxf(mx, lg[h * S + pos]);
        mx = fused_block_reduce<KL>(mx, true, scratch, tid);
        float sum = 0.f;
        for (int pos = tid; pos < S; pos += (SlabCfg<KL>::kThreads)) {
            const float x = lg[h * S + pos];
            const float e = (x == -INFINITY) ? 0.f : expf(x - mx);
            lg[h * S + pos] = e;
            sum += e;
        }
        sum = fused_block_reduce<KL>(sum, false, scratch, tid);
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
        constexpr int kSteps32 = (SlabCfg<KL>::kSlabG32) / ((SlabCfg<KL>::kThreads) / 4), kStepsRef3 = ((SlabCfg<KL>::kSlabRef3) + (SlabCfg<KL>::kThreads) / 4 - 1) / ((SlabCfg<KL>::kThreads) / 4);
        if (S == (SlabCfg<KL>::kSlabG32)) {
            switch (a.v_mode) {
            case 4: slab_value_quant<4, NREP, kSteps32, KL>(a, kv, t0, t_end, lg, acc, tid); break;
            case 2: slab_value_quant<2, NREP, kSteps32, KL>(a, kv, t0, t_end, lg, acc, tid); break;
            case 1: slab_value_quant<1, NREP, kSteps32, KL>(a, kv, t0, t_end, lg, acc, tid); break;
            default: slab_value_quant<3, NREP, kSteps32, KL>(a, kv, t0, t_end, lg, acc, tid); break;
            }
        } else {
            switch (a.v_mode) {
            case 4: slab_value_quant<4, NREP, kStepsRef3, KL>(a, kv, t0, t_end, lg, acc, tid); break;
            case 2: slab_value_quant<2, NREP, kStepsRef3, KL>(a, kv, t0, t_end, lg, acc, tid); break;
            case 1: slab_value_quant<1, NREP, kStepsRef3, KL>(a, kv, t0, t_end, lg, acc, tid); break;
            default: slab_value_quant<3, NREP, kStepsRef3, KL>(a, kv, t0, t_end, lg, acc, tid); break;
            }
        }
    }
    {
        const int grp = tid % 4, tok = tid / 4;
        const int64_t j_begin = t0 > a.v_tokens ? t0 - a.v_tokens : 0;
        const int64_t j_end = t1 - a.v_tokens < v_len ? t1 - a.v_tokens : v_len;
        const uint16_t *vt = a.v_tail + kv * a.vt_bs + grp * 32;
        for (int64_t j = j_begin + tok; j < j_end; j += (SlabCfg<KL>::kThreads) / 4) {
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
    for (int idx = tid; idx < NREP * kFusedD; idx += (SlabCfg<KL>::kThreads)) {
        const int h = idx / kFusedD, c = idx % kFusedD;
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < (SlabCfg<KL>::kWaves); w++) o += red[(w * NREP + h) * kFusedD + c];
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


}  // namespace fused

// The launch of a large single-pass step (attn_step_mfma in dequant_gemv.hip): matrix-core tiles over the quantized
// positions [0, a.tokens) plus `tail_blocks` vector-ALU slabs (8 lanes per key row, 256 threads; `f` describes them:
// f.t_begin = a.tokens, f.slab0 = the number of tiles) over the rest.  k_bits in {1, 2, 4} (tiles of 1024 positions,
// a.tokens a multiple of 32) or 3 = the reference's 3-bit words (tiles of 1408, a.tokens a multiple of 352); v_mode
// in {1, 2, 4, 30 (dense 3-bit)}.
// coop (k_bits 1, 2, 4 only): a block's four waves share one tile -- a quarter of the channel rows each in the key
// phase, then 256 positions each as a slab of its own (four workspace slabs per tile) -- for steps with too few
// (query head, tile) pairs to fill the GPU with one wave each.
int launch_attn_step_mfma(const AttnSlabArgs &a, const fused::FusedArgs &f, int k_bits, bool coop, int v_mode, int64_t samples,
                          int64_t tail_blocks, hipStream_t stream);
// grid and block of that launch (KVMIX_ERR_SHAPE for sizes the kernel does not take: fewer positions than one tile,
// not whole groups, too many blocks for a grid)
int plan_attn_slab_mfma(int k_mode, bool coop, int64_t tokens, int64_t samples, int64_t tail_blocks, unsigned grid[3],
                        unsigned block[3]);

}  // namespace kvmix
