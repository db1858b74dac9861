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
#include "fused_slab.h"

#include <cstdlib>

namespace kvmix {

using namespace fused;

// the stand-alone slab kernel: 16 lanes per key row, 512 threads, slabs of 512 positions (704 with the reference's
// 3-bit keys); grid = slabs x head groups x kv heads blocks, one-dimensional
#ifndef KVMIX_FUSED_KEY_LANES
#define KVMIX_FUSED_KEY_LANES 16
#endif
constexpr int kKeyLanes = KVMIX_FUSED_KEY_LANES;
constexpr int kFusedThreads = SlabCfg<kKeyLanes>::kThreads;
constexpr int kSlabG32 = SlabCfg<kKeyLanes>::kSlabG32;
constexpr int kSlabRef3 = SlabCfg<kKeyLanes>::kSlabRef3;

template <int NREP>
__global__ void __launch_bounds__(kFusedThreads) attn_fused_slab(FusedArgs a)
{
    __shared__ float smem[SlabCfg<kKeyLanes>::lds_floats(NREP)];
    attn_fused_slab_body<NREP, kKeyLanes>(a, blockIdx.x, gridDim.x, threadIdx.x, smem);
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

// How a row's positions are divided into slabs.  Keys of 1, 2 or 4 bits or in the reference's 3-bit words, with
// at least one tile quantized on both sides, take the positions [0, min(k_tokens, v_tokens)) through the matrix-core
// tiles (attn_slab_mfma_body: 1024 positions, the formats of gemv_cols_mfma2 and gemv_rows_mfma; attn_slab_ref3_body:
// 1408 positions, gemv_cols3's arithmetic for the keys) -- one wave per tile, or, for steps with few (query head,
// tile) pairs, the four waves of a block per tile -- and the rest -- the fp16 tails, and the few positions quantized
// on one side only when keys and values are quantized to different lengths -- through slabs of the vector-ALU kind
// that run as trailing blocks of the same launch (256 threads, 256 positions each); everything else goes through
// attn_fused_slab (512 threads) from position 0.
constexpr int64_t kSmallStepEntries = 1 << 19, kSmallStepEntriesRef3 = 360000;  // (see kvmix_decode_attention_fused_plan)
constexpr int64_t kSlabMfmaMinWaves = 512;   // one wave per tile from this many (query head, tile) pairs on
constexpr int64_t kSlabRef3MaxPairs = 768;   // the reference's 3-bit keys: the single pass is ahead up to here
struct FusedLayout {
    bool mfma;
    bool coop;           // four waves per tile (attn_step_mfma<.., true>): four workspace slabs per tile
    int64_t tiles;       // slabs of the matrix-core kernel (first in the workspace)
    int64_t tail_slabs;  // vector-ALU slabs, from position t_begin on
    int64_t t_begin;
    int slab;            // positions per vector-ALU slab
    int64_t slabs() const { return tiles + tail_slabs; }
};

// With fewer (query head, tile) pairs than this, four waves share a tile (attn_step_mfma<.., true>).  Measured,
// one wave per tile -> four (us, Llama-2-7B heads): 4-bit keys 4 x 2304: 30.3 -> 20.1, 1 x 4096: 18.5 -> 13.8 (those two
// against the vector-ALU slabs, which took these sizes before), 4 x 4224 (512 pairs): 26.1 -> 29.7, 8 x 2304 (768):
// 27.7 -> 34.1; reference 3-bit keys 8 x 2304 (512 pairs): 34.6 -> 31.3, 8 x 4224 (768): 38.3 -> 46.6.  With the
// reference's 3-bit keys and fewer than 128 pairs the vector-ALU slabs stay ahead (2 x 1664: 21.2 against 23.1).
static int64_t coop_below(int km)
{
#ifdef KVMIX_EXPERIMENT
    if (const char *e = getenv("KVMIX_DBG_COOP_BELOW")) return atoll(e);
#endif
    return km == 3 ? kSlabRef3MaxPairs : kSlabMfmaMinWaves;
}
static bool coop_ok(int km, int64_t pairs)
{
#ifdef KVMIX_EXPERIMENT
    if (const char *e = getenv("KVMIX_DBG_COOP")) return atoi(e) != 0;
#endif
    return km == 3 ? pairs >= 128 : true;
}

static FusedLayout fused_layout(const kvmix_decode_attn_t *p)
{
    FusedLayout l{false, false, 0, fused_slabs(p), 0, fused_slab(p)};
    const int km = fused_key_mode(p), vm = fused_value_mode(p);
    const int vbits = vm == 3 ? 3 : vm;
    // positions quantized on both sides, in whole words of the keys and whole groups of the values; tiles of 1024
    // positions, or 1408 with the reference's 3-bit keys
    const int64_t unit = km == 3 ? 352 : 32, tile = km == 3 ? 1408 : 1024;
    const int64_t both = (p->k_tokens < p->v_tokens ? p->k_tokens : p->v_tokens) / unit * unit;
    const int64_t tiles = (both + tile - 1) / tile;
    if (both >= tile && (km == 1 || km == 2 || km == 3 || km == 4) && vm != 0 &&
        p->v_code_row_stride == kFusedD * vbits / 32 && p->v_sz_row_stride == kFusedD / 32 &&
        (kFusedD + 1) * p->k_code_row_stride < (1ll << 29) && (kFusedD + 1) * p->k_sz_row_stride < (1ll << 30) &&
        // (the value phase forms 32-bit byte offsets of code rows and 32-bit element offsets of scale rows)
        p->v_tokens * p->v_code_row_stride < (1ll << 30) && p->v_tokens * p->v_sz_row_stride < (1ll << 31) &&
        (p->samples * tiles >= coop_below(km) || coop_ok(km, p->samples * tiles))) {
        l.mfma = true;
        l.coop = p->samples * tiles < coop_below(km);
        l.tiles = l.coop ? 4 * tiles : tiles;
        l.t_begin = both;
        l.slab = km == 3 ? SlabCfg<8>::kSlabRef3 : SlabCfg<8>::kSlabG32;
        l.tail_slabs = (fused_width(p) - both + l.slab - 1) / l.slab;
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
    // Which form is faster (MI355X, Llama-2-7B heads, graph-replayed; four launches -> single pass, us).  Keys of 1,
    // 2 or 4 bits: the single pass wherever the matrix-core tiles take it (1 x 4096: 29 -> 14, 4 x 2304 4/4 bits: 32 ->
    // 20, 2/2 bits: 30 -> 18; 8 x 8192: 4/4 bits 71 -> 61, 2/2 bits 54 -> 45, 2/4 bits 63 -> 52; 16 x 8192: 129 -> 116,
    // 90 -> 80, 110 -> 98), else (rows under 1024 quantized positions) the vector-ALU slabs up to about 2^19 (query head
    // x position) entries.  The reference's 3-bit keys: on the tiles up to 768 (query head, tile) pairs (4 x 4224: 37 ->
    // 27, 8 x 4224: 47 -> 38, 4 x 8192: 49 -> 40); behind beyond (8 x 8192: 69 -> 72, 16 x 8192: 124 -> 140: the key phase
    // of a tile is vector arithmetic over all 128 rows in a block that also holds the value phase's registers);
    // without tiles the vector-ALU slabs up to 360 000 entries.
    {
        const int64_t entries = p->samples * fused_width(p);
        const bool ref3 = p->k_tokens > 0 && fused_key_mode(p) == 3;
        const int64_t pairs = p->samples * (lay.coop ? lay.tiles / 4 : lay.tiles);
        // (the positions past the tiles run as vector-ALU slabs: no more of them than those do well on their own)
        const int64_t rest = p->samples * (fused_width(p) - lay.t_begin);
        if (lay.mfma)
            plan->recommended = (!ref3 || pairs <= kSlabRef3MaxPairs) && rest <= kSmallStepEntries ? 1 : 0;
        else
            plan->recommended = entries <= (ref3 ? kSmallStepEntriesRef3 : kSmallStepEntries) ? 1 : 0;
    }
    plan->matrix_tile_waves = lay.mfma ? (lay.coop ? 4 : 1) : 0;
    plan->matrix_tiles = lay.coop ? lay.tiles / 4 : lay.tiles;
    plan->slab_positions = lay.slab;
    plan->slab_begin = lay.t_begin;
    plan->slabs = lay.tail_slabs;
    if (lay.mfma) {
        // one launch: the tiles' blocks, then the slabs' blocks
        const int prc = plan_attn_slab_mfma(fused_key_mode(p), lay.coop, lay.t_begin, p->samples, lay.tail_slabs * p->samples,
                                            plan->matrix_grid, plan->matrix_block);
        if (prc != KVMIX_OK) return prc;
        plan->slab_blocks = lay.tail_slabs * p->samples;
        plan->launches++;
    } else if (lay.tail_slabs > 0) {
        plan->slab_blocks = lay.tail_slabs * p->samples;
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
    a.slab = lay.slab;
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
        m.tokens = lay.t_begin;
        m.heads_per_kv = p->heads_per_kv, m.heads = p->heads;
        m.slabs = (int)slabs;
        m.inv_sqrt_d = a.inv_sqrt_d;
        rc = launch_attn_step_mfma(m, a, k_mode, lay.coop, v_mode == 3 ? 30 : v_mode, p->samples, lay.tail_slabs * p->samples, st);
    } else if (lay.tail_slabs > 0) {
        const dim3 grid((unsigned)(lay.tail_slabs * kv_samples * p->heads_per_kv));
        hipLaunchKernelGGL(attn_fused_slab<1>, grid, dim3(kFusedThreads), 0, st, a);
        rc = launch_status();
    }
    if (rc != KVMIX_OK || (slabs == 1 && !lay.mfma)) return rc;  // a single slab of attn_fused_slab is normalised and stored by that kernel
    hipLaunchKernelGGL(attn_fused_merge, dim3((unsigned)p->samples), dim3(kFusedD), 0, st, a.ws_o, a.ws_ml, (int)slabs,
                       (uint16_t *)p->out, p->out_stride);
    return launch_status();
}
