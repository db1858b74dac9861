/*
 * kvmix_oracle.c -- CPU restatement of the KVmix KV-cache hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels are
 * compared against (tests/, the smoke check, and the CPU-baseline leg of the
 * benchmark).  The product path never links, loads or calls it.
 *
 * It follows the reference's CUDA sources as text, evaluated in IEEE-754
 * binary32 (no fast-math, no flush-to-zero):
 *   quant_cuda/csrc/quantization_cuda.cu:540-721     one-shot quantize + pack
 *   quant_cuda/csrc/quantization_cuda.cu:12-185,298-411   key append variant
 *   quant_cuda/csrc/quantization_cuda.cu:188-296,413-537  value append variant
 *   quant_cuda/csrc/dequantization_gemv_cuda.cu:7-248     fused dequant GEMV
 *
 * Pinning (what fixes each function besides this restatement) lives in
 * tests/test_oracle_*.py: closed-form known answers (grids mn + k*s, hand-packed
 * words), brute-force pack/unpack inverses, the |dequant - x| <= scale/2 bound,
 * and agreement of the GEMV with a float64 dense matmul.  The reference holds no
 * golden vectors for this path.
 *
 * Parity unpinned (cannot be fixed without running the reference on NVIDIA
 * hardware): the effect of nvcc --use_fast_math (approximate divide, FTZ) on
 * codes within 2 ulp of a rounding tie, and the exact order of the 32-lane
 * shuffle tree is restated literally here but only compared within tolerance.
 *
 * Plain C99 + OpenMP (the OpenMP pragmas only parallelise independent rows; the
 * arithmetic per row is scalar and sequential).
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define KVO_OK 0
#define KVO_ERR_BITS -1
#define KVO_ERR_GROUP3 -2
#define KVO_ERR_DIVISIBLE -3
#define KVO_ERR_HEADS -4
#define KVO_ERR_ALLOC -5

/* ------------------------------------------------------------------------- */
/* fp16 <-> fp32 (binary16, round-to-nearest-even on the way down)            */
/* ------------------------------------------------------------------------- */

float kvo_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal half -> normal float */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t kvo_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) { /* inf / nan */
        if (absx > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((absx >> 13) & 0x3FFu));
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx >= 0x477FF000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx < 0x33000001u) { /* <= 2^-25 rounds to zero (tie goes to even = 0) */
        return (uint16_t)sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    uint32_t shift;
    uint32_t base;
    if (e < -14) { /* subnormal result: value = m * 2^(e-23), unit 2^-24 */
        shift = (uint32_t)(13 + (-14 - e));
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7FFFFFu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half_ulp = 1u << (shift - 1);
    uint32_t r = base + q;
    if (rem > half_ulp || (rem == half_ulp && (r & 1u))) r++;
    return (uint16_t)(sign | r);
}

void kvo_half_to_float_n(const uint16_t *src, float *dst, int64_t n)
{
    for (int64_t i = 0; i < n; i++) dst[i] = kvo_half_to_float(src[i]);
}

void kvo_float_to_half_n(const float *src, uint16_t *dst, int64_t n)
{
    for (int64_t i = 0; i < n; i++) dst[i] = kvo_float_to_half(src[i]);
}

/* ------------------------------------------------------------------------- */
/* shared scalar pieces                                                      */
/* ------------------------------------------------------------------------- */

/* float -> int32 the way the GPU conversion instruction does it: NaN -> 0,
 * saturating.  (C's cast is undefined for those inputs.)                    */
static int32_t cvt_sat_i32(float v)
{
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}

/* q = clamp(roundf((x - mn) / scale), 0, hi)   quantization_cuda.cu:578-581,590-592 */
static uint32_t quantize_one(float x, float mn, float scale, int hi)
{
    float normalized = (x - mn) / scale;
    int32_t q = cvt_sat_i32(roundf(normalized));
    if (q > hi) q = hi;
    if (q < 0) q = 0;
    return (uint32_t)q;
}

static int values_per_word(int bits) { return bits == 3 ? 11 : 32 / bits; }

static int bits_ok(int bits) { return bits == 1 || bits == 2 || bits == 3 || bits == 4; }

/* min / max of one group with fminf/fmaxf NaN-ignoring semantics and the
 * +-FLT_MAX start values (quantization_cuda.cu:555-565).                     */
static void group_min_max(const float *x, int n, float *mn, float *mx)
{
    float lo = FLT_MAX, hi = -FLT_MAX;
    for (int i = 0; i < n; i++) {
        lo = fminf(lo, x[i]);
        hi = fmaxf(hi, x[i]);
    }
    *mn = lo;
    *mx = hi;
}

/* Quantize and pack one row of `steps` values whose groups run along the row.
 * bits 1/2/4: value i of a word sits at bit i*bits.  bits 3 (the reference's
 * 11-per-word format): ten 3-bit codes at bits 0..29, the 11th clamped to 0..3
 * at bits 30..31 (quantization_cuda.cu:573-584,617-621).
 * scale_mode 0: scale_out = (mx-mn) * (1.0f/qmax)  -- what ATen's CUDA
 *               division-by-a-scalar computes for quantization_cuda.cu:711
 *               (torch 2.5.1, aten/src/ATen/native/cuda/BinaryDivTrueKernel.cu:
 *               a CPU-scalar divisor is turned into a multiply by its fp32
 *               reciprocal);
 * scale_mode 1: scale_out = (mx-mn) / qmax          -- the in-kernel form the
 *               append variants store (quantization_cuda.cu:50-51,150-151,234).
 * The codes always use the in-kernel true division (quantization_cuda.cu:571). */
static void quant_row(const float *x, int64_t steps, int g, int bits, int scale_mode,
                      uint32_t *code, float *scale_out, float *min_out)
{
    const int qmax = (1 << bits) - 1;
    const int vpw = values_per_word(bits);
    const int64_t groups = steps / g;
    const int64_t words = steps / vpw;
    for (int64_t w = 0; w < words; w++) code[w] = 0;
    for (int64_t gi = 0; gi < groups; gi++) {
        const float *xg = x + gi * g;
        float mn, mx;
        group_min_max(xg, g, &mn, &mx);
        float scale = (mx - mn) / (float)qmax;
        min_out[gi] = mn;
        scale_out[gi] = scale_mode == 0 ? (mx - mn) * (1.0f / (float)qmax) : scale;
        for (int i = 0; i < g; i++) {
            int64_t idx = gi * g + i;
            int hi = qmax;
            int shift;
            if (bits == 3) {
                int pos = (int)(idx % 11); /* == i, because g == 11 */
                hi = pos < 10 ? 7 : 3;
                shift = pos < 10 ? pos * 3 : 30;
            } else {
                shift = (int)(idx % vpw) * bits;
            }
            uint32_t q = quantize_one(xg[i], mn, scale, hi);
            code[idx / vpw] |= q << shift;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* quantize_pack_last_dim_cuda            quantization_cuda.cu:631-721        */
/* ------------------------------------------------------------------------- */

int kvo_quantize_pack_last_dim(const float *x, int64_t rows, int64_t steps, int group_length,
                               int quant_bits, int scale_mode, int32_t *code, float *scale, float *mn)
{
    if (!bits_ok(quant_bits)) return KVO_ERR_BITS;
    if (quant_bits == 3) {
        if (group_length != 11) return KVO_ERR_GROUP3;
        if (steps % 11 != 0) return KVO_ERR_DIVISIBLE;
    } else {
        if (group_length <= 0 || steps % group_length != 0) return KVO_ERR_DIVISIBLE;
        if (steps % (32 / quant_bits) != 0) return KVO_ERR_DIVISIBLE;
    }
    const int vpw = values_per_word(quant_bits);
    const int64_t words = steps / vpw, groups = steps / group_length;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        quant_row(x + r * steps, steps, group_length, quant_bits, scale_mode,
                  (uint32_t *)code + r * words, scale + r * groups, mn + r * groups);
    }
    return KVO_OK;
}

/* Same, fp16 in / fp16 scale+min out, including the up-cast the reference does
 * on the host (quantization_cuda.cu:641-642,715-718).  Used as the timed CPU
 * baseline so that no numpy conversion sits inside the timed region.          */
int kvo_quantize_pack_last_dim_f16(const uint16_t *x, int64_t rows, int64_t steps, int group_length,
                                   int quant_bits, int scale_mode, int32_t *code, uint16_t *scale,
                                   uint16_t *mn)
{
    if (!bits_ok(quant_bits)) return KVO_ERR_BITS;
    if (quant_bits == 3) {
        if (group_length != 11) return KVO_ERR_GROUP3;
        if (steps % 11 != 0) return KVO_ERR_DIVISIBLE;
    } else {
        if (group_length <= 0 || steps % group_length != 0) return KVO_ERR_DIVISIBLE;
        if (steps % (32 / quant_bits) != 0) return KVO_ERR_DIVISIBLE;
    }
    const int vpw = values_per_word(quant_bits);
    const int64_t words = steps / vpw, groups = steps / group_length;
    int failed = 0;
#pragma omp parallel
    {
        float *xf = (float *)malloc(sizeof(float) * (size_t)(steps + 2 * groups + 2));
        if (!xf) {
#pragma omp atomic write
            failed = 1;
        } else {
            float *sc = xf + steps, *lo = sc + groups;
#pragma omp for schedule(static)
            for (int64_t r = 0; r < rows; r++) {
                kvo_half_to_float_n(x + r * steps, xf, steps);
                quant_row(xf, steps, group_length, quant_bits, scale_mode, (uint32_t *)code + r * words, sc,
                          lo);
                kvo_float_to_half_n(sc, scale + r * groups, groups);
                kvo_float_to_half_n(lo, mn + r * groups, groups);
            }
            free(xf);
        }
    }
    return failed ? KVO_ERR_ALLOC : KVO_OK;
}

/* ------------------------------------------------------------------------- */
/* Dense 3-bit stream -- an EXTENSION with no counterpart in the reference     */
/* (the reference's 3-bit is the 11-per-word format above).  Same min / max /  */
/* scale / round / clamp arithmetic with qmax = 7 for every value; code i of a */
/* row occupies stream bits [3i, 3i+3), little-endian across uint32 words, so  */
/* 32 codes fill exactly three words.  group_length must be a multiple of 32.  */
/* Pinned only by closed forms and round trips (tests/test_oracle_dense3.py):  */
/* no reference parity is possible for this format.                            */
/* ------------------------------------------------------------------------- */

int kvo_quantize_pack_dense3(const float *x, int64_t rows, int64_t steps, int group_length,
                             int scale_mode, int32_t *code, float *scale, float *mn)
{
    if (group_length <= 0 || group_length % 32 != 0) return KVO_ERR_DIVISIBLE;
    if (steps % group_length != 0) return KVO_ERR_DIVISIBLE;
    const int64_t words = steps * 3 / 32, groups = steps / group_length;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        uint32_t *cw = (uint32_t *)code + r * words;
        for (int64_t w = 0; w < words; w++) cw[w] = 0;
        for (int64_t gi = 0; gi < groups; gi++) {
            const float *xg = x + r * steps + gi * group_length;
            float lo, hi;
            group_min_max(xg, group_length, &lo, &hi);
            const float sc = (hi - lo) / 7.0f;
            mn[r * groups + gi] = lo;
            scale[r * groups + gi] = scale_mode == 0 ? (hi - lo) * (1.0f / 7.0f) : sc;
            for (int i = 0; i < group_length; i++) {
                const int64_t bit = (gi * group_length + i) * 3;
                const uint64_t q = quantize_one(xg[i], lo, sc, 7);
                const uint64_t spread = q << (bit % 32);
                cw[bit / 32] |= (uint32_t)spread;
                if ((bit % 32) > 29) cw[bit / 32 + 1] |= (uint32_t)(spread >> 32);
            }
        }
    }
    return KVO_OK;
}

static uint32_t extract_dense3(const uint32_t *row_words, int64_t n)
{
    const int64_t bit = 3 * n;
    uint64_t two = row_words[bit / 32];
    if ((bit % 32) > 29) two |= (uint64_t)row_words[bit / 32 + 1] << 32;
    return (uint32_t)(two >> (bit % 32)) & 7u;
}

void kvo_unpack_dense3_row(const int32_t *code, int64_t n_values, int32_t *out)
{
    for (int64_t n = 0; n < n_values; n++) out[n] = (int32_t)extract_dense3((const uint32_t *)code, n);
}

/* dense-3 form of kvo_quantized_gemm (sequential fp32 accumulation; float64 side outputs) */
int kvo_quantized_gemm_dense3(int group_size, const uint16_t *fA, int64_t a_batch_stride, int64_t lda,
                              const int32_t *qB, const uint16_t *scales, const uint16_t *zeros,
                              int64_t BH, int heads_per_kv, int64_t M, int64_t K, int64_t N,
                              uint16_t *out, double *out64, double *abs64)
{
    if (heads_per_kv <= 0 || BH % heads_per_kv != 0) return KVO_ERR_HEADS;
    if (group_size <= 0 || group_size % 32 != 0 || N % group_size != 0) return KVO_ERR_DIVISIBLE;
    const int64_t words = N * 3 / 32, groups = N / group_size;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t s = 0; s < BH; s++) {
        for (int64_t m = 0; m < M; m++) {
            const int64_t kv = s / heads_per_kv;
            const uint16_t *x = fA + s * a_batch_stride + m * lda;
            for (int64_t n = 0; n < N; n++) {
                float acc = 0.f;
                double acc64 = 0.0, a64 = 0.0;
                for (int64_t k = 0; k < K; k++) {
                    const uint32_t *row = (const uint32_t *)qB + (kv * K + k) * words;
                    const float c = (float)extract_dense3(row, n);
                    const float sc = kvo_half_to_float(scales[(kv * K + k) * groups + n / group_size]);
                    const float zr = kvo_half_to_float(zeros[(kv * K + k) * groups + n / group_size]);
                    const float xv = kvo_half_to_float(x[k]);
                    const float wv = sc * c + zr;
                    acc += wv * xv;
                    const double wd = (double)sc * (double)c + (double)zr;
                    acc64 += wd * (double)xv;
                    a64 += fabs(wd) * fabs((double)xv);
                }
                const int64_t o = (s * M + m) * N + n;
                if (out) out[o] = kvo_float_to_half(acc);
                if (out64) out64[o] = acc64;
                if (abs64) abs64[o] = a64;
            }
        }
    }
    return KVO_OK;
}

/* ------------------------------------------------------------------------- */
/* process_key_quantization_cuda          quantization_cuda.cu:298-411        */
/*   x_new [rows, new_steps] (rows = B*H*D), groups along the steps           */
/*   out_* [rows, old + new]; the old part is a copy of prev_*                */
/* ------------------------------------------------------------------------- */

int kvo_process_key(const float *x_new, int64_t rows, int64_t new_steps, const int32_t *prev_code,
                    int64_t old_words, const float *prev_scale, const float *prev_min,
                    int64_t old_groups, int group_length, int quant_bits, int32_t *out_code,
                    float *out_scale, float *out_min)
{
    if (!bits_ok(quant_bits)) return KVO_ERR_BITS;
    if (quant_bits == 3) {
        if (group_length != 11) return KVO_ERR_GROUP3;
        if (new_steps % 11 != 0) return KVO_ERR_DIVISIBLE;
    } else if (group_length <= 0 || new_steps % group_length != 0) {
        return KVO_ERR_DIVISIBLE;
    }
    const int qmax = (1 << quant_bits) - 1;
    const int vpw = values_per_word(quant_bits);
    const int64_t new_words = new_steps / vpw, new_groups = new_steps / group_length;
    const int64_t tw = old_words + new_words, tg = old_groups + new_groups;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const float *x = x_new + r * new_steps;
        uint32_t *cw = (uint32_t *)out_code + r * tw + old_words;
        float *sc = out_scale + r * tg + old_groups;
        float *lo = out_min + r * tg + old_groups;
        memcpy(out_code + r * tw, prev_code + r * old_words, sizeof(int32_t) * (size_t)old_words);
        memcpy(out_scale + r * tg, prev_scale + r * old_groups, sizeof(float) * (size_t)old_groups);
        memcpy(out_min + r * tg, prev_min + r * old_groups, sizeof(float) * (size_t)old_groups);
        for (int64_t gi = 0; gi < new_groups; gi++) {
            float mn, mx;
            group_min_max(x + gi * group_length, group_length, &mn, &mx);
            sc[gi] = (mx - mn) / (float)qmax; /* :49-51, :149-151 */
            lo[gi] = mn;
        }
        if (quant_bits == 3) { /* fused kernel :108-185: one word per 11-group */
            for (int64_t gi = 0; gi < new_groups; gi++) {
                uint32_t word = 0;
                for (int i = 0; i < 11; i++) {
                    uint32_t q = quantize_one(x[gi * 11 + i], lo[gi], sc[gi], i < 10 ? 7 : 3);
                    word |= q << (i < 10 ? 3 * i : 30);
                }
                cw[gi] = word;
            }
        } else { /* :58-105: the whole word uses the group of its first value (:88-90) */
            for (int64_t w = 0; w < new_words; w++) {
                const int64_t gi = (w * vpw) / group_length;
                uint32_t word = 0;
                for (int i = 0; i < vpw; i++)
                    word |= quantize_one(x[w * vpw + i], lo[gi], sc[gi], qmax) << (i * quant_bits);
                cw[w] = word;
            }
        }
    }
    return KVO_OK;
}

/* ------------------------------------------------------------------------- */
/* process_value_quantization_cuda        quantization_cuda.cu:413-537        */
/*   x_new [rows, new_steps, head_dim] (rows = B*H), groups along head_dim    */
/* The 3-bit branch is the reference's "placeholder": plain i*3 shifts with   */
/* qmax 7 for all 11 values, so the 11th code keeps only its low two bits in  */
/* the 32-bit word (:282-289 with j == 10).                                   */
/* ------------------------------------------------------------------------- */

int kvo_process_value(const float *x_new, int64_t rows, int64_t new_steps, int64_t head_dim,
                      const int32_t *prev_code, const float *prev_scale, const float *prev_min,
                      int64_t old_steps, int group_length, int quant_bits, int32_t *out_code,
                      float *out_scale, float *out_min)
{
    if (!bits_ok(quant_bits)) return KVO_ERR_BITS;
    if (quant_bits == 3) {
        if (group_length != 11) return KVO_ERR_GROUP3;
        if (head_dim % 11 != 0) return KVO_ERR_DIVISIBLE;
    } else if (group_length <= 0 || head_dim % group_length != 0) {
        return KVO_ERR_DIVISIBLE;
    }
    const int qmax = (1 << quant_bits) - 1;
    const int vpw = values_per_word(quant_bits);
    const int64_t wpt = head_dim / vpw;          /* words per time step  */
    const int64_t gpt = head_dim / group_length; /* groups per time step */
    const int64_t total = old_steps + new_steps;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        memcpy(out_code + r * total * wpt, prev_code + r * old_steps * wpt,
               sizeof(int32_t) * (size_t)(old_steps * wpt));
        memcpy(out_scale + r * total * gpt, prev_scale + r * old_steps * gpt,
               sizeof(float) * (size_t)(old_steps * gpt));
        memcpy(out_min + r * total * gpt, prev_min + r * old_steps * gpt,
               sizeof(float) * (size_t)(old_steps * gpt));
        for (int64_t t = 0; t < new_steps; t++) {
            const float *xt = x_new + (r * new_steps + t) * head_dim;
            float *sc = out_scale + (r * total + old_steps + t) * gpt;
            float *lo = out_min + (r * total + old_steps + t) * gpt;
            uint32_t *cw = (uint32_t *)out_code + (r * total + old_steps + t) * wpt;
            for (int64_t gi = 0; gi < gpt; gi++) {
                float mn, mx;
                group_min_max(xt + gi * group_length, group_length, &mn, &mx);
                sc[gi] = (mx - mn) / (float)qmax;
                lo[gi] = mn;
            }
            for (int64_t w = 0; w < wpt; w++) {
                int64_t gi = (w * vpw) / group_length;
                uint32_t word = 0;
                for (int j = 0; j < vpw; j++) {
                    uint32_t q = quantize_one(xt[w * vpw + j], lo[gi], sc[gi], qmax);
                    word |= q << (j * quant_bits); /* 3-bit, j == 10: bits past 31 fall off */
                }
                cw[w] = word;
            }
        }
    }
    return KVO_OK;
}

/* ------------------------------------------------------------------------- */
/* unpack / dequantize helpers                                               */
/* ------------------------------------------------------------------------- */

/* value at position pos (0..vpw-1) of a packed word; unpack order of
 * dequantization_gemv_cuda.cu:81-105                                         */
static uint32_t extract_code(uint32_t word, int pos, int bits)
{
    if (bits == 3) return pos < 10 ? (word >> (3 * pos)) & 7u : (word >> 30) & 3u;
    return (word >> (pos * bits)) & ((1u << bits) - 1u);
}

void kvo_unpack_row(const int32_t *code, int64_t words, int bits, int32_t *out)
{
    const int vpw = values_per_word(bits);
    for (int64_t w = 0; w < words; w++)
        for (int p = 0; p < vpw; p++) out[w * vpw + p] = (int32_t)extract_code((uint32_t)code[w], p, bits);
}

/* ------------------------------------------------------------------------- */
/* quantized_gemm                  dequantization_gemv_cuda.cu:7-124,127-248  */
/*   fA     [BH, M, K] fp16, row stride lda (elements) between the M rows and */
/*          a_batch_stride between (b,h) samples                              */
/*   qB     [BHkv, K, N/vpw]   scales, zeros [BHkv, K, N/g] fp16              */
/*   out    [BH, M, N] fp16                                                   */
/* out[n] = sum_k x[k] * (scale[k, grp] * code[k, n] + zero[k, grp]) with     */
/* grp = (first value of n's word) / g  (:23-24), head mapping :29-30.        */
/* mode 0: the reference's arithmetic order -- 32 lanes, lane l owns          */
/*         k = 128c + 4l + s, fma(scale, code, zero) then fma into the lane's */
/*         fp32 accumulator, shuffle-down tree 16,8,4,2,1, fp16 store.        */
/* mode 1: plain sequential fp32 accumulation over k (dequant-then-matmul).   */
/* out64 (optional): the same sum in float64, unrounded.                      */
/* abs64 (optional): sum_k |x[k]| * |w[k,n]| in float64 (error-bound scale).  */
/* The reference only produces row m == 0 (the kernel ignores blockIdx.z);    */
/* rows m >= 1 are defined here as the same formula on fA's row m.            */
/* ------------------------------------------------------------------------- */

int kvo_quantized_gemm(int group_size, const uint16_t *fA, int64_t a_batch_stride, int64_t lda,
                       const int32_t *qB, const uint16_t *scales, const uint16_t *zeros, int bits,
                       int64_t BH, int heads_per_kv, int64_t M, int64_t K, int64_t N, int mode,
                       uint16_t *out, double *out64, double *abs64)
{
    if (!bits_ok(bits)) return KVO_ERR_BITS;
    if (bits == 3 && group_size != 11) return KVO_ERR_GROUP3;
    if (heads_per_kv <= 0 || BH % heads_per_kv != 0) return KVO_ERR_HEADS;
    const int vpw = values_per_word(bits);
    if (group_size <= 0 || N % group_size != 0 || N % vpw != 0) return KVO_ERR_DIVISIBLE;
    const int64_t words = N / vpw, groups = N / group_size;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t s = 0; s < BH; s++) {
        for (int64_t m = 0; m < M; m++) {
            const int64_t kv = s / heads_per_kv;
            const uint16_t *x = fA + s * a_batch_stride + m * lda;
            const uint32_t *wq = (const uint32_t *)qB + kv * K * words;
            const uint16_t *sc = scales + kv * K * groups;
            const uint16_t *zr = zeros + kv * K * groups;
            for (int64_t w = 0; w < words; w++) {
                const int64_t grp = (w * vpw) / group_size;
                float lane_acc[32][32];
                float seq_acc[32];
                double acc64[32], a64[32];
                memset(lane_acc, 0, sizeof lane_acc);
                memset(seq_acc, 0, sizeof seq_acc);
                memset(acc64, 0, sizeof acc64);
                memset(a64, 0, sizeof a64);
                for (int64_t k = 0; k < K; k++) {
                    const float xv = kvo_half_to_float(x[k]);
                    const float scv = kvo_half_to_float(sc[k * groups + grp]);
                    const float zv = kvo_half_to_float(zr[k * groups + grp]);
                    const uint32_t word = wq[k * words + w];
                    const int lane = (int)((k % 128) / 4);
                    for (int p = 0; p < vpw; p++) {
                        const float c = (float)extract_code(word, p, bits);
                        if (mode == 0) {
                            lane_acc[lane][p] = fmaf(fmaf(scv, c, zv), xv, lane_acc[lane][p]);
                        } else {
                            float wv = scv * c + zv;
                            seq_acc[p] += wv * xv;
                        }
                        if (out64 || abs64) {
                            double wd = (double)scv * (double)c + (double)zv;
                            acc64[p] += wd * (double)xv;
                            a64[p] += fabs(wd) * fabs((double)xv);
                        }
                    }
                }
                for (int p = 0; p < vpw; p++) {
                    float r;
                    if (mode == 0) {
                        float v[32];
                        for (int l = 0; l < 32; l++) v[l] = lane_acc[l][p];
                        for (int off = 16; off > 0; off >>= 1) {
                            float nv[32];
                            for (int l = 0; l < 32; l++) nv[l] = v[l] + (l + off < 32 ? v[l + off] : v[l]);
                            memcpy(v, nv, sizeof v);
                        }
                        r = v[0];
                    } else {
                        r = seq_acc[p];
                    }
                    const int64_t o = (s * M + m) * N + w * vpw + p;
                    if (out) out[o] = kvo_float_to_half(r);
                    if (out64) out64[o] = acc64[p];
                    if (abs64) abs64[o] = a64[p];
                }
            }
        }
    }
    return KVO_OK;
}

/* Dequantize a packed [rows, K... ] tensor to fp32: w[k, n] = fp32(scale)*code + fp32(zero),
 * evaluated as one multiply and one add (no contraction).                    */
int kvo_dequantize(const int32_t *qB, const uint16_t *scales, const uint16_t *zeros, int bits,
                   int group_size, int64_t rows, int64_t N, float *out)
{
    if (!bits_ok(bits)) return KVO_ERR_BITS;
    const int vpw = values_per_word(bits);
    if (group_size <= 0 || N % group_size != 0 || N % vpw != 0) return KVO_ERR_DIVISIBLE;
    const int64_t words = N / vpw, groups = N / group_size;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t n = 0; n < N; n++) {
            const int64_t w = n / vpw;
            const int64_t grp = (w * vpw) / group_size;
            const volatile float prod = kvo_half_to_float(scales[r * groups + grp]) *
                                        (float)extract_code((uint32_t)qB[r * words + w], (int)(n % vpw), bits);
            out[r * N + n] = prod + kvo_half_to_float(zeros[r * groups + grp]);
        }
    }
    return KVO_OK;
}

int kvo_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void kvo_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
