// Group quantize + bit-pack kernels for the KV cache append path (gfx950).
//
// What is computed (per group of `group` consecutive values of the last dimension):
//   mn = min, mx = max            (fp32, NaN-ignoring like fminf/fmaxf)
//   scale = (mx - mn) / qmax      (IEEE fp32 division)
//   code_i = clamp(roundf((x_i - mn) / scale), 0, qmax)     roundf = ties away from zero
//   words  = codes packed LSB-first
// following quant_cuda/csrc/quantization_cuda.cu:540-629 of the reference.  Unlike the
// reference there is no fp32 staging copy of the input, no int32-per-element temporary
// and no second packing kernel: min/max, codes and words stay in registers.
//
// Three kernels:
//   quant_rows_g32_f16   fast path: fp16 input, group 32, four lanes per group, each lane
//                        one 128-bit load (8 halves); quad shuffles for min/max and packing.
//   quant_rows_generic   any group / dtype / format, one thread per lcm(group, codes-per-word)
//                        values, serial like the reference (used for group 11, fp32 input,
//                        unaligned rows).
//   quant_key_tokens     keys straight from the token-major fp16 tail: one thread per channel
//                        holds one group of tokens in registers (fuses the caller's transpose).
//   quant_key_tokens_slab  the same for D = 128 with aligned rows: a block takes a chunk of groups of 64
//                        channels through LDS and writes each channel row's results as contiguous pieces.

#include "kvmix_common.h"

#include <vector>

namespace kvmix {

#ifndef KVMIX_FLUSH_VALUE_PIECES
#define KVMIX_FLUSH_VALUE_PIECES 1
#endif
#ifndef KVMIX_FLUSH_IDX32
#define KVMIX_FLUSH_IDX32 0
#endif
constexpr int kFlushValuePieces = KVMIX_FLUSH_VALUE_PIECES;  // value half of the fused flush: 128-bit pieces per thread (more measured no faster)
constexpr bool kFlushIdx32 = KVMIX_FLUSH_IDX32 != 0;

struct QuantArgs {
    const void *x;
    uint32_t *code;
    void *scale;
    void *zero;
    int64_t outer, inner, steps;
    int64_t x_os, x_is;        // element strides of x
    int64_t c_os, c_is;        // word strides of code
    int64_t s_os, s_is;        // element strides of scale / zero
    int group;
    int bits;
    int fmt;
    int scale_mode;
    float inv_qmax;
};

template <typename T>
__device__ __forceinline__ float load_as_float(const T *p);
template <>
__device__ __forceinline__ float load_as_float<__half>(const __half *p)
{
    return __half2float(*p);
}
template <>
__device__ __forceinline__ float load_as_float<float>(const float *p)
{
    return *p;
}

template <typename T>
__device__ __forceinline__ void store_from_float(T *p, float v);
template <>
__device__ __forceinline__ void store_from_float<__half>(__half *p, float v)
{
    *p = __float2half_rn(v);
}
template <>
__device__ __forceinline__ void store_from_float<float>(float *p, float v)
{
    *p = v;
}

// ---------------------------------------------------------------------------------------
// generic: one thread per `unit` = lcm(group, codes per word) consecutive values
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) quant_rows_generic(QuantArgs a, int unit, int64_t units_per_row,
                                                          int64_t total_units)
{
    const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (u >= total_units) return;
    const int64_t row = u / units_per_row;
    const int64_t ur = u - row * units_per_row;
    const int64_t o = row / a.inner;
    const int64_t i = row - o * a.inner;
    const T *x = (const T *)a.x + o * a.x_os + i * a.x_is + ur * unit;
    const int qmax = (1 << a.bits) - 1;
    const bool ref3 = (a.bits == 3 && a.fmt != KVMIX_FMT_DENSE3);
    const bool wrap11 = a.fmt == KVMIX_FMT_REF3_WRAP;
    const int vpw = ref3 ? 11 : 32 / a.bits;  // dense3: handled by the bit buffer below
    const int groups_per_unit = unit / a.group;
    T *sc = (T *)a.scale + o * a.s_os + i * a.s_is + ur * groups_per_unit;
    T *zr = (T *)a.zero + o * a.s_os + i * a.s_is + ur * groups_per_unit;
    // words per unit: ref formats unit/vpw; dense3 unit*3/32
    const int64_t words_per_unit = (a.bits == 3 && !ref3) ? (int64_t)unit * 3 / 32 : unit / vpw;
    uint32_t *cw = a.code + o * a.c_os + i * a.c_is + ur * words_per_unit;

    uint64_t buf = 0;
    int filled = 0;
    int pos3 = 0;  // position inside an 11-code word (reference 3-bit format)
    for (int g = 0; g < groups_per_unit; g++) {
        const T *xg = x + (int64_t)g * a.group;
        float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
        for (int j = 0; j < a.group; j++) {
            float v = load_as_float<T>(xg + j);
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
        }
        const float range = mx - mn;
        const float scale = range / (float)qmax;
        const float rcp = quantize_rcp(scale);
        store_from_float<T>(sc + g, scale_for_output(range, scale, a.inv_qmax, a.scale_mode));
        store_from_float<T>(zr + g, mn);
        for (int j = 0; j < a.group; j++) {
            float v = load_as_float<T>(xg + j);
            if (ref3) {
                uint32_t q = quantize_code(v, mn, scale, rcp, (pos3 < 10 || wrap11) ? 7 : 3);
                if (pos3 == 10) q &= 3u;  // only two bits of the word are left
                buf |= (uint64_t)q << (pos3 < 10 ? 3 * pos3 : 30);
                if (++pos3 == 11) {
                    *cw++ = (uint32_t)buf;
                    buf = 0;
                    pos3 = 0;
                }
            } else {
                uint32_t q = quantize_code(v, mn, scale, rcp, qmax);
                buf |= (uint64_t)q << filled;
                filled += a.bits;
                if (filled >= 32) {
                    *cw++ = (uint32_t)buf;
                    buf >>= 32;
                    filled -= 32;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// fast path: fp16, group 32, 4 lanes per group, 8 halves (one 128-bit load) per lane.
// BITS = 1, 2, 4 (reference layout) or 3 with DENSE3 = true (bit-stream extension).
// ---------------------------------------------------------------------------------------
// A thread handles P pieces (P*256 threads apart, so every load instruction of a wave is one
// contiguous kilobyte): the P loads are issued first, then the pieces are processed one by one.
// With one piece per thread the kernel is bound by wave turnover (one load latency per wave
// lifetime); with several it streams.  IDX32: the group index fits 32 bits (no 64-bit divisions).
template <int BITS, int P, bool IDX32>
__device__ __forceinline__ void rows_g32_f16_body(const QuantArgs &a, int64_t groups_per_row,
                                                  int64_t total_groups, int64_t first_tid)
{
    const int j = (int)(first_tid & 3);
    bool active[P];
    int64_t o[P], i[P], gr[P];
    uint4 raw[P];
#pragma unroll
    for (int p = 0; p < P; p++) {
        int64_t g = (first_tid + (int64_t)p * 256) >> 2;
        active[p] = g < total_groups;
        if (!active[p]) g = total_groups - 1;  // keep the quad's shuffles convergent
        if constexpr (IDX32) {
            const uint32_t g32 = (uint32_t)g, gpr = (uint32_t)groups_per_row, inner = (uint32_t)a.inner;
            const uint32_t row = g32 / gpr;
            gr[p] = g32 - row * gpr;
            o[p] = row / inner;
            i[p] = row - (uint32_t)o[p] * inner;
        } else {
            const int64_t row = g / groups_per_row;
            gr[p] = g - row * groups_per_row;
            o[p] = row / a.inner;
            i[p] = row - o[p] * a.inner;
        }
        const __half *x = (const __half *)a.x + o[p] * a.x_os + i[p] * a.x_is + gr[p] * 32 + j * 8;
        raw[p] = *reinterpret_cast<const uint4 *>(x);
    }
#pragma unroll
    for (int p = 0; p < P; p++) {
        float v[8];
        {
            const uint32_t r[4] = {raw[p].x, raw[p].y, raw[p].z, raw[p].w};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                v[2 * t] = h16_to_f32((uint16_t)(r[t] & 0xffffu));
                v[2 * t + 1] = h16_to_f32((uint16_t)(r[t] >> 16));
            }
        }
        float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
#pragma unroll
        for (int t = 0; t < 8; t++) {
            mn = fminf(mn, v[t]);
            mx = fmaxf(mx, v[t]);
        }
        mn = fminf(mn, __shfl_xor(mn, 1));
        mx = fmaxf(mx, __shfl_xor(mx, 1));
        mn = fminf(mn, __shfl_xor(mn, 2));
        mx = fmaxf(mx, __shfl_xor(mx, 2));

        constexpr int qmax = (1 << BITS) - 1;
        const float range = mx - mn;
        const float scale = range / (float)qmax;
        const float rcp = quantize_rcp(scale);
        uint32_t piece = 0;  // this lane's 8 codes, 8*BITS bits
        uint32_t q8[8];
        quantize_codes<8>(v, mn, scale, rcp, [](int) { return qmax; }, q8);
#pragma unroll
        for (int t = 0; t < 8; t++) piece |= q8[t] << (t * BITS);

        const bool act = active[p];
        uint32_t *cw = a.code + o[p] * a.c_os + i[p] * a.c_is + gr[p] * BITS;  // BITS words per group of 32
        if (BITS == 4) {
            if (act) cw[j] = piece;
        } else if (BITS == 2) {
            const uint32_t other = __shfl_xor(piece, 1);
            if (act && (j & 1) == 0) cw[j >> 1] = piece | (other << 16);
        } else if (BITS == 1) {
            uint32_t w = piece << (8 * j);
            w |= __shfl_xor(w, 1);
            w |= __shfl_xor(w, 2);
            if (act && j == 0) cw[0] = w;
        } else {  // BITS == 3, bit stream: lane j holds stream bits [24j, 24j+24)
            const uint32_t next = __shfl_down(piece, 1);  // lane j+1's piece (unused for j == 3)
            uint32_t w;
            if (j == 0)
                w = piece | (next << 24);
            else if (j == 1)
                w = (piece >> 8) | (next << 16);
            else
                w = (piece >> 16) | (next << 8);
            if (act && j < 3) cw[j] = w;
        }
        if (act && j == 0) {
            __half *sc = (__half *)a.scale + o[p] * a.s_os + i[p] * a.s_is + gr[p];
            *sc = __float2half_rn(scale_for_output(range, scale, a.inv_qmax, a.scale_mode));
        }
        if (act && j == 1) {
            __half *zr = (__half *)a.zero + o[p] * a.s_os + i[p] * a.s_is + gr[p];
            *zr = __float2half_rn(mn);
        }
    }
}

constexpr int kRowsPieces = 4;  // pieces per thread in the streaming configuration

template <int BITS, int P, bool IDX32>
__global__ void __launch_bounds__(256) quant_rows_g32_f16(QuantArgs a, int64_t groups_per_row,
                                                          int64_t total_groups)
{
    rows_g32_f16_body<BITS, P, IDX32>(a, groups_per_row, total_groups,
                                      (int64_t)blockIdx.x * (256 * P) + threadIdx.x);
}

// ---------------------------------------------------------------------------------------
// large inputs, fp16, group 32: one thread per group (four 128-bit loads, no lane exchange),
// P groups per thread with the loads issued first; codes leave as one vector store per group.
// ---------------------------------------------------------------------------------------
template <int BITS, int P>
__device__ __forceinline__ void rows_g32_f16_stream_body(const QuantArgs &a, uint32_t groups_per_row,
                                                         int64_t total_groups, int64_t first)
{
    uint4 raw[P][4];
    int64_t o[P], i[P];
    uint32_t gr[P];
    bool active[P];
#pragma unroll
    for (int p = 0; p < P; p++) {
        int64_t g = first + (int64_t)p * 256;
        active[p] = g < total_groups;
        if (!active[p]) g = total_groups - 1;
        const int64_t row = g / groups_per_row;
        gr[p] = (uint32_t)(g - row * groups_per_row);
        o[p] = row / a.inner;
        i[p] = row - o[p] * a.inner;
        const uint4 *x = reinterpret_cast<const uint4 *>((const __half *)a.x + o[p] * a.x_os + i[p] * a.x_is + (int64_t)gr[p] * 32);
#pragma unroll
        for (int q = 0; q < 4; q++) raw[p][q] = x[q];
    }
#pragma unroll
    for (int p = 0; p < P; p++) {
        float v[32];
        float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t r[4] = {raw[p][q].x, raw[p][q].y, raw[p][q].z, raw[p][q].w};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                v[8 * q + 2 * t] = h16_to_f32((uint16_t)(r[t] & 0xffffu));
                v[8 * q + 2 * t + 1] = h16_to_f32((uint16_t)(r[t] >> 16));
            }
        }
#pragma unroll
        for (int t = 0; t < 32; t++) {
            mn = fminf(mn, v[t]);
            mx = fmaxf(mx, v[t]);
        }
        constexpr int qmax = (1 << BITS) - 1;
        const float range = mx - mn;
        const float scale = range / (float)qmax;
        const float rcp = quantize_rcp(scale);
        uint32_t w[BITS];
#pragma unroll
        for (int t = 0; t < BITS; t++) w[t] = 0;
#pragma unroll
        for (int t0 = 0; t0 < 32; t0 += 8) {
            uint32_t q8[8];
            quantize_codes<8>(v + t0, mn, scale, rcp, [](int) { return qmax; }, q8);
#pragma unroll
            for (int t = t0; t < t0 + 8; t++) {
                const uint32_t q = q8[t - t0];
                const int bit = t * BITS;
                w[bit >> 5] |= q << (bit & 31);
                if ((bit & 31) + BITS > 32) w[(bit >> 5) + 1] |= q >> (32 - (bit & 31));
            }
        }
        if (active[p]) {
            uint32_t *cw = a.code + o[p] * a.c_os + i[p] * a.c_is + (int64_t)gr[p] * BITS;
#pragma unroll
            for (int t = 0; t < BITS; t++) cw[t] = w[t];
            ((__half *)a.scale)[o[p] * a.s_os + i[p] * a.s_is + gr[p]] =
                __float2half_rn(scale_for_output(range, scale, a.inv_qmax, a.scale_mode));
            ((__half *)a.zero)[o[p] * a.s_os + i[p] * a.s_is + gr[p]] = __float2half_rn(mn);
        }
    }
}

template <int BITS, int P>
__global__ void __launch_bounds__(256) quant_rows_g32_f16_stream(QuantArgs a, uint32_t groups_per_row,
                                                                 int64_t total_groups)
{
    rows_g32_f16_stream_body<BITS, P>(a, groups_per_row, total_groups, (int64_t)blockIdx.x * (256 * P) + threadIdx.x);
}

// ---------------------------------------------------------------------------------------
// reference 3-bit format, fp16 rows: one thread per 11-code word (= one group of 11 values,
// 22 bytes at 2-byte alignment, fetched with three vector loads), P words per thread with the
// loads issued first.  WRAP: the append-V "placeholder" packing (11th code quantized to 0..7,
// low two bits kept).
// ---------------------------------------------------------------------------------------
struct __attribute__((packed, aligned(2))) Half11 {
    uint16_t v[11];
};

template <int P, bool WRAP>
__global__ void __launch_bounds__(256) quant_rows_ref3_f16(QuantArgs a, uint32_t words_per_row, int64_t total_words)
{
    const int64_t first = (int64_t)blockIdx.x * (256 * P) + threadIdx.x;
    Half11 raw[P];
    int64_t o[P], i[P];
    uint32_t wr[P];
    bool active[P];
#pragma unroll
    for (int p = 0; p < P; p++) {
        int64_t w = first + (int64_t)p * 256;
        active[p] = w < total_words;
        if (!active[p]) w = total_words - 1;
        const int64_t row = w / words_per_row;  // (64-bit: the word count may exceed 2^32)
        wr[p] = (uint32_t)(w - row * words_per_row);
        o[p] = row / a.inner;
        i[p] = row - o[p] * a.inner;
        const __half *x = (const __half *)a.x + o[p] * a.x_os + i[p] * a.x_is + (int64_t)wr[p] * 11;
        raw[p] = *reinterpret_cast<const Half11 *>(x);
    }
#pragma unroll
    for (int p = 0; p < P; p++) {
        float v[11];
        float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
#pragma unroll
        for (int t = 0; t < 11; t++) {
            v[t] = h16_to_f32(raw[p].v[t]);
            mn = fminf(mn, v[t]);
            mx = fmaxf(mx, v[t]);
        }
        const float range = mx - mn;
        const float scale = range / 7.0f;
        const float rcp = quantize_rcp(scale);
        uint32_t word = 0;
        uint32_t q11[11];
        quantize_codes<11>(v, mn, scale, rcp, [](int t) { return t < 10 || WRAP ? 7 : 3; }, q11);
#pragma unroll
        for (int t = 0; t < 10; t++) word |= q11[t] << (3 * t);
        word |= (q11[10] & 3u) << 30;
        if (active[p]) {
            a.code[o[p] * a.c_os + i[p] * a.c_is + wr[p]] = word;
            ((__half *)a.scale)[o[p] * a.s_os + i[p] * a.s_is + wr[p]] =
                __float2half_rn(scale_for_output(range, scale, a.inv_qmax, a.scale_mode));
            ((__half *)a.zero)[o[p] * a.s_os + i[p] * a.s_is + wr[p]] = __float2half_rn(mn);
        }
    }
}

// ---------------------------------------------------------------------------------------
// keys from the token-major tail: k [outer, n, D] -> code [outer, D, n/vpw], groups of G
// tokens per channel.  One thread per (group, channel) holds the group in registers.
// MODE: 1, 2, 4 = reference layout bits; 3 = reference 3-bit (G must be 11); 30 = dense 3-bit.
// ---------------------------------------------------------------------------------------
struct KeyTokArgs {
    const __half *k;
    uint32_t *code;
    __half *scale;
    __half *zero;
    int64_t n, D;
    int64_t k_os, k_ts;
    int64_t c_os, c_is;
    int64_t s_os, s_is;
    int scale_mode;
    float inv_qmax;
};

// words of one quantization group of a channel
template <int G, int MODE>
constexpr int key_group_words() { return MODE == 3 ? 1 : (G * (MODE == 30 ? 3 : MODE)) / 32; }

// G values of one channel -> packed words, scale, zero
template <int G, int MODE>
__device__ __forceinline__ void key_group_codes(const KeyTokArgs &a, const float (&v)[G],
                                                uint32_t (&w)[key_group_words<G, MODE>()], __half &scale_out,
                                                __half &zero_out)
{
    constexpr int BITS = MODE == 30 ? 3 : MODE;
    constexpr int qmax = (1 << BITS) - 1;
    constexpr int WORDS = key_group_words<G, MODE>();
    float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
#pragma unroll
    for (int t = 0; t < G; t++) {
        mn = fminf(mn, v[t]);
        mx = fmaxf(mx, v[t]);
    }
    const float range = mx - mn;
    const float scale = range / (float)qmax;
    const float rcp = quantize_rcp(scale);
#pragma unroll
    for (int t = 0; t < WORDS; t++) w[t] = 0;
    if constexpr (MODE == 3) {
        uint32_t q11[11];
        quantize_codes<11>(v, mn, scale, rcp, [](int t) { return t < 10 ? 7 : 3; }, q11);
#pragma unroll
        for (int t = 0; t < 11; t++) w[0] |= q11[t] << (t < 10 ? 3 * t : 30);
    } else {
#pragma unroll
        for (int t0 = 0; t0 < G; t0 += 8) {
            uint32_t q8[8];
            quantize_codes<8>(v + t0, mn, scale, rcp, [](int) { return qmax; }, q8);
#pragma unroll
            for (int t = t0; t < t0 + 8; t++) {
                const uint32_t q = q8[t - t0];
                const int bit = t * BITS;
                w[bit >> 5] |= q << (bit & 31);
                if ((bit & 31) + BITS > 32) w[(bit >> 5) + 1] |= q >> (32 - (bit & 31));
            }
        }
    }
    scale_out = __float2half_rn(scale_for_output(range, scale, a.inv_qmax, a.scale_mode));
    zero_out = __float2half_rn(mn);
}

// ... stored at group gi of channel d
template <int G, int MODE>
__device__ __forceinline__ void key_group_store(const KeyTokArgs &a, const float (&v)[G], int64_t gi, int64_t o,
                                                int64_t d)
{
    constexpr int WORDS = key_group_words<G, MODE>();
    uint32_t w[WORDS];
    __half sc, zr;
    key_group_codes<G, MODE>(a, v, w, sc, zr);
    uint32_t *cw = a.code + o * a.c_os + d * a.c_is + gi * WORDS;
#pragma unroll
    for (int t = 0; t < WORDS; t++) cw[t] = w[t];
    a.scale[o * a.s_os + d * a.s_is + gi] = sc;
    a.zero[o * a.s_os + d * a.s_is + gi] = zr;
}

template <int G, int MODE>
__device__ __forceinline__ void key_tokens_body(const KeyTokArgs &a, int64_t gi, int64_t o, int64_t d)
{
    const __half *src = a.k + o * a.k_os + gi * G * a.k_ts + d;
    float v[G];
#pragma unroll
    for (int t = 0; t < G; t++) v[t] = __half2float(src[t * a.k_ts]);
    key_group_store<G, MODE>(a, v, gi, o, d);
}

// The same for D = 128 with 16-byte-aligned token rows: 256 threads take a chunk of groups (four of 32
// tokens, or eleven of the reference 3-bit format's 11) of 64 channels of one outer slice.  The
// [tokens][64] tile is fetched with 128-bit loads (a thread: 8 channels of one token) into LDS; thread
// (channel t % 64, t / 64) reads its channel's column and packs groups t / 64, + 4, + 8 of the chunk; the
// words, scales and zeros are then handed over through LDS so that neighbouring lanes write neighbouring
// entries of a channel row: one contiguous piece of codes, one of scales and one of zeros per row (for
// the reference 3-bit format 44 + 22 + 22 bytes instead of 33 separate stores from different blocks).
// Units: (outer, chunk, channel half), channel half fastest.  Every thread of the block must call it
// (block barriers).
#ifndef KVMIX_KEY_SLAB_CHANNELS
#define KVMIX_KEY_SLAB_CHANNELS 64
#endif
constexpr int kKeySlabChannels = KVMIX_KEY_SLAB_CHANNELS;
constexpr int kKeySlabParts = 128 / kKeySlabChannels;       // channel parts of a head
constexpr int kKeySlabThreadGroups = 256 / kKeySlabChannels; // groups of a chunk packed at a time
template <int MODE>
constexpr int key_slab_groups() { return MODE == 3 ? 11 : 4; }   // 121 or 128 tokens: a 16 KB tile
static inline int64_t key_slab_units(int mode, int64_t outer, int64_t k_groups)
{
    const int gc = mode == 3 ? key_slab_groups<3>() : key_slab_groups<4>();
    return outer * ((k_groups + gc - 1) / gc) * kKeySlabParts;
}
// what the slab path asks of the operand: D = 128, token rows that 128-bit loads can fetch
static inline bool key_rows_tileable(const KeyTokArgs &a)
{
    return a.D == 128 && (uintptr_t)a.k % 16 == 0 && a.k_ts % 8 == 0 && a.k_os % 8 == 0;
}
constexpr int kKeySlabTile = 8192;  // fp16 elements of LDS a block needs (128 tokens x 64 channels)

template <int G, int MODE>
__device__ __forceinline__ void key_tokens_slab_body(const KeyTokArgs &a, int64_t k_groups, int64_t unit,
                                                     uint16_t *tile)
{
    constexpr int GC = key_slab_groups<MODE>(), CH = kKeySlabChannels, PPR = CH / 8;  // 16-byte pieces per tile row
    constexpr int WORDS = key_group_words<G, MODE>();
    constexpr int NGQ = kKeySlabThreadGroups, JMAX = (GC + NGQ - 1) / NGQ;  // groups per thread
    static_assert(GC * G * CH <= kKeySlabTile, "the tile of a chunk");
    const int tid = threadIdx.x;
    const uint32_t chunks = (uint32_t)((k_groups + GC - 1) / GC);
    const uint32_t u = (uint32_t)unit;  // (the host keeps the units below 2^31)
    const uint32_t half = u % (uint32_t)kKeySlabParts, rest = u / (uint32_t)kKeySlabParts, chunk = rest % chunks;
    const int64_t o = rest / chunks;
    const int g0 = (int)chunk * GC;
    const int ng = (int)(k_groups - g0 < GC ? k_groups - g0 : GC);
    const int pieces = ng * G * PPR;
    const __half *src = a.k + o * a.k_os + (int64_t)g0 * G * a.k_ts + half * CH;
    constexpr int ROUNDS = (GC * G * PPR + 255) / 256;
    uint4 raw[ROUNDS];
#pragma unroll
    for (int i = 0; i < ROUNDS; i++) {
        int pc = i * 256 + tid;
        pc = pc < pieces ? pc : pieces - 1;
        raw[i] = *reinterpret_cast<const uint4 *>(src + (int64_t)(pc / PPR) * a.k_ts + (pc % PPR) * 8);
    }
#pragma unroll
    for (int i = 0; i < ROUNDS; i++) {
        const int pc = i * 256 + tid;
        if (pc < pieces) *reinterpret_cast<uint4 *>(tile + (pc / PPR) * CH + (pc % PPR) * 8) = raw[i];
    }
    __syncthreads();
    const int dl = tid % CH, gq = tid / CH;
    uint32_t w[JMAX][WORDS];
    __half sc[JMAX], zr[JMAX];
#pragma unroll
    for (int j = 0; j < JMAX; j++) {
        const int g = gq + NGQ * j;
        if (g < ng) {
            float v[G];
#pragma unroll
            for (int r = 0; r < G; r++) v[r] = h16_to_f32(tile[(g * G + r) * CH + dl]);
            key_group_codes<G, MODE>(a, v, w[j], sc[j], zr[j]);
        }
    }
    __syncthreads();  // the tile is read: its memory now carries the results, [channel][group] at odd pitches
    const int nw = ng * WORDS, wp = nw | 1, sp = ng | 1;
    uint32_t *ow = reinterpret_cast<uint32_t *>(tile);
    __half *os = reinterpret_cast<__half *>(tile + 2 * CH * ((GC * WORDS) | 1)), *oz = os + CH * (GC | 1);
#pragma unroll
    for (int j = 0; j < JMAX; j++) {
        const int g = gq + NGQ * j;
        if (g < ng) {
#pragma unroll
            for (int t = 0; t < WORDS; t++) ow[dl * wp + g * WORDS + t] = w[j][t];
            os[dl * sp + g] = sc[j];
            oz[dl * sp + g] = zr[j];
        }
    }
    __syncthreads();
    const int64_t row0 = (int64_t)half * CH;
    for (int idx = tid; idx < CH * nw; idx += 256) {
        const int d = idx / nw, t = idx - d * nw;
        a.code[o * a.c_os + (row0 + d) * a.c_is + (int64_t)g0 * WORDS + t] = ow[d * wp + t];
    }
    for (int idx = tid; idx < CH * ng; idx += 256) {
        const int d = idx / ng, g = idx - d * ng;
        a.scale[o * a.s_os + (row0 + d) * a.s_is + g0 + g] = os[d * sp + g];
        a.zero[o * a.s_os + (row0 + d) * a.s_is + g0 + g] = oz[d * sp + g];
    }
}

template <int G, int MODE>
__global__ void __launch_bounds__(256) quant_key_tokens_slab(KeyTokArgs a, int64_t k_groups)
{
    __shared__ __attribute__((aligned(16))) uint16_t tile[kKeySlabTile];
    key_tokens_slab_body<G, MODE>(a, k_groups, blockIdx.x, tile);
}

template <int G, int MODE>
__global__ void __launch_bounds__(128) quant_key_tokens(KeyTokArgs a)
{
    const int64_t d = (int64_t)blockIdx.z * blockDim.x + threadIdx.x;
    if (d >= a.D) return;
    key_tokens_body<G, MODE>(a, blockIdx.x, blockIdx.y, d);
}

// ---------------------------------------------------------------------------------------
// both flushes of a decode step in one launch: blocks [0, k_blocks) run the key-token
// quantizer (one thread per (group, outer, channel)), the rest the group-32 value quantizer.
// The two parts touch disjoint tensors; a launch of this size is latency-bound, so one
// launch costs about what either part costs alone.
// ---------------------------------------------------------------------------------------
// One block of a layer's flush: blocks [0, k_blocks) run the key-token quantizer (slabs where the rows can be tiled,
// one thread per (group, channel) otherwise), the rest the value quantizer.  `bx`: the block's index within the layer.
struct FlushItem {
    KeyTokArgs ka;
    QuantArgs va;
    int64_t k_groups, k_threads, v_groups_per_row, v_total_groups;
    unsigned k_blocks, blocks;  // key blocks; key + value blocks
    int kmode, k_tiled;
    int v_stream;               // value half: one thread per group, two groups a thread (rows_g32_f16_stream_body)
};

#ifndef KVMIX_FLUSH_STREAM_P
#define KVMIX_FLUSH_STREAM_P 1
#endif
constexpr int kFlushStreamP = KVMIX_FLUSH_STREAM_P;  // groups a thread of the streaming value form takes (measured per launch
                                                     // of eight layers: two groups, 80 registers, six waves per SIMD 51 us; one group, 58, eight waves 47 us)
// One case of a switch over the formats, kept apart from its siblings: the value passes through an empty asm, so the
// compiler cannot merge the cases' common heads above the switch -- merged, the batched kernel needs 107 registers
// where its largest case alone needs 77 (four waves per SIMD instead of six).
#define KVMIX_CASE_V(var) asm volatile("" : "+v"(var))
#define KVMIX_CASE_S(var) asm volatile("" : "+s"(var))
template <bool STREAM>  // (the streaming value form needs more registers: only the batched kernel carries it)
__device__ __forceinline__ void flush_block(const FlushItem &f, unsigned bx, uint16_t *tile)
{
    if (bx < f.k_blocks && f.k_tiled) {
        switch (f.kmode) {
        case 1: KVMIX_CASE_S(bx); key_tokens_slab_body<32, 1>(f.ka, f.k_groups, bx, tile); break;
        case 2: KVMIX_CASE_S(bx); key_tokens_slab_body<32, 2>(f.ka, f.k_groups, bx, tile); break;
        case 3: KVMIX_CASE_S(bx); key_tokens_slab_body<11, 3>(f.ka, f.k_groups, bx, tile); break;
        case 4: KVMIX_CASE_S(bx); key_tokens_slab_body<32, 4>(f.ka, f.k_groups, bx, tile); break;
        default: KVMIX_CASE_S(bx); key_tokens_slab_body<32, 30>(f.ka, f.k_groups, bx, tile); break;
        }
    } else if (bx < f.k_blocks) {
        const int64_t id = (int64_t)bx * 256 + threadIdx.x;
        if (id >= f.k_threads) return;
        // (32-bit divisions: the host keeps the thread count below 2^31)
        const uint32_t id32 = (uint32_t)id, D32 = (uint32_t)f.ka.D, pair = id32 / D32;
        int64_t d = id32 - pair * D32;
        const int64_t o = pair / (uint32_t)f.k_groups, gi = pair - (uint32_t)o * (uint32_t)f.k_groups;
        switch (f.kmode) {
        case 1: KVMIX_CASE_V(d); key_tokens_body<32, 1>(f.ka, gi, o, d); break;
        case 2: KVMIX_CASE_V(d); key_tokens_body<32, 2>(f.ka, gi, o, d); break;
        case 3: KVMIX_CASE_V(d); key_tokens_body<11, 3>(f.ka, gi, o, d); break;
        case 4: KVMIX_CASE_V(d); key_tokens_body<32, 4>(f.ka, gi, o, d); break;
        default: KVMIX_CASE_V(d); key_tokens_body<32, 30>(f.ka, gi, o, d); break;
        }
    } else if (STREAM && f.v_stream) {
        int64_t first = (int64_t)(bx - f.k_blocks) * (256 * kFlushStreamP) + threadIdx.x;
        switch (f.va.bits) {
        case 1: KVMIX_CASE_V(first); rows_g32_f16_stream_body<1, kFlushStreamP>(f.va, (uint32_t)f.v_groups_per_row, f.v_total_groups, first); break;
        case 2: KVMIX_CASE_V(first); rows_g32_f16_stream_body<2, kFlushStreamP>(f.va, (uint32_t)f.v_groups_per_row, f.v_total_groups, first); break;
        case 3: KVMIX_CASE_V(first); rows_g32_f16_stream_body<3, kFlushStreamP>(f.va, (uint32_t)f.v_groups_per_row, f.v_total_groups, first); break;
        default: KVMIX_CASE_V(first); rows_g32_f16_stream_body<4, kFlushStreamP>(f.va, (uint32_t)f.v_groups_per_row, f.v_total_groups, first); break;
        }
    } else {
        int64_t tid = (int64_t)(bx - f.k_blocks) * (256 * kFlushValuePieces) + threadIdx.x;
        switch (f.va.bits) {
        case 1: KVMIX_CASE_V(tid); rows_g32_f16_body<1, kFlushValuePieces, kFlushIdx32>(f.va, f.v_groups_per_row, f.v_total_groups, tid); break;
        case 2: KVMIX_CASE_V(tid); rows_g32_f16_body<2, kFlushValuePieces, kFlushIdx32>(f.va, f.v_groups_per_row, f.v_total_groups, tid); break;
        case 3: KVMIX_CASE_V(tid); rows_g32_f16_body<3, kFlushValuePieces, kFlushIdx32>(f.va, f.v_groups_per_row, f.v_total_groups, tid); break;
        default: KVMIX_CASE_V(tid); rows_g32_f16_body<4, kFlushValuePieces, kFlushIdx32>(f.va, f.v_groups_per_row, f.v_total_groups, tid); break;
        }
    }
}
#undef KVMIX_CASE_V
#undef KVMIX_CASE_S

__global__ void __launch_bounds__(256) quant_kv_flush(FlushItem f)
{
    __shared__ __attribute__((aligned(16))) uint16_t tile[kKeySlabTile];
    flush_block<false>(f, blockIdx.x, tile);
}

// The flushes of up to kFlushBatch layers in one launch (kvmix_quant_pack_kv_flush_batch): first the key blocks of all
// layers -- the longer chains of dependent steps -- then the value blocks.  The items travel as kernel arguments.
constexpr int kFlushBatch = 8;
#ifndef KVMIX_FLUSH_BATCH_OCC
#define KVMIX_FLUSH_BATCH_OCC 8  // waves per SIMD the compiler plans for (58 registers with one group a thread in the streaming value form)
#endif
#ifndef KVMIX_FLUSH_STREAM_GROUPS
#define KVMIX_FLUSH_STREAM_GROUPS 16384
#endif
constexpr int64_t kFlushStreamGroups = KVMIX_FLUSH_STREAM_GROUPS;  // value groups of a pair from which on its half streams
struct FlushBatchArgs {
    FlushItem item[kFlushBatch];
    unsigned k_first[kFlushBatch + 1];  // first key block of item i among the launch's key blocks
    unsigned v_first[kFlushBatch + 1];  // first value block of item i among the launch's value blocks
    int count;
};

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(KVMIX_FLUSH_BATCH_OCC)))
quant_kv_flush_batch(FlushBatchArgs b)
{
    __shared__ __attribute__((aligned(16))) uint16_t tile[kKeySlabTile];
    const unsigned k_all = b.k_first[b.count];
    const bool key = blockIdx.x < k_all;
    const unsigned bx = key ? blockIdx.x : blockIdx.x - k_all;
    const unsigned *first = key ? b.k_first : b.v_first;
    int i = 0;
    while (i + 1 < b.count && bx >= first[i + 1]) i++;  // (uniform over the block; at most kFlushBatch - 1 steps)
    const FlushItem &f = b.item[i];
    flush_block<true>(f, key ? bx - first[i] : f.k_blocks + (bx - first[i]), tile);
}

static int64_t gcd64(int64_t a, int64_t b)
{
    while (b) {
        int64_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

// Validation shared by both entry points.  Returns the number of codes per word
// through *vpw (0 for the dense 3-bit stream, whose unit is 32 codes in 3 words).
static int check_format(int group, int bits, int fmt, int64_t steps, int *vpw)
{
    if (fmt != KVMIX_FMT_REF && fmt != KVMIX_FMT_DENSE3 && fmt != KVMIX_FMT_REF3_WRAP) return KVMIX_ERR_FORMAT;
    if (bits != 1 && bits != 2 && bits != 3 && bits != 4) return KVMIX_ERR_BITS;
    if (fmt != KVMIX_FMT_REF && bits != 3) return KVMIX_ERR_FORMAT;
    if (bits == 3 && fmt != KVMIX_FMT_DENSE3) {
        if (group != 11) return KVMIX_ERR_GROUP3;
        if (steps % 11 != 0) return KVMIX_ERR_STEPS_GROUP;
        *vpw = 11;
        return KVMIX_OK;
    }
    if (group <= 0 || steps % group != 0) return KVMIX_ERR_STEPS_GROUP;
    if (fmt == KVMIX_FMT_DENSE3) {
        if (group % 32 != 0) return KVMIX_ERR_UNSUPPORTED;
        *vpw = 0;
        return KVMIX_OK;
    }
    if (steps % (32 / bits) != 0) return KVMIX_ERR_STEPS_WORD;
    *vpw = 32 / bits;
    return KVMIX_OK;
}

// Validation and argument set-up shared by the separate and the fused entry points.
// *empty is set when there is nothing to do; *fast when the group-32 fp16 kernel applies.
static int setup_last_dim(const void *x, int x_dtype, int64_t outer, int64_t inner, int64_t steps,
                          int64_t x_outer_stride, int64_t x_inner_stride, int group, int bits, int fmt,
                          int scale_mode, uint32_t *code, int64_t code_outer_stride,
                          int64_t code_inner_stride, void *scale, void *zero, int64_t sz_outer_stride,
                          int64_t sz_inner_stride, QuantArgs &a, int &vpw, bool &empty, bool &fast)
{
    vpw = 0;
    empty = false;
    fast = false;
    if (x_dtype != KVMIX_F16 && x_dtype != KVMIX_F32) return KVMIX_ERR_DTYPE;
    if (outer < 0 || inner < 0 || steps < 0) return KVMIX_ERR_SHAPE;
    int rc = check_format(group, bits, fmt, steps, &vpw);
    if (rc != KVMIX_OK) return rc;
    if (scale_mode != KVMIX_SCALE_RECIPROCAL && scale_mode != KVMIX_SCALE_DIVIDE) return KVMIX_ERR_FORMAT;
    if (outer == 0 || inner == 0 || steps == 0) {
        empty = true;
        return KVMIX_OK;
    }
    if (!x || !code || !scale || !zero) return KVMIX_ERR_NULL;
    const int64_t words = vpw ? steps / vpw : steps * 3 / 32;
    const int64_t groups = steps / group;
    if (x_inner_stride < steps || code_inner_stride < words || sz_inner_stride < groups) return KVMIX_ERR_SHAPE;
    if (inner > 1 && (x_outer_stride < x_inner_stride || code_outer_stride < code_inner_stride ||
                      sz_outer_stride < sz_inner_stride))
        return KVMIX_ERR_SHAPE;

    a.x = x;
    a.code = code;
    a.scale = scale;
    a.zero = zero;
    a.outer = outer;
    a.inner = inner;
    a.steps = steps;
    a.x_os = x_outer_stride;
    a.x_is = x_inner_stride;
    a.c_os = code_outer_stride;
    a.c_is = code_inner_stride;
    a.s_os = sz_outer_stride;
    a.s_is = sz_inner_stride;
    a.group = group;
    a.bits = bits;
    a.fmt = fmt;
    a.scale_mode = scale_mode;
    a.inv_qmax = 1.0f / (float)((1 << bits) - 1);
    const bool ref3 = bits == 3 && fmt != KVMIX_FMT_DENSE3;
    const bool aligned16 = ((uintptr_t)x % 16 == 0) && (x_outer_stride % 8 == 0) && (x_inner_stride % 8 == 0);
    fast = x_dtype == KVMIX_F16 && group == 32 && !ref3 && aligned16;
    return KVMIX_OK;
}

static int launch_last_dim(const QuantArgs &a, int x_dtype, int vpw, bool fast, hipStream_t st)
{
    const int64_t groups = a.steps / a.group;
    if (fast) {
        const int64_t total_groups = a.outer * a.inner * groups;
        if (total_groups >= (int64_t)256 * 2 * 4096 && groups < (1ll << 31)) {
            const unsigned nb = (unsigned)((total_groups + 511) / 512);
            switch (a.bits) {
            case 1: hipLaunchKernelGGL((quant_rows_g32_f16_stream<1, 2>), dim3(nb), dim3(256), 0, st, a, (uint32_t)groups, total_groups); break;
            case 2: hipLaunchKernelGGL((quant_rows_g32_f16_stream<2, 2>), dim3(nb), dim3(256), 0, st, a, (uint32_t)groups, total_groups); break;
            case 3: hipLaunchKernelGGL((quant_rows_g32_f16_stream<3, 2>), dim3(nb), dim3(256), 0, st, a, (uint32_t)groups, total_groups); break;
            default: hipLaunchKernelGGL((quant_rows_g32_f16_stream<4, 2>), dim3(nb), dim3(256), 0, st, a, (uint32_t)groups, total_groups); break;
            }
            return launch_status();
        }
        const int64_t threads = total_groups * 4;
        // large inputs stream with several pieces per thread; small ones keep one (more waves)
        const bool many = threads >= (int64_t)256 * kRowsPieces * 2048;
        const bool idx32 = total_groups < (1ll << 30);
        const int64_t per_block = 256 * (many ? kRowsPieces : 1);
        const unsigned blocks = (unsigned)((threads + per_block - 1) / per_block);
#define KVMIX_ROWS_LAUNCH(B_)                                                                                         \
    do {                                                                                                              \
        if (many && idx32)                                                                                            \
            hipLaunchKernelGGL((quant_rows_g32_f16<B_, kRowsPieces, true>), dim3(blocks), dim3(256), 0, st, a, groups, \
                               total_groups);                                                                         \
        else if (many)                                                                                                \
            hipLaunchKernelGGL((quant_rows_g32_f16<B_, kRowsPieces, false>), dim3(blocks), dim3(256), 0, st, a,       \
                               groups, total_groups);                                                                 \
        else if (idx32)                                                                                               \
            hipLaunchKernelGGL((quant_rows_g32_f16<B_, 1, true>), dim3(blocks), dim3(256), 0, st, a, groups,          \
                               total_groups);                                                                         \
        else                                                                                                          \
            hipLaunchKernelGGL((quant_rows_g32_f16<B_, 1, false>), dim3(blocks), dim3(256), 0, st, a, groups,         \
                               total_groups);                                                                         \
    } while (0)
        switch (a.bits) {
        case 1: KVMIX_ROWS_LAUNCH(1); break;
        case 2: KVMIX_ROWS_LAUNCH(2); break;
        case 3: KVMIX_ROWS_LAUNCH(3); break;
        default: KVMIX_ROWS_LAUNCH(4); break;
        }
#undef KVMIX_ROWS_LAUNCH
        return launch_status();
    }
    if (x_dtype == KVMIX_F16 && a.bits == 3 && a.fmt != KVMIX_FMT_DENSE3 && a.group == 11) {
        const int64_t wpr = a.steps / 11, total = a.outer * a.inner * wpr;
        if (wpr < (1ll << 31)) {
            const unsigned blocks = (unsigned)((total + 256 * 2 - 1) / (256 * 2));
            if (a.fmt == KVMIX_FMT_REF3_WRAP)
                hipLaunchKernelGGL((quant_rows_ref3_f16<2, true>), dim3(blocks), dim3(256), 0, st, a, (uint32_t)wpr, total);
            else
                hipLaunchKernelGGL((quant_rows_ref3_f16<2, false>), dim3(blocks), dim3(256), 0, st, a, (uint32_t)wpr, total);
            return launch_status();
        }
    }
    // generic path: a thread owns lcm(group, codes per word) values, i.e. whole groups and whole words
    const int64_t word_span = vpw ? vpw : 32;
    const int64_t unit = (int64_t)a.group / gcd64(a.group, word_span) * word_span;
    if (a.steps % unit != 0 || unit > (1 << 20)) return KVMIX_ERR_UNSUPPORTED;
    const int64_t units_per_row = a.steps / unit;
    const int64_t total_units = a.outer * a.inner * units_per_row;
    const unsigned blocks = (unsigned)((total_units + 255) / 256);
    if (x_dtype == KVMIX_F16)
        hipLaunchKernelGGL(quant_rows_generic<__half>, dim3(blocks), dim3(256), 0, st, a, (int)unit,
                           units_per_row, total_units);
    else
        hipLaunchKernelGGL(quant_rows_generic<float>, dim3(blocks), dim3(256), 0, st, a, (int)unit,
                           units_per_row, total_units);
    return launch_status();
}

// *mode: 1, 2, 4 (reference layout), 3 (reference 3-bit), 30 (dense 3-bit)
static int setup_key_tokens(const void *k, int64_t outer, int64_t n, int64_t D, int64_t k_outer_stride,
                            int64_t k_token_stride, int group, int bits, int fmt, int scale_mode,
                            uint32_t *code, int64_t code_outer_stride, int64_t code_inner_stride,
                            void *scale, void *zero, int64_t sz_outer_stride, int64_t sz_inner_stride,
                            KeyTokArgs &a, int &mode, int64_t &groups, bool &empty)
{
    int vpw = 0;
    empty = false;
    if (outer < 0 || n < 0 || D < 0) return KVMIX_ERR_SHAPE;
    if (fmt == KVMIX_FMT_REF3_WRAP) return KVMIX_ERR_FORMAT;
    int rc = check_format(group, bits, fmt, n, &vpw);
    if (rc != KVMIX_OK) return rc;
    const bool ref3 = bits == 3 && fmt == KVMIX_FMT_REF;
    if (scale_mode != KVMIX_SCALE_RECIPROCAL && scale_mode != KVMIX_SCALE_DIVIDE) return KVMIX_ERR_FORMAT;
    if (outer == 0 || n == 0 || D == 0) {
        // (before the group check: an empty key half of kvmix_quant_pack_kv_flush may name any group)
        empty = true;
        return KVMIX_OK;
    }
    if (!ref3 && group != 32) return KVMIX_ERR_UNSUPPORTED;
    if (!k || !code || !scale || !zero) return KVMIX_ERR_NULL;
    const int64_t words = vpw ? n / vpw : n * 3 / 32;
    groups = n / group;
    if (k_token_stride < D || code_inner_stride < words || sz_inner_stride < groups) return KVMIX_ERR_SHAPE;
    if (groups > 0x7fffffff) return KVMIX_ERR_SHAPE;
    a.k = (const __half *)k;
    a.code = code;
    a.scale = (__half *)scale;
    a.zero = (__half *)zero;
    a.n = n;
    a.D = D;
    a.k_os = k_outer_stride;
    a.k_ts = k_token_stride;
    a.c_os = code_outer_stride;
    a.c_is = code_inner_stride;
    a.s_os = sz_outer_stride;
    a.s_is = sz_inner_stride;
    a.scale_mode = scale_mode;
    a.inv_qmax = 1.0f / (float)((1 << bits) - 1);
    mode = ref3 ? 3 : (bits == 3 ? 30 : bits);
    return KVMIX_OK;
}

static int launch_key_tokens(const KeyTokArgs &a, int mode, int64_t groups, int64_t outer, hipStream_t st)
{
    if (key_rows_tileable(a)) {
        const int64_t units = key_slab_units(mode, outer, groups);
        if (units > 0x7fffffff) return KVMIX_ERR_SHAPE;
        const dim3 grid((unsigned)units);
        switch (mode) {
        case 3: hipLaunchKernelGGL((quant_key_tokens_slab<11, 3>), grid, dim3(256), 0, st, a, groups); break;
        case 30: hipLaunchKernelGGL((quant_key_tokens_slab<32, 30>), grid, dim3(256), 0, st, a, groups); break;
        case 4: hipLaunchKernelGGL((quant_key_tokens_slab<32, 4>), grid, dim3(256), 0, st, a, groups); break;
        case 2: hipLaunchKernelGGL((quant_key_tokens_slab<32, 2>), grid, dim3(256), 0, st, a, groups); break;
        default: hipLaunchKernelGGL((quant_key_tokens_slab<32, 1>), grid, dim3(256), 0, st, a, groups); break;
        }
        return launch_status();
    }
    const int block = a.D >= 128 ? 128 : 64;
    if ((a.D + block - 1) / block > 65535) return KVMIX_ERR_SHAPE;
    // (grid.y holds at most 65535 blocks: more (batch, head) slices than that go out in several launches)
    for (int64_t o0 = 0; o0 < outer; o0 += 65535) {
        KeyTokArgs p = a;
        p.k += o0 * a.k_os;
        p.code += o0 * a.c_os;
        p.scale += o0 * a.s_os;
        p.zero += o0 * a.s_os;
        const int64_t no = outer - o0 < 65535 ? outer - o0 : 65535;
        const dim3 grid((unsigned)groups, (unsigned)no, (unsigned)((a.D + block - 1) / block));
        switch (mode) {
        case 3: hipLaunchKernelGGL((quant_key_tokens<11, 3>), grid, dim3(block), 0, st, p); break;
        case 30: hipLaunchKernelGGL((quant_key_tokens<32, 30>), grid, dim3(block), 0, st, p); break;
        case 4: hipLaunchKernelGGL((quant_key_tokens<32, 4>), grid, dim3(block), 0, st, p); break;
        case 2: hipLaunchKernelGGL((quant_key_tokens<32, 2>), grid, dim3(block), 0, st, p); break;
        default: hipLaunchKernelGGL((quant_key_tokens<32, 1>), grid, dim3(block), 0, st, p); break;
        }
    }
    return launch_status();
}

}  // namespace kvmix

using namespace kvmix;

extern "C" int kvmix_quant_pack_last_dim(const void *x, int x_dtype, int64_t outer, int64_t inner,
                                         int64_t steps, int64_t x_outer_stride, int64_t x_inner_stride,
                                         int group, int bits, int fmt, int scale_mode, uint32_t *code,
                                         int64_t code_outer_stride, int64_t code_inner_stride,
                                         void *scale, void *zero, int64_t sz_outer_stride,
                                         int64_t sz_inner_stride, kvmix_stream_t stream)
{
    QuantArgs a;
    int vpw;
    bool empty, fast;
    const int rc = setup_last_dim(x, x_dtype, outer, inner, steps, x_outer_stride, x_inner_stride, group, bits, fmt,
                                  scale_mode, code, code_outer_stride, code_inner_stride, scale, zero,
                                  sz_outer_stride, sz_inner_stride, a, vpw, empty, fast);
    if (rc != KVMIX_OK || empty) return rc;
    return launch_last_dim(a, x_dtype, vpw, fast, (hipStream_t)stream);
}

extern "C" int kvmix_quant_pack_key_tokens(const void *k, int64_t outer, int64_t n, int64_t D,
                                           int64_t k_outer_stride, int64_t k_token_stride, int group,
                                           int bits, int fmt, int scale_mode, uint32_t *code,
                                           int64_t code_outer_stride, int64_t code_inner_stride,
                                           void *scale, void *zero, int64_t sz_outer_stride,
                                           int64_t sz_inner_stride, kvmix_stream_t stream)
{
    KeyTokArgs a;
    int mode = 0;
    int64_t groups = 0;
    bool empty;
    const int rc = setup_key_tokens(k, outer, n, D, k_outer_stride, k_token_stride, group, bits, fmt, scale_mode, code,
                                    code_outer_stride, code_inner_stride, scale, zero, sz_outer_stride,
                                    sz_inner_stride, a, mode, groups, empty);
    if (rc != KVMIX_OK || empty) return rc;
    return launch_key_tokens(a, mode, groups, outer, (hipStream_t)stream);
}

// Both halves of a layer's flush checked and laid out.  KVMIX_OK with `fused` false: one half is empty or the value
// half needs the generic quantizer -- the halves then go out as launches of their own.
struct FlushSetup {
    FlushItem item;
    bool kempty, vempty, vfast, fused;
    int vpw;
};
static int setup_flush(const kvmix_key_flush_t *kf, const kvmix_value_flush_t *vf, FlushSetup &fs, bool batched = false)
{
    if (!kf || !vf) return KVMIX_ERR_NULL;
    FlushItem &f = fs.item;
    int rc = setup_key_tokens(kf->k, kf->outer, kf->n, kf->D, kf->k_outer_stride, kf->k_token_stride, kf->group,
                              kf->bits, kf->fmt, kf->scale_mode, kf->code, kf->code_outer_stride,
                              kf->code_inner_stride, kf->scale, kf->zero, kf->sz_outer_stride, kf->sz_inner_stride,
                              f.ka, f.kmode, f.k_groups, fs.kempty);
    if (rc != KVMIX_OK) return rc;
    rc = setup_last_dim(vf->x, KVMIX_F16, vf->outer, vf->inner, vf->steps, vf->x_outer_stride, vf->x_inner_stride,
                        vf->group, vf->bits, vf->fmt, vf->scale_mode, vf->code, vf->code_outer_stride,
                        vf->code_inner_stride, vf->scale, vf->zero, vf->sz_outer_stride, vf->sz_inner_stride, f.va, fs.vpw,
                        fs.vempty, fs.vfast);
    if (rc != KVMIX_OK) return rc;  // (nothing was launched: both halves are checked first)
    fs.fused = !(fs.kempty || fs.vempty || !fs.vfast);
    if (!fs.fused) return KVMIX_OK;
    // key slab path: D = 128, token rows 16-byte aligned
    f.k_tiled = key_rows_tileable(f.ka);
    f.k_threads = f.k_groups * kf->outer * kf->D;
    const int64_t k_blocks = f.k_tiled ? key_slab_units(f.kmode, kf->outer, f.k_groups) : (f.k_threads + 255) / 256;
    f.v_groups_per_row = f.va.steps / 32;
    f.v_total_groups = f.va.outer * f.va.inner * f.v_groups_per_row;
    // A flush alone is a latency-bound launch and wants many small threads (four to a group); in a batch of layers
    // the value half is a streaming kernel and takes the prompt quantizer's form, a thread per group (measured, the
    // 32 flushes of a step in four launches: 222.8 -> 206.7 us).
    f.v_stream = batched && f.v_total_groups >= kFlushStreamGroups && f.v_groups_per_row < (1ll << 31) ? 1 : 0;
    const int64_t v_blocks = f.v_stream ? (f.v_total_groups + 256 * kFlushStreamP - 1) / (256 * kFlushStreamP)
                                        : (f.v_total_groups * 4 + 256 * kFlushValuePieces - 1) / (256 * kFlushValuePieces);
    if (k_blocks + v_blocks > 0x7fffffff || f.k_threads > 0x7fffffff) return KVMIX_ERR_SHAPE;
    f.k_blocks = (unsigned)k_blocks;
    f.blocks = (unsigned)(k_blocks + v_blocks);
    return KVMIX_OK;
}

// the halves of a flush that cannot share a launch
static int launch_flush_halves(const kvmix_key_flush_t *kf, const FlushSetup &fs, hipStream_t st)
{
    if (!fs.kempty) {
        const int rc = launch_key_tokens(fs.item.ka, fs.item.kmode, fs.item.k_groups, kf->outer, st);
        if (rc != KVMIX_OK) return rc;
    }
    return fs.vempty ? KVMIX_OK : launch_last_dim(fs.item.va, KVMIX_F16, fs.vpw, fs.vfast, st);
}

extern "C" int kvmix_quant_pack_kv_flush(const kvmix_key_flush_t *kf, const kvmix_value_flush_t *vf,
                                         kvmix_stream_t stream)
{
    FlushSetup fs;
    const int rc = setup_flush(kf, vf, fs);
    if (rc != KVMIX_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    if (!fs.fused) return launch_flush_halves(kf, fs, st);
    hipLaunchKernelGGL(quant_kv_flush, dim3(fs.item.blocks), dim3(256), 0, st, fs.item);
    return launch_status();
}

extern "C" int kvmix_quant_pack_kv_flush_batch(const kvmix_key_flush_t *const *kf, const kvmix_value_flush_t *const *vf,
                                               int count, kvmix_stream_t stream)
{
    if (count < 0) return KVMIX_ERR_SHAPE;
    if (count == 0) return KVMIX_OK;
    if (!kf || !vf) return KVMIX_ERR_NULL;
    // every layer is checked before anything is launched
    std::vector<FlushSetup> fs((size_t)count);
    for (int i = 0; i < count; i++) {
        const int rc = setup_flush(kf[i], vf[i], fs[(size_t)i], true);
        if (rc != KVMIX_OK) return rc;
    }
    hipStream_t st = (hipStream_t)stream;
    FlushBatchArgs b;
    b.count = 0;
    uint64_t k_blocks = 0, v_blocks = 0;
    auto flush_launch = [&]() {
        if (b.count == 0) return KVMIX_OK;
        b.k_first[b.count] = (unsigned)k_blocks;
        b.v_first[b.count] = (unsigned)v_blocks;
        hipLaunchKernelGGL(quant_kv_flush_batch, dim3((unsigned)(k_blocks + v_blocks)), dim3(256), 0, st, b);
        b.count = 0;
        k_blocks = v_blocks = 0;
        return launch_status();
    };
    for (int i = 0; i < count; i++) {
        const FlushSetup &s = fs[(size_t)i];
        if (!s.fused) {
            const int rc = launch_flush_halves(kf[i], s, st);
            if (rc != KVMIX_OK) return rc;
            continue;
        }
        if (b.count == kFlushBatch || k_blocks + v_blocks + s.item.blocks > 0x7fffffffull) {
            const int rc = flush_launch();
            if (rc != KVMIX_OK) return rc;
        }
        b.item[b.count] = s.item;
        b.k_first[b.count] = (unsigned)k_blocks;
        b.v_first[b.count] = (unsigned)v_blocks;
        k_blocks += s.item.k_blocks;
        v_blocks += s.item.blocks - s.item.k_blocks;
        b.count++;
    }
    return flush_launch();
}
