// Fused dequantize + GEMV over the packed KV cache (gfx950).
//
//   out[s, m, n] = fp16( sum_k x[s, m, k] * ( scale[s', k, n/g] * code[s', k, n] + zero[s', k, n/g] ) )
//
// the operator of quant_cuda/csrc/dequantization_gemv_cuda.cu:7-248 in the reference,
// computed on the cache's stored layout ([.., K, N/vpw] words, [.., K, N/g] scale/zero) --
// the reference transposes codes, scales and zeros into new buffers on every call
// (dequantization_gemv_cuda.cu:154-171); here nothing is copied.
//
// The sum is split as  sum_k (x_k * scale_k) * code_kn  +  sum_k x_k * zero_k : the second
// term is one fma per (k, group) instead of one per element, and the first needs no
// int->float conversion (see mix2 below).  All accumulation is fp32.
//
// Kernels (each documented where it is defined)
//   gemv_rows_mfma  p.V (K = tokens large, N = 128), 1/2/4-bit and dense 3-bit: matrix cores.
//   gemv_cols_mfma2 q.K^T (K = head_dim small, N = tokens large), 1/2/4-bit, one query head per kv
//                   head: matrix cores, two 8-code elements per lane; small launches let several
//                   waves share a tile and slice K.
//   gemv_cols_mfma  q.K^T, 1/2/4-bit: matrix cores, one element per lane; GQA (four query heads per
//                   pass) and 1-bit.
//   gemv_cols3      q.K^T, the reference's 3-bit format: register streaming, vector ALU.
//   gemv_cols       q.K^T, 1/2/4-bit at large batch with long rows, dense 3-bit: vector ALU,
//                   (scale, zero) staged in LDS.
//   gemv_rows       p.V for N = 64 / 256 or strided code rows: vector ALU.
//   gemv_generic    any shape/group, and rows shorter than one tile of the kernels above: one thread
//                   per packed word, the block's spare threads slice K.
//   reduce_splits   sums the split-K partials of the p.V kernels and stores fp16.
// Which kernel a call gets is decided in launch_cols / launch_rows / kvmix_quantized_gemv at the
// end of the file; the thresholds there are measured ones.
//
// Common rules of the streaming kernels (measured on MI355X): scale/zero never by 2-byte loads
// per lane (they cost a third of the run time) but by 128-bit loads of whichever lane the
// address falls to, handed on through a wave-private LDS tile (no block barrier in the stream);
// every load unconditional, in one fixed order from the first iteration on, and pinned with
// scheduling barriers -- otherwise the compiler sinks the prefetch loads to the end of the loop
// body and every iteration starts by draining the load queue.

#include "fused_slab.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <mutex>

// Switches kept for measurement: with the hint compiled out the HBM counters show the bytes a kernel reads without it.
#ifndef KVMIX_STREAM_NT
#define KVMIX_STREAM_NT 1  // non-temporal loads for the packed operands
#endif
#ifndef KVMIX_ROWS_RAW_PERM
#define KVMIX_ROWS_RAW_PERM 1
#endif
#ifndef KVMIX_COLS_NT_CODES
#define KVMIX_COLS_NT_CODES 1  // q.K^T kernels: codes non-temporal (the matrix-core kernels: 2 and 4 bits only -- a wave's 1-bit row piece is 64 or 128 bytes and shares its cache lines with the neighbours')
#endif
#ifndef KVMIX_SLAB3_NT_CODES
#define KVMIX_SLAB3_NT_CODES KVMIX_COLS_NT_CODES  // attention step, reference 3-bit keys: codes / scales and zeros non-temporal
#endif
#ifndef KVMIX_SLAB3_NT_SZ
#define KVMIX_SLAB3_NT_SZ 1
#endif
#ifndef KVMIX_SLAB_BARRIER
#define KVMIX_SLAB_BARRIER 1   // attention step, 1/2/4-bit keys: one s_barrier per 16-row chunk of the key phase
#endif
#ifndef KVMIX_SLAB3_BARRIER
#define KVMIX_SLAB3_BARRIER 1  // ... one s_barrier per step of the key phase
#endif
#ifndef KVMIX_COLS3_NT_SZ
#define KVMIX_COLS3_NT_SZ 1  // q.K^T, reference 3-bit words, one head per pass: scales and zeros (as large as the codes) non-temporal
#endif

namespace kvmix {

constexpr int kMaxDevices = 64;  // per-device set-up state is kept for device ordinals below this

// Measured constants of the dispatch (MI355X: 256 CUs x 4 SIMDs).  tests/test_gemv_plan_cpu.py pins the kernel
// each benchmark shape ends up with.
constexpr int kTargetWaves = 4096;          // 16 waves on each of 256 CUs
#ifndef KVMIX_COLS3_HEADS_U
#define KVMIX_COLS3_HEADS_U 4
#endif
#ifndef KVMIX_COLS3_HEADS_OCC
#define KVMIX_COLS3_HEADS_OCC 2
#endif
constexpr int kCols3HeadsU = KVMIX_COLS3_HEADS_U;   // gemv_cols3, four heads per pass: rows in flight per lane
constexpr int kCols3U = 8;                  // gemv_cols3, one head per pass: rows in flight per lane
constexpr int kCols3HeadsOcc = KVMIX_COLS3_HEADS_OCC;   // waves per SIMD the compiler may plan for: gemv_cols3, four heads
#ifndef KVMIX_MFMA_HEADS_OCC
#define KVMIX_MFMA_HEADS_OCC 2
#endif
constexpr int kMfmaHeadsOcc = KVMIX_MFMA_HEADS_OCC;   // ... gemv_rows_mfma / gemv_cols_mfma, four heads
constexpr int kMfma2Occ = 2;                // ... gemv_cols_mfma2 (at least; it comes out at three)
constexpr int kHeadsWaveDiv = 2;            // p.V, four heads per pass: half as many waves wanted
constexpr int kMfma2MaxWaves = kTargetWaves;    // two-element matrix-core q.K^T kernel up to this many tiles
constexpr int kMfma1MaxWaves = kTargetWaves;    // one-element matrix-core q.K^T kernel (one head) below this many tiles
constexpr int kMfma2ResidentWaves = 3072;   // gemv_cols_mfma2: 3 waves on each of 1024 SIMDs
constexpr int64_t kMfma2WideMinCodes = 6144;    // gemv_cols_mfma2: rows from this many codes on may take the wide tiles
constexpr int64_t kMfma2WideMaxWaves = 2048;    // ... in launches of up to this many of them (one round, two waves per SIMD)
constexpr int kMfma2KsplitWaves = 1536;     // gemv_cols_mfma2: waves share a tile (slicing K) while that keeps the launch below this many waves
#ifndef KVMIX_ROWS_CHUNKS_PER_WAVE
#define KVMIX_ROWS_CHUNKS_PER_WAVE 8
#endif
constexpr int kRowsChunksPerWave = KVMIX_ROWS_CHUNKS_PER_WAVE;  // p.V: chunks a wave should get before more waves per row are used
constexpr int kRowsSingleBlockChunks = 2;   // p.V: keep one block per output row up to this many chunks per wave
constexpr int kCols3WideWaves = 4096;       // gemv_cols3: widest tiles (one wave each) from this many of them on
constexpr int kCols3MinWaves = 2048;        // gemv_cols3: 128-word one-wave tiles from this many of them on

struct GemvArgs {
    const __half *x;
    const uint32_t *code;
    const __half *scale;
    const __half *zero;
    __half *out;
    float *partial;
    int64_t x_bs, x_rs;
    int64_t c_bs, c_rs;
    int64_t s_bs, s_rs;
    int64_t o_bs, o_rs;
    int64_t K, N;
    int64_t M;
    int64_t rows_per_split;
    int heads_per_kv;
    int group;
    int splits;
    int ksplit;  // gemv_cols_mfma2: waves that share a tile and slice K
};

// Buffer addressing for the streaming loops: address = descriptor base (scalar registers) + a per-lane
// byte offset that never changes (one vector register) + a byte offset that is the same for the whole
// wave (a scalar register: the row).  A flat global load needs the full 64-bit address in two vector
// registers per load, formed by vector-ALU adds; here the row arithmetic runs on the scalar unit and costs
// the vector ALU nothing.  Offsets are 32-bit: the host only sends problems whose (batch, kv-head)
// slice stays below 2^32 bytes to the kernels that use this.
// `bytes` is the extent of the slice (from its first byte to the end of its last row): the descriptor's
// num_records.  The hardware compares every dword's byte offset with it and returns zero for a dword at or past
// it, so a wave that were handed a tile outside its operand would compute with zeros instead of touching memory
// that is not the caller's -- the kernels' own index arithmetic never goes there, this is the second fence.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t stream_rsrc(const void *base, uint32_t bytes)
{
    // raw buffer, no stride, 32-bit data format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
// extent in bytes of one (batch, kv-head) slice of `rows` rows at a pitch of `row_stride` elements of `elem_bytes`
// bytes, the last row holding `row_elems` of them
__device__ __forceinline__ uint32_t slice_bytes(int64_t rows, int64_t row_stride, int64_t row_elems, int elem_bytes)
{
    return rows > 0 ? (uint32_t)(((rows - 1) * row_stride + row_elems) * elem_bytes) : 0u;
}
template <typename T, bool NT>
__device__ __forceinline__ T ld_buffer(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_bytes, uint32_t wave_bytes)
{
    constexpr int AUX = (NT && KVMIX_STREAM_NT) ? 2 : 0;  // bit 1 of the cache policy = non-temporal
    T out;
    if constexpr (sizeof(T) == 16) {
        const auto v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes, wave_bytes, AUX);
        __builtin_memcpy(&out, &v, 16);
    } else if constexpr (sizeof(T) == 8) {
        const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, lane_bytes, wave_bytes, AUX);
        __builtin_memcpy(&out, &v, 8);
    } else if constexpr (sizeof(T) == 4) {
        const auto v = __builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_bytes, wave_bytes, AUX);
        __builtin_memcpy(&out, &v, 4);
    } else {
        static_assert(sizeof(T) == 2, "unsupported size for a buffer load");
        const auto v = __builtin_amdgcn_raw_buffer_load_b16(rsrc, lane_bytes, wave_bytes, AUX);
        __builtin_memcpy(&out, &v, 2);
    }
    return out;
}

// MODE: 1, 2, 4 = reference layout with that many bits (group 32 in the fast kernels),
//       3 = the reference's 3-bit layout (11 codes per word, group 11),
//       30 = dense 3-bit stream (32 codes in 3 words, group 32).
template <int MODE>
struct Fmt {
    static constexpr int BITS = MODE == 30 ? 3 : MODE;
    static constexpr int VALS = MODE == 3 ? 11 : 32;                       // codes per group unit
    static constexpr int WORDS = MODE == 3 ? 1 : (MODE == 30 ? 3 : MODE);  // words per group unit
    // accumulate_unit leaves the 3-bit formats' sums scaled by 2^-59 (see there)
    static constexpr float OUT_SCALE = (MODE == 3 || MODE == 30) ? 576460752303423488.0f : 1.0f;
};

// Vectors with relaxed alignment: the compiler still emits one wide global load, and gfx9
// global memory accepts any byte alignment (a misaligned access only costs extra cycles).
template <int W>
struct __attribute__((packed, aligned(4))) Words {
    uint32_t v[W];
};
struct __attribute__((packed, aligned(2))) Half8 {
    uint16_t v[8];
};

// Packed codes are read exactly once per launch: they are loaded non-temporally (the `nt` bit of
// global_load), which keeps the stream from displacing itself and its neighbours in the caches on
// the way.  Measured on MI355X with a kernel that only reads: 6.0-6.2 TB/s with plain loads against
// 6.7-6.9 TB/s with non-temporal ones for contiguous slabs (the p.V pattern), 6.1 against 6.4-6.6 TB/s
// for row pieces (the q.K^T pattern).  The scales and zeros of the q.K^T kernels stay on plain loads:
// their 64-byte row pieces share cache lines with the neighbouring wave's, which the L2 has to keep.
// T: a trivially copyable type of 1, 2, 4, 8, 12 or 16 bytes whose alignment (2 or at least 4) is all
// that is assumed of the address.
typedef uint32_t nt_u4a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t nt_u2a4 __attribute__((ext_vector_type(2), aligned(4)));
typedef uint32_t nt_u1a4 __attribute__((aligned(4)));
typedef uint16_t nt_h8a2 __attribute__((ext_vector_type(8), aligned(2)));
typedef uint16_t nt_h4a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint16_t nt_h2a2 __attribute__((ext_vector_type(2), aligned(2)));

template <typename V, bool NT, typename T>
__device__ __forceinline__ void ld_stream_as(T &out, const void *p)
{
    static_assert(sizeof(V) == sizeof(T), "size");
    V v;
    if constexpr (NT && KVMIX_STREAM_NT)
        v = __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
    else
        v = *reinterpret_cast<const V *>(p);
    __builtin_memcpy(&out, &v, sizeof(T));
}

template <typename T, bool NT = true>
__device__ __forceinline__ T ld_stream(const void *p)
{
    constexpr int N = sizeof(T);
    constexpr int A = alignof(T);
    T out;
    if constexpr (A >= 4 && N == 16) {
        ld_stream_as<nt_u4a4, NT>(out, p);
    } else if constexpr (A >= 4 && N == 8) {
        ld_stream_as<nt_u2a4, NT>(out, p);
    } else if constexpr (A >= 4 && N == 4) {
        ld_stream_as<nt_u1a4, NT>(out, p);
    } else if constexpr (A >= 4 && N == 12) {
        struct __attribute__((packed, aligned(4))) Lo {
            uint32_t v[2];
        } lo;
        uint32_t hi;
        ld_stream_as<nt_u2a4, NT>(lo, p);
        ld_stream_as<nt_u1a4, NT>(hi, reinterpret_cast<const uint8_t *>(p) + 8);
        __builtin_memcpy(&out, &lo, 8);
        __builtin_memcpy(reinterpret_cast<uint8_t *>(&out) + 8, &hi, 4);
    } else if constexpr (A == 2 && N == 16) {
        ld_stream_as<nt_h8a2, NT>(out, p);
    } else if constexpr (A == 2 && N == 8) {
        ld_stream_as<nt_h4a2, NT>(out, p);
    } else if constexpr (A == 2 && N == 4) {
        ld_stream_as<nt_h2a2, NT>(out, p);
    } else if constexpr (N == 2) {
        ld_stream_as<uint16_t, NT>(out, p);
    } else {
        static_assert(N == 1, "unsupported size for a streamed load");
        ld_stream_as<uint8_t, NT>(out, p);
    }
    return out;
}

// Integer codes are fed to the multiplier as fp16 SUBNORMALS: a 16-bit pattern p < 2048 read
// as binary16 is exactly p * 2^-24 (the first two binades share one ulp).  Masking a field of
// the packed word in place therefore yields two fp16 operands (low and high half of the
// register) with no shift and no int->float conversion, and v_fma_mix_f32 multiplies an fp32
// by an fp16 half directly into an fp32 accumulator.  The 2^-24 and the field's bit offset are
// folded into the fp32 multiplier (powers of two: exact).
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void mix2(float q, uint32_t m, float &acc_lo, float &acc_hi)
{
    const half2_t h = __builtin_bit_cast(half2_t, m);
    acc_lo = fmaf(q, (float)h.x, acc_lo);
    acc_hi = fmaf(q, (float)h.y, acc_hi);
}

__device__ __forceinline__ void mix1(float q, uint32_t m, float &acc)
{
    const half2_t h = __builtin_bit_cast(half2_t, m);
    acc = fmaf(q, (float)h.x, acc);
}

// acc[i] += qs * code_i for the VALS codes held in w[]; qs = x_k * scale_k.
template <int MODE>
__device__ __forceinline__ void accumulate_unit(const uint32_t *w, float qs, float *acc)
{
    [[maybe_unused]] const float q0 = qs * 16777216.0f;  // 2^24 undoes the fp16-subnormal scaling
    if constexpr (MODE == 4) {
        const float q1 = q0 * 0.0625f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t v = w[j], v8 = w[j] >> 8;
            float *a = acc + 8 * j;  // nibble i sits at bit 4i: low half 0..3, high half 4..7
            mix2(q0, v & 0x000F000Fu, a[0], a[4]);
            mix2(q1, v & 0x00F000F0u, a[1], a[5]);
            mix2(q0, v8 & 0x000F000Fu, a[2], a[6]);
            mix2(q1, v8 & 0x00F000F0u, a[3], a[7]);
        }
    } else if constexpr (MODE == 2) {
        const float q1 = q0 * 0.25f, q2 = q0 * 0.0625f, q3 = q0 * 0.015625f;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t v = w[j], v8 = w[j] >> 8;
            float *a = acc + 16 * j;  // code i at bit 2i: low half 0..7, high half 8..15
            mix2(q0, v & 0x00030003u, a[0], a[8]);
            mix2(q1, v & 0x000C000Cu, a[1], a[9]);
            mix2(q2, v & 0x00300030u, a[2], a[10]);
            mix2(q3, v & 0x00C000C0u, a[3], a[11]);
            mix2(q0, v8 & 0x00030003u, a[4], a[12]);
            mix2(q1, v8 & 0x000C000Cu, a[5], a[13]);
            mix2(q2, v8 & 0x00300030u, a[6], a[14]);
            mix2(q3, v8 & 0x00C000C0u, a[7], a[15]);
        }
    } else if constexpr (MODE == 1) {
        float qv[8];
        qv[0] = q0;
#pragma unroll
        for (int s = 1; s < 8; s++) qv[s] = qv[s - 1] * 0.5f;
        const uint32_t v = w[0], v8 = w[0] >> 8;  // bit i: low half 0..15, high half 16..31
#pragma unroll
        for (int s = 0; s < 8; s++) {
            mix2(qv[s], v & (0x00010001u << s), acc[s], acc[16 + s]);
            mix2(qv[s], v8 & (0x00010001u << s), acc[8 + s], acc[24 + s]);
        }
    } else {
        // 3-bit formats: fields are not byte- or half-aligned, so the fp16 trick would need an
        // extract per code.  Instead a masked field of a 32-bit word is read as an fp32
        // SUBNORMAL: a pattern p < 2^24 is exactly p * 2^-149, so `word & (7 << o)` is
        // code * 2^(o-149) and one v_and_b32 + one v_fmac_f32 (both 2-operand encodings, the
        // cheapest VALU class) handle a code.  The multiplier carries 2^(90-o); the sums come
        // out scaled by 2^(90-149) = 2^-59, undone by Fmt::OUT_SCALE.  2^90 keeps x*scale*2^90
        // finite for any fp16 x and scale, and the products stay far above the fp32 subnormals.
        float mq[4];
        mq[0] = qs * 1237940039285380274899124224.0f;  // 2^90
#pragma unroll
        for (int s = 1; s < 4; s++) mq[s] = mq[s - 1] * 0.125f;  // offsets 0, 3, 6, 9
        if constexpr (MODE == 3) {
            // word = ten 3-bit codes at bits 0..29 + a 2-bit code at bits 30..31
            const uint32_t v[3] = {w[0], w[0] >> 12, w[0] >> 24};
#pragma unroll
            for (int i = 0; i < 11; i++) {
                const uint32_t mask = (i == 10 ? 3u : 7u) << (3 * (i % 4));
                acc[i] = fmaf(mq[i % 4], __uint_as_float(v[i / 4] & mask), acc[i]);
            }
        } else {
            // 96-bit stream, code i at bits [3i, 3i+3): eight 12-bit windows of four codes
            uint32_t v[8];
            v[0] = w[0];
            v[1] = w[0] >> 12;
            v[2] = __builtin_amdgcn_alignbit(w[1], w[0], 24);
            v[3] = w[1] >> 4;
            v[4] = w[1] >> 16;
            v[5] = __builtin_amdgcn_alignbit(w[2], w[1], 28);
            v[6] = w[2] >> 8;
            v[7] = w[2] >> 20;
#pragma unroll
            for (int i = 0; i < 32; i++)
                acc[i] = fmaf(mq[i % 4], __uint_as_float(v[i / 4] & (7u << (3 * (i % 4)))), acc[i]);
        }
    }
}

// The same unpack for NREP query heads that share one kv head (GQA): the field of a code is
// isolated ONCE as an fp32 subnormal (`word & mask` is code * 2^(offset-149)) and each head
// pays a single v_fmac_f32.  Shifted copies of the word keep the number of distinct field
// offsets -- hence of per-head multipliers q * 2^(90-offset) -- at four (eight for 1 bit).
// The sums come out scaled by 2^-59 (kHeadsOutScale undoes it), for every format.
constexpr float kHeadsOutScale = 576460752303423488.0f;  // 2^59

template <int MODE, int NREP>
__device__ __forceinline__ void accumulate_heads(const uint32_t *w, const float *q,
                                                 float (*acc)[Fmt<MODE>::VALS])
{
    constexpr int NM = MODE == 1 ? 8 : 4;                       // distinct field offsets
    constexpr int STEP = MODE == 30 ? 3 : MODE;                 // bits between fields of a copy
    constexpr float DOWN = MODE == 4 ? 0.0625f : (MODE == 2 ? 0.25f : (MODE == 1 ? 0.5f : 0.125f));
    float mq[NREP][NM];
#pragma unroll
    for (int h = 0; h < NREP; h++) {
        mq[h][0] = q[h] * 1237940039285380274899124224.0f;  // 2^90
#pragma unroll
        for (int s = 1; s < NM; s++) mq[h][s] = mq[h][s - 1] * DOWN;
    }
    // one masked field -> NREP fmacs
    auto field = [&](uint32_t copy, uint32_t mask, int s, int code) {
        const float f = __uint_as_float(copy & mask);
#pragma unroll
        for (int h = 0; h < NREP; h++) acc[h][code] = fmaf(mq[h][s], f, acc[h][code]);
    };
    if constexpr (MODE == 4) {
#pragma unroll
        for (int j = 0; j < 4; j++) {  // nibble i at bit 4i: copies w and w >> 16, offsets 0,4,8,12
            const uint32_t v0 = w[j], v1 = w[j] >> 16;
#pragma unroll
            for (int s = 0; s < 4; s++) {
                field(v0, 0xFu << (4 * s), s, 8 * j + s);
                field(v1, 0xFu << (4 * s), s, 8 * j + 4 + s);
            }
        }
    } else if constexpr (MODE == 2) {
#pragma unroll
        for (int j = 0; j < 2; j++) {  // code i at bit 2i: copies w >> 8k, offsets 0,2,4,6
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t v = w[j] >> (8 * k);
#pragma unroll
                for (int s = 0; s < 4; s++) field(v, 3u << (2 * s), s, 16 * j + 4 * k + s);
            }
        }
    } else if constexpr (MODE == 1) {
#pragma unroll
        for (int k = 0; k < 4; k++) {  // bit i: copies w >> 8k, offsets 0..7
            const uint32_t v = w[0] >> (8 * k);
#pragma unroll
            for (int s = 0; s < 8; s++) field(v, 1u << s, s, 8 * k + s);
        }
    } else if constexpr (MODE == 3) {
        const uint32_t v[3] = {w[0], w[0] >> 12, w[0] >> 24};
#pragma unroll
        for (int i = 0; i < 11; i++) field(v[i / 4], (i == 10 ? 3u : 7u) << (3 * (i % 4)), i % 4, i);
    } else {
        uint32_t v[8];
        v[0] = w[0];
        v[1] = w[0] >> 12;
        v[2] = __builtin_amdgcn_alignbit(w[1], w[0], 24);
        v[3] = w[1] >> 4;
        v[4] = w[1] >> 16;
        v[5] = __builtin_amdgcn_alignbit(w[2], w[1], 28);
        v[6] = w[2] >> 8;
        v[7] = w[2] >> 20;
#pragma unroll
        for (int i = 0; i < 32; i++) field(v[i / 4], 7u << (3 * (i % 4)), i % 4, i);
    }
}

// Workgroups are handed to the 8 XCDs (each with its own L2) round-robin in launch order, so
// neighbours in launch order never share an L2.  This maps the launch-order index to a
// logical index such that CONSECUTIVE logical indices run on the SAME XCD: column tiles of
// one cache row (they share the 128-byte lines that straddle tile borders) and query heads
// of one kv head (they read the same packed data) then meet in one L2.
constexpr int kXcds = 8;
__device__ __forceinline__ void xcd_swizzled_block(int64_t &bx, int64_t &by, bool enable)
{
    const int64_t nx = gridDim.x, n = nx * (int64_t)gridDim.y;
    const int64_t l = (int64_t)blockIdx.y * nx + blockIdx.x;
    const int64_t xcd = l % kXcds, slot = l / kXcds;
    const int64_t per = n / kXcds, rem = n % kXcds;
    const int64_t j = enable ? xcd * per + (xcd < rem ? xcd : rem) + slot : l;
    bx = j % nx;
    by = j / nx;
}

// LDS traffic between lanes of ONE wave: the wave's instructions execute in order, so a
// ds_read issued after a ds_write sees it; this only stops the compiler from moving them.
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------------------
// gemv_cols<MODE, RQ, UPL>
//   A lane owns UPL consecutive group units of N (one unit = one (scale, zero) pair: 32 codes,
//   or one 11-code word of the reference's 3-bit format) for one of RQ sections of the K rows.
//   wave tile  = TU = (64/RQ) * UPL consecutive units; the LAST tile of a row is shifted left
//                so that it ends exactly at N: every lane of every tile is whole (the overlap
//                is recomputed and stored twice with identical values), so there are no edge
//                cases along N.  The host only takes this kernel when N holds >= TU units.
//   row chunk  = KC = 2048/TU rows: 8 KiB of (scale, zero) half2 pairs per wave in LDS, staged
//                with four 128-bit loads per array per lane; inside a chunk a lane walks
//                KC/RQ = 32/UPL rows of its section, 8 rows of packed codes in flight.
//   Rows past K (last chunk only) are read from row K-1 and meet x == 0.
//   block = (64, 2..4) waves on neighbouring tiles; grid = (tiles/waves, samples, M), XCD-swizzled.
// Offsets inside one (batch, kv-head) slice are 32-bit (the host checks the extents).
// ---------------------------------------------------------------------------------------
constexpr int kColsWaves = 4;

template <int MODE, int RQ, int UPL>
__global__ void __launch_bounds__(64 * kColsWaves) gemv_cols(GemvArgs a)
{
    using F = Fmt<MODE>;
    constexpr int VALS = F::VALS, WORDS = F::WORDS;
    constexpr int GL = kWave / RQ;      // lanes per row section
    constexpr int TU = GL * UPL;        // units per wave tile
    constexpr int KC = 2048 / TU;       // rows per chunk
    constexpr int RPL = KC / RQ;        // rows per lane per chunk (= 32 / UPL)
    constexpr int U = 8;                // rows whose code loads are in flight together
    constexpr int SEGS = TU / 8;        // 8-unit segments per staged row
    constexpr int NIT = (KC * SEGS) / kWave;
    constexpr int LW = WORDS * UPL;     // packed words per lane per row
    static_assert(RPL % U == 0 && NIT == 4 && TU % 8 == 0, "chunk geometry");

    __shared__ uint32_t sz_lds[kColsWaves][KC * TU];  // (scale | zero << 16) per (row, unit)
    __shared__ float x_lds[kColsWaves][KC];

    const int lane = threadIdx.x;
    const int wy = threadIdx.y;
    const int rq = lane / GL;
    const int gl = lane % GL;
    int64_t bx, sample;
    xcd_swizzled_block(bx, sample, true);
    const int64_t m = blockIdx.z;
    const int64_t kv = sample / a.heads_per_kv;
    const int K = (int)a.K;
    const int nunits = (int)(a.N / VALS);
    if (nunits < TU) return;                    // (never launched so: a tile wider than the row would leave the operand)
    int t0 = (int)(bx * blockDim.y + wy) * TU;  // first unit of this wave's tile
    if (t0 >= nunits) return;                   // whole wave outside (no block barrier below)
    t0 = t0 + TU <= nunits ? t0 : max(nunits - TU, 0);  // last tile: shifted left, still whole
    const int unit0 = t0 + gl * UPL;            // this lane's first unit
    const uint32_t c_rs = (uint32_t)a.c_rs, s_rs = (uint32_t)a.s_rs;

    const uint16_t *xp = reinterpret_cast<const uint16_t *>(a.x) + sample * a.x_bs + m * a.x_rs;
    const uint32_t *cp = a.code + kv * a.c_bs;
    const uint16_t *sp = reinterpret_cast<const uint16_t *>(a.scale) + kv * a.s_bs;
    const uint16_t *zp = reinterpret_cast<const uint16_t *>(a.zero) + kv * a.s_bs;
    uint32_t *szw = sz_lds[wy];
    float *xw = x_lds[wy];

    float acc[UPL][VALS];
    float zsum[UPL];
#pragma unroll
    for (int j = 0; j < UPL; j++) {
        zsum[j] = 0.f;
#pragma unroll
        for (int i = 0; i < VALS; i++) acc[j][i] = 0.f;
    }

    const int r0 = rq * RPL;  // this lane's rows inside a chunk: [r0, r0 + RPL)
    const uint32_t lane_word0 = (uint32_t)unit0 * WORDS;

    auto load_batch = [&](Words<LW>(&w)[U], int kc, int b, bool full) {
        const int kfirst = kc + r0 + b;
        if (full) {
            const uint32_t off0 = (uint32_t)kfirst * c_rs + lane_word0;
#pragma unroll
            for (int u = 0; u < U; u++)
                w[u] = ld_stream<Words<LW>, KVMIX_COLS_NT_CODES>(cp + (off0 + (uint32_t)u * c_rs));
        } else {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int k = kfirst + u < K ? kfirst + u : K - 1;
                w[u] = ld_stream<Words<LW>, KVMIX_COLS_NT_CODES>(cp + ((uint32_t)k * c_rs + lane_word0));
            }
        }
    };
    auto compute_batch = [&](const Words<LW>(&w)[U], int b) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int r = r0 + b + u;
            const float xv = xw[r];
#pragma unroll
            for (int j = 0; j < UPL; j++) {
                const half2_t sz = __builtin_bit_cast(half2_t, szw[r * TU + gl * UPL + j]);
                zsum[j] = fmaf(xv, (float)sz.y, zsum[j]);
                accumulate_unit<MODE>(w[u].v + j * WORDS, xv * (float)sz.x, acc[j]);
            }
        }
    };

    for (int kc = 0; kc < K; kc += KC) {
        const int rows = K - kc < KC ? K - kc : KC;
        const bool full = rows == KC;
        // ---- loads of the chunk's (scale, zero) tile and x, then -- before waiting for
        //      them -- the first batch of packed codes ----
        Half8 s8[NIT], z8[NIT];
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int idx = it * kWave + lane;
            const int row = idx / SEGS, seg = idx % SEGS;
            const int rowc = kc + (row < rows ? row : rows - 1);
            const uint32_t off = (uint32_t)rowc * s_rs + (uint32_t)(t0 + seg * 8);
            s8[it] = ld_stream<Half8, false>(sp + off);
            z8[it] = ld_stream<Half8, false>(zp + off);
        }
        uint16_t xh[(KC + kWave - 1) / kWave];
#pragma unroll
        for (int i = 0; i < (KC + kWave - 1) / kWave; i++) {
            const int r = i * kWave + lane;
            xh[i] = xp[kc + (r < rows ? r : rows - 1)];
        }
        Words<LW> w[U];
        load_batch(w, kc, 0, full);
        // ---- tile to LDS ----
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int idx = it * kWave + lane;
            uint32_t pk[8];
#pragma unroll
            for (int e = 0; e < 8; e++) pk[e] = s8[it].v[e] | ((uint32_t)z8[it].v[e] << 16);
            uint4 *dst = reinterpret_cast<uint4 *>(szw + (idx / SEGS) * TU + (idx % SEGS) * 8);
            dst[0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            dst[1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
        }
#pragma unroll
        for (int i = 0; i < (KC + kWave - 1) / kWave; i++) {
            const int r = i * kWave + lane;
            if (r < KC) xw[r] = r < rows ? h16_to_f32(xh[i]) : 0.f;
        }
        wave_lds_fence();
        // ---- stream the codes ----
        compute_batch(w, 0);
#pragma unroll 1
        for (int b = U; b < RPL; b += U) {
            load_batch(w, kc, b, full);
            compute_batch(w, b);
        }
        wave_lds_fence();  // the next chunk overwrites the tile
    }

    // ---- combine the RQ row sections (butterfly over lanes), store fp16 ----
    constexpr float kOut = F::OUT_SCALE;
#pragma unroll
    for (int j = 0; j < UPL; j++) {
#pragma unroll
        for (int i = 0; i < VALS; i++) {
            float v = fmaf(acc[j][i], kOut, zsum[j]);
#pragma unroll
            for (int off = GL; off < kWave; off <<= 1) v += __shfl_xor(v, off);
            acc[j][i] = v;
        }
    }
    uint16_t *op = reinterpret_cast<uint16_t *>(a.out) + sample * a.o_bs + m * a.o_rs + (int64_t)unit0 * VALS;
    constexpr int TOT = UPL * VALS;  // consecutive outputs of this lane
    if constexpr (TOT % (2 * RQ) == 0) {
        // every lane of a column holds all sums: section rq stores its share
        constexpr int PER = TOT / RQ;
#pragma unroll
        for (int s = 0; s < RQ; s++) {
            if (rq == s) {
#pragma unroll
                for (int i = 0; i < PER; i += 2) {
                    const int e = s * PER + i;
                    const uint32_t pk = f32_to_h16(acc[e / VALS][e % VALS]) |
                                        ((uint32_t)f32_to_h16(acc[(e + 1) / VALS][(e + 1) % VALS]) << 16);
                    __builtin_memcpy(op + e, &pk, 4);
                }
            }
        }
    } else {
        if (rq == 0) {
#pragma unroll
            for (int e = 0; e < TOT; e++) op[e] = f32_to_h16(acc[e / VALS][e % VALS]);
        }
    }
}

// ---------------------------------------------------------------------------------------
// gemv_cols3<RQ>   q.K^T shape for the reference's 3-bit format (11 codes per word, one
// (scale, zero) pair per word, so half of the bytes are scales and zeros).
//   A lane owns 4 consecutive words of N for one of RQ sections of the K rows: per row it
//   loads 16 bytes of codes, 8 of scales and 8 of zeros straight into registers -- no LDS
//   staging, no barriers in the stream.  U rows are in flight per lane: a row's registers
//   are refilled with row k+U right after row k is consumed, every load unconditional
//   (rows past the section are redirected to the last row and meet x == 0) and pinned in
//   place with scheduling barriers, so the load queue never drains.
//   x is converted once per block into LDS (fp32, with a zero in slot K for the redirected
//   rows).  Tiles as in gemv_cols: TU = (64/RQ)*4 words per wave, last tile shifted left.
//   block = (64, 2..4); grid = (tiles/waves, samples, M), XCD-swizzled; dynamic LDS = (K+1)*4.
// ---------------------------------------------------------------------------------------
constexpr float kCols3ZeroDown = 8.0779356694631608874e-28f;  // 2^-90: the zero term is accumulated with x * 2^90
// 2^(59 - offset of code i inside its word or inside word >> 24): undoes the fp32-pattern scaling
__device__ __forceinline__ constexpr float cols3_out_scale(int i)
{
    float v = 576460752303423488.0f;  // 2^59
    for (int k = 0; k < 3 * (i < 8 ? i : i - 8); k++) v *= 0.5f;
    return v;
}

template <int RQ, int UPL, int U, int NREP>
__global__ void __launch_bounds__(64 * kColsWaves) __attribute__((amdgpu_waves_per_eu(NREP > 1 ? kCols3HeadsOcc : 3)))
gemv_cols3(GemvArgs a)
{
    constexpr int VALS = 11;
    constexpr int GL = kWave / RQ;
    constexpr int TU = GL * UPL;
    extern __shared__ float xs[];  // [NREP][K + 1]

    const int lane = threadIdx.x;
    const int wy = threadIdx.y;
    const int rq = lane / GL;
    const int gl = lane % GL;
    // grid.y counts head groups: NREP query heads that share one kv head (NREP == 1: plain)
    int64_t bx, hg;
    xcd_swizzled_block(bx, hg, true);
    const int64_t sample0 = hg * NREP;
    const int64_t m = blockIdx.z;
    const int64_t kv = sample0 / a.heads_per_kv;
    const int K = (int)a.K;
    const int nunits = (int)(a.N / VALS);
    if (nunits < TU) return;  // (never launched so: a tile wider than the row would leave the operand; the same for every thread)

    const uint16_t *xp = reinterpret_cast<const uint16_t *>(a.x) + sample0 * a.x_bs + m * a.x_rs;
    for (int i = wy * kWave + lane; i < NREP * (K + 1); i += blockDim.y * kWave) {
        const int h = i / (K + 1), k = i % (K + 1);
        xs[i] = k < K ? h16_to_f32(xp[h * a.x_bs + k]) * 1237940039285380274899124224.0f : 0.f;  // x * 2^90, see compute_row
    }
    __syncthreads();

    // ks > 1: ks neighbouring waves share a tile and each takes a share of the K rows (wide tiles --
    // long contiguous pieces per row -- for launches that would otherwise have too few waves);
    // their sums meet in LDS behind the x vector
    const int ks = a.ksplit;
    const int slice = wy % ks;
    int t0 = (int)(bx * (blockDim.y / ks) + wy / ks) * TU;
    if (t0 >= nunits) {
        if (ks > 1) __syncthreads();  // (the barrier of the combine step)
        return;
    }
    t0 = t0 + TU <= nunits ? t0 : max(nunits - TU, 0);
    const int unit0 = t0 + gl * UPL;
    const uint32_t c_rs = (uint32_t)a.c_rs, s_rs = (uint32_t)a.s_rs;
    const uint32_t *cp = a.code + kv * a.c_bs + unit0;
    const uint16_t *sp = reinterpret_cast<const uint16_t *>(a.scale) + kv * a.s_bs + unit0;
    const uint16_t *zp = reinterpret_cast<const uint16_t *>(a.zero) + kv * a.s_bs + unit0;

    float acc[UPL][NREP][VALS];
    float zsum[NREP][UPL];
#pragma unroll
    for (int j = 0; j < UPL; j++) {
#pragma unroll
        for (int h = 0; h < NREP; h++) {
            zsum[h][j] = 0.f;
#pragma unroll
            for (int i = 0; i < VALS; i++) acc[j][h][i] = 0.f;
        }
    }

    // this lane's rows: [kbeg, kend), walked in steps of U
    const int kq = (K + RQ * ks - 1) / (RQ * ks);
    const int kbeg = (slice * RQ + rq) * kq;
    const int kend = kbeg + kq < K ? kbeg + kq : K;
    const int steps = (kq + U - 1) / U;  // the same for every section: uniform control flow

    struct __attribute__((packed, aligned(2))) HalfN {
        uint16_t v[UPL];
    };
    Words<UPL> cw[U];
    HalfN sw[U], zw[U];
    auto load_row = [&](int u, int k) {
        const uint32_t kc = (uint32_t)(k < kend ? k : K - 1);
        cw[u] = ld_stream<Words<UPL>, KVMIX_COLS_NT_CODES>(cp + kc * c_rs);
        sw[u] = ld_stream<HalfN, (KVMIX_COLS3_NT_SZ && NREP == 1)>(sp + kc * s_rs);
        zw[u] = ld_stream<HalfN, (KVMIX_COLS3_NT_SZ && NREP == 1)>(zp + kc * s_rs);
    };
    // x of the U rows of a step is read from LDS in one go at the head of the step: read row by row,
    // each read's latency sits in front of that row's arithmetic
    float xr[U][NREP];
    auto load_x = [&](int k0) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int kx = k0 + u < kend ? k0 + u : K;
#pragma unroll
            for (int h = 0; h < NREP; h++) xr[u][h] = xs[h * (K + 1) + kx];
        }
    };
    auto compute_row = [&](int u, int k) {
        float xv[NREP];
#pragma unroll
        for (int h = 0; h < NREP; h++) xv[h] = xr[u][h];
#pragma unroll
        for (int j = 0; j < UPL; j++) {
            const half2_t sz = __builtin_bit_cast(half2_t, (uint32_t)sw[u].v[j] | ((uint32_t)zw[u].v[j] << 16));
            // A masked field of the word, read as an fp32 pattern below 2^24, is code * 2^(offset-149)
            // (subnormals and the first binade share one ulp): codes 0..7 come straight out of the
            // word (offsets 0..21), codes 8..10 out of word >> 24.  One multiplier x*scale*2^90 per
            // head serves every position; the factor 2^offset stays in the sum and is taken out once,
            // at the end (cols3_out_scale) -- a power of two, so nothing is rounded differently.
            const uint32_t w = cw[u].v[j], hi = w >> 24;
            float f[VALS];
#pragma unroll
            for (int i = 0; i < 8; i++) f[i] = __uint_as_float(w & (7u << (3 * i)));
            f[8] = __uint_as_float(hi & 0x07u);
            f[9] = __uint_as_float(hi & 0x38u);
            f[10] = __uint_as_float(hi & 0xC0u);
#pragma unroll
            // (x arrives multiplied by 2^90: the zero term carries the factor too and loses it at the end;
            // it stays finite up to |sum x * zero| = 2^37, far beyond what an fp16 result can hold)
            for (int h = 0; h < NREP; h++) {
                zsum[h][j] = fmaf(xv[h], (float)sz.y, zsum[h][j]);
                const float mq = fmaf(xv[h], (float)sz.x, 0.f);  // (a multiply; written as an fma so that the fp16 operand needs no conversion)
#pragma unroll
                for (int i = 0; i < VALS; i++) acc[j][h][i] = fmaf(mq, f[i], acc[j][h][i]);
            }
        }
    };

    if (kq % U == 0 && kbeg + kq <= K) {
        // Every section is a whole number of steps (head dimensions of 64, 128, 256 are): the rows are
        // walked with three running pointers -- one 64-bit add per load instead of a clamp, a
        // multiply and an add -- and the last step prefetches nothing, so no row past the section is
        // ever addressed.
        // (uniform bases and 32-bit byte offsets per lane: the form a load with a scalar base takes)
        const uint8_t *cb = reinterpret_cast<const uint8_t *>(a.code + kv * a.c_bs);
        const uint8_t *sb = reinterpret_cast<const uint8_t *>(reinterpret_cast<const uint16_t *>(a.scale) + kv * a.s_bs);
        const uint8_t *zb = reinterpret_cast<const uint8_t *>(reinterpret_cast<const uint16_t *>(a.zero) + kv * a.s_bs);
        uint32_t co = ((uint32_t)unit0 + (uint32_t)kbeg * c_rs) * 4u;
        uint32_t so = ((uint32_t)unit0 + (uint32_t)kbeg * s_rs) * 2u;
        const uint32_t c_step = c_rs * 4u, s_step = s_rs * 2u;
        auto next_row = [&](int u) {
            cw[u] = ld_stream<Words<UPL>, KVMIX_COLS_NT_CODES>(cb + co);
            sw[u] = ld_stream<HalfN, (KVMIX_COLS3_NT_SZ && NREP == 1)>(sb + so);
            zw[u] = ld_stream<HalfN, (KVMIX_COLS3_NT_SZ && NREP == 1)>(zb + so);
            co += c_step;
            so += s_step;
        };
        auto step_x = [&](int k0) {
#pragma unroll
            for (int u = 0; u < U; u++) {
#pragma unroll
                for (int h = 0; h < NREP; h++) xr[u][h] = xs[h * (K + 1) + k0 + u];
            }
        };
#pragma unroll
        for (int u = 0; u < U; u++) {
            next_row(u);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll 1
        for (int st = 0; st < steps - 1; st++) {
            const int k0 = kbeg + st * U;
            step_x(k0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U; u++) {
                compute_row(u, k0 + u);
                next_row(u);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        step_x(kbeg + (steps - 1) * U);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; u++) compute_row(u, kbeg + (steps - 1) * U + u);
    } else {
#pragma unroll
        for (int u = 0; u < U; u++) {
            load_row(u, kbeg + u);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll 1
        for (int st = 0; st < steps; st++) {
            const int k0 = kbeg + st * U;
            load_x(k0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U; u++) {
                compute_row(u, k0 + u);
                load_row(u, k0 + U + u);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // ---- combine the RQ row sections, store fp16 (2^59 undoes the fp32-subnormal scaling) ----
    constexpr int TOT = UPL * VALS;  // consecutive outputs of this lane
    float *part = xs + NREP * (K + 1);  // [waves][NREP][TOT][64] when ks > 1
    if (ks > 1) {
        if (slice > 0) {
#pragma unroll
            for (int h = 0; h < NREP; h++) {
#pragma unroll
                for (int j = 0; j < UPL; j++) {
#pragma unroll
                    for (int i = 0; i < VALS; i++)
                        part[((wy * NREP + h) * TOT + j * VALS + i) * kWave + lane] = fmaf(acc[j][h][i], cols3_out_scale(i), zsum[h][j] * kCols3ZeroDown);
                }
            }
        }
        __syncthreads();
        if (slice > 0) return;
    }
#pragma unroll
    for (int h = 0; h < NREP; h++) {
        float flat[TOT];
#pragma unroll
        for (int j = 0; j < UPL; j++) {
#pragma unroll
            for (int i = 0; i < VALS; i++) flat[j * VALS + i] = fmaf(acc[j][h][i], cols3_out_scale(i), zsum[h][j] * kCols3ZeroDown);
        }
        for (int o = 1; o < ks; o++) {
#pragma unroll
            for (int e = 0; e < TOT; e++) flat[e] += part[(((wy + o) * NREP + h) * TOT + e) * kWave + lane];
        }
        uint16_t *op = reinterpret_cast<uint16_t *>(a.out) + (sample0 + h) * a.o_bs + m * a.o_rs + (int64_t)unit0 * VALS;
        if constexpr (RQ == 1) {
#pragma unroll
            for (int e = 0; e + 1 < TOT; e += 2) {
                const uint32_t pk = f32_to_h16(flat[e]) | ((uint32_t)f32_to_h16(flat[e + 1]) << 16);
                __builtin_memcpy(op + e, &pk, 4);
            }
            if constexpr (TOT % 2 == 1) op[TOT - 1] = f32_to_h16(flat[TOT - 1]);
        } else {
            // halving butterfly: each section ends with its share of the sums (TOT / RQ each)
            static_assert(RQ == 2 && TOT % 2 == 0, "two sections, equal shares");
            const int first = scatter_reduce<TOT, GL, 1>(flat, lane);
            constexpr int PER = TOT / RQ;
            if constexpr (PER % 2 == 0) {
#pragma unroll
                for (int e = 0; e < PER; e += 2) {
                    const uint32_t pk = f32_to_h16(flat[e]) | ((uint32_t)f32_to_h16(flat[e + 1]) << 16);
                    __builtin_memcpy(op + first + e, &pk, 4);
                }
            } else {
#pragma unroll
                for (int e = 0; e < PER; e++) op[first + e] = f32_to_h16(flat[e]);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// gemv_rows<MODE, LPR>
//   LPR = N/32 lanes per row (one 32-code group each), RPW = 64/LPR rows per tile,
//   chunk = 8 tiles = 512/LPR rows: its scale array is 512 halves = one 128-bit load per lane.
//   The lane that loads scale/zero element e also loads that row's x, forms x*scale (to LDS,
//   fp32) and accumulates x*zero privately; the zero term is reduced once at the end.
//   Chunks of a block's row range go round-robin to its KW waves.
//   block = (64, KW); grid = (splits, samples, M); dynamic LDS = KW * (512 + N) floats.
//   Requires scale/zero rows to be contiguous (row stride == LPR).
// ---------------------------------------------------------------------------------------
constexpr int kRowsMaxWaves = 16;  // plain (one head per block) configuration

// NREP > 1 (GQA): one block serves NREP query heads of a kv head from one pass over the
// packed data -- NREP x 32 accumulators per lane, so such a block has at most four waves and
// the kernel is compiled for the larger register budget that goes with it.
constexpr int kRowsHeadsWaves = 4;

template <int MODE, int LPR, int NREP>
__global__ void __launch_bounds__(NREP > 1 ? 64 * kRowsHeadsWaves : 64 * kRowsMaxWaves) gemv_rows(GemvArgs a)
{
    using F = Fmt<MODE>;
    constexpr int VALS = F::VALS, WORDS = F::WORDS;
    static_assert(VALS == 32, "gemv_rows handles 32-code groups");
    static_assert(LPR <= 8 && 8 % LPR == 0, "one staging lane covers whole rows");
    constexpr int RPW = kWave / LPR;   // rows per tile
    constexpr int TILES = 8;           // tiles per chunk, all in flight
    constexpr int CH = TILES * RPW;    // rows per chunk (= 512 / LPR)
    constexpr int RPS = 8 / LPR;       // rows covered by one staging lane's 8 halves
    constexpr int QT = CH * LPR;       // floats of one head's x*scale tile (= 512)

    extern __shared__ float lds[];
    const int lane = threadIdx.x;
    const int wy = threadIdx.y;
    const int KW = blockDim.y;
    float *qw = lds + wy * (NREP * QT);           // this wave's x*scale tiles, one per query head
    float *red = lds + KW * (NREP * QT);          // [KW][NREP][LPR*VALS] block reduction
    const int r = lane / LPR;
    const int j = lane % LPR;
    // grid.y counts head groups: NREP query heads that share one kv head (NREP divides
    // heads_per_kv; NREP == 1 is the plain case)
    // (measured: with one query head per kv head nothing is shared between blocks and the
    // launch order is 3 us faster at B=16, T=8k; with GQA the heads of a kv head want one L2)
    int64_t split, hg;
    xcd_swizzled_block(split, hg, a.heads_per_kv > NREP);
    const int64_t sample0 = hg * NREP;
    const int64_t m = blockIdx.z;
    const int64_t kv = sample0 / a.heads_per_kv;
    const int64_t kbeg = split * a.rows_per_split;
    const int64_t kend = kbeg + a.rows_per_split < a.K ? kbeg + a.rows_per_split : a.K;

    const uint16_t *xp = reinterpret_cast<const uint16_t *>(a.x) + sample0 * a.x_bs + m * a.x_rs;
    const uint32_t *cp = a.code + kv * a.c_bs + j * WORDS;
    const uint16_t *sp = reinterpret_cast<const uint16_t *>(a.scale) + kv * a.s_bs;
    const uint16_t *zp = reinterpret_cast<const uint16_t *>(a.zero) + kv * a.s_bs;

    float acc[NREP][VALS];
    float zacc[NREP][LPR];  // x*zero sums of the elements this lane staged, by head and group
#pragma unroll
    for (int h = 0; h < NREP; h++) {
#pragma unroll
        for (int i = 0; i < VALS; i++) acc[h][i] = 0.f;
#pragma unroll
        for (int i = 0; i < LPR; i++) zacc[h][i] = 0.f;
    }

    const int e0 = lane * 8;    // first element of the chunk's [CH][LPR] scale array this lane stages
    const int row0 = e0 / LPR;  // its 8 elements are RPS whole rows

    // ---- rotating software pipeline over this wave's chunks -----------------------------
    // Register sets: S (scale / zero / x of a chunk), X (codes of row tiles 0..3), Y (tiles
    // 4..7).  Each set is refilled with the NEXT chunk's data right after its last use, so
    // while a chunk is being consumed the next one's loads are in flight and nothing is held
    // twice.  No load sits behind a branch (a conditional load makes the compiler drain the
    // whole queue): rows past the end are redirected to the last valid row and meet
    // x*scale == 0; a prefetch past the last chunk re-reads the current one.
    // With NREP > 1 the packed codes, scales and zeros are loaded once and used for every
    // query head of the group; the field masks of the unpack are shared as well.
    constexpr int HT = TILES / 2;
    const uint32_t c_rs = (uint32_t)a.c_rs;
    const int ke32 = (int)kend;
    const int stride = KW * CH;
    const int kfirst = (int)kbeg + wy * CH;
    Half8 s8, z8;
    uint16_t xh[NREP][RPS];
    Words<WORDS> wx[HT], wz[HT];

    auto load_small = [&](int k0) {
        int kr = k0 + row0;  // a window cut by the end of the range is read one window early
        kr = kr + RPS <= ke32 ? kr : ke32 - RPS;  // (in bounds: the host routes K < 8 elsewhere)
        kr = kr < 0 ? 0 : kr;
        s8 = ld_stream<Half8>(sp + (uint32_t)kr * LPR);
        z8 = ld_stream<Half8>(zp + (uint32_t)kr * LPR);
#pragma unroll
        for (int h = 0; h < NREP; h++) {
#pragma unroll
            for (int q = 0; q < RPS; q++)
                xh[h][q] = xp[h * a.x_bs + (k0 + row0 + q < ke32 ? k0 + row0 + q : ke32 - 1)];
        }
    };
    auto load_codes = [&](Words<WORDS>(&w)[HT], int k0, int t0) {
#pragma unroll
        for (int t = 0; t < HT; t++) {
            int k = k0 + (t0 + t) * RPW + r;
            k = k < ke32 ? k : ke32 - 1;
            w[t] = ld_stream<Words<WORDS>>(cp + (uint32_t)k * c_rs);
        }
    };
    auto stage = [&](int k0) {
        const int rows = ke32 - k0;  // >= 1; >= CH for every chunk but the last
        if (row0 < rows && row0 + RPS > rows) {
            // the lane whose window is cut by the end of the range: element loads
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const bool ok = (e0 + e) / LPR < rows;
                const uint32_t off = (uint32_t)k0 * LPR + (ok ? e0 + e : 0);
                const uint16_t s1 = sp[off], z1 = zp[off];
                s8.v[e] = ok ? s1 : (uint16_t)0;
                z8.v[e] = ok ? z1 : (uint16_t)0;
            }
        }
        float sf[8], zf[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            sf[e] = h16_to_f32(s8.v[e]);
            zf[e] = h16_to_f32(z8.v[e]);
        }
#pragma unroll
        for (int h = 0; h < NREP; h++) {
            float qv[8];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float xv = row0 + e / LPR < rows ? h16_to_f32(xh[h][e / LPR]) : 0.f;
                qv[e] = xv * sf[e];
                zacc[h][e % LPR] = fmaf(xv, zf[e], zacc[h][e % LPR]);
            }
            float4 *dst = reinterpret_cast<float4 *>(qw + h * QT + e0);
            dst[0] = make_float4(qv[0], qv[1], qv[2], qv[3]);
            dst[1] = make_float4(qv[4], qv[5], qv[6], qv[7]);
        }
    };
    auto compute = [&](const Words<WORDS>(&w)[HT], int t0) {
#pragma unroll
        for (int t = 0; t < HT; t++) {
            if constexpr (NREP == 1) {
                accumulate_unit<MODE>(w[t].v, qw[((t0 + t) * RPW + r) * LPR + j], acc[0]);
            } else {
                float qs[NREP];
#pragma unroll
                for (int h = 0; h < NREP; h++) qs[h] = qw[h * QT + ((t0 + t) * RPW + r) * LPR + j];
                accumulate_heads<MODE, NREP>(w[t].v, qs, acc);
            }
        }
    };

    if (kfirst < ke32) {
        load_small(kfirst);
        load_codes(wx, kfirst, 0);
        load_codes(wz, kfirst, HT);
#pragma unroll 1
        for (int k0 = kfirst; k0 < ke32; k0 += stride) {
            const int kn = k0 + stride < ke32 ? k0 + stride : k0;
            stage(k0);
            wave_lds_fence();
            load_small(kn);
            compute(wx, 0);
            load_codes(wx, kn, 0);
            compute(wz, HT);
            load_codes(wz, kn, HT);
            wave_lds_fence();  // the next chunk overwrites the tile
        }
    }

    // ---- reduce over the wave's rows ------------------------------------------------------
    // Both sums use a halving butterfly: at every step a lane keeps one half of its values
    // and hands the other half to its partner, so the exchange count halves per step.
    // zero term: zacc[h][g] summed over all lanes; lane (r, j) ends with the sum for g == j
    float zterm[NREP];
#pragma unroll
    for (int h = 0; h < NREP; h++) {
        float z[LPR];
#pragma unroll
        for (int g = 0; g < LPR; g++) z[g] = zacc[h][g];
        scatter_reduce<LPR, LPR / 2, 0>(z, lane);          // over j: the lane's own group remains
#pragma unroll
        for (int off = LPR; off < kWave; off <<= 1) z[0] += __shfl_xor(z[0], off);  // over rows
        zterm[h] = z[0];
    }
    // code sums: NREP*32 values summed over the RPW rows, NREP*32/RPW of them left per lane
    constexpr int NV = NREP * VALS;
    constexpr int KEEP = NV / RPW;
    static_assert(KEEP >= 1, "a lane keeps at least one sum");
    float *flat = &acc[0][0];
    const int first = scatter_reduce<NV, LPR, 1>(flat, lane);  // index (h*32 + i) of flat[0]
#pragma unroll
    for (int i = 0; i < KEEP; i++) {
        const int f = first + i;
        const int h = f / VALS;  // (KEEP divides 32: a lane's sums belong to one head)
        float zt = zterm[0];
#pragma unroll
        for (int hh = 1; hh < NREP; hh++) zt = h == hh ? zterm[hh] : zt;
        red[(wy * NREP + h) * (LPR * VALS) + j * VALS + f % VALS] =
            fmaf(flat[i], NREP == 1 ? F::OUT_SCALE : kHeadsOutScale, zt);
    }
    __syncthreads();
    for (int t = wy * kWave + lane; t < NREP * LPR * VALS; t += KW * kWave) {
        const int h = t / (LPR * VALS), n = t % (LPR * VALS);
        float v = 0.f;
        for (int w = 0; w < KW; w++) v += red[(w * NREP + h) * (LPR * VALS) + n];
        if (a.splits == 1)
            a.out[(sample0 + h) * a.o_bs + m * a.o_rs + n] = __float2half_rn(v);
        else
            a.partial[(((sample0 + h) * a.M + m) * a.splits + split) * a.N + n] = v;
    }
}

// ---------------------------------------------------------------------------------------
// gemv_rows_mfma<BITS, NREP>   p.V shape, 1/2/4-bit codes, N = 128: the multiply-accumulate
// runs on the matrix cores, the vector ALU only isolates the code fields.
//
// Instruction: v_mfma_f32_4x4x4 (bf16, 16 independent 4x4x4 blocks per wave).  Block b is
// lanes 4b..4b+3; per block  D[i][j] += sum_k A[i][k] * B[k][j]  with lane 4b+j supplying
// column j of B (four k values, two registers), lane 4b+i supplying row i of A, and lane
// 4b+j receiving column j of D (four registers, i = 0..3).
//
// Mapping: a lane owns 8 consecutive codes of a row (BITS bytes: one dword, ushort or byte
// load), 16 lanes cover a row, so one load instruction reads 4 cache rows (contiguous).
// The four lanes of a block hold the 32 codes of ONE quantization group of one row, so they
// share x*scale: that is the A operand.
//   k   <-> the 4 rows a lane holds after four loads (rows rs, rs+4, rs+8, rs+12 of a
//           16-row k-block, rs = lane/16);
//   B   <-> codes: v_perm_b32 puts byte b of two rows' elements into the low bytes of the two
//           halves of a register and one v_and_b32 isolates a field of both.  An 8-bit
//           pattern p in the low byte of a bf16 IS the number p * 2^-133 (subnormals and the
//           first binade share one ulp), so the masked register is a bf16 pair with no
//           shift and no conversion; a field at bit offset o simply counts 2^o-fold.
//   A   <-> x*scale*2^90 split into three bf16 (8 significant bits each: the product of two
//           fp16 has at most 22, so the split is exact).  2^90 keeps every product far above
//           the fp32 subnormals and below overflow for any fp16 x and scale.  The 3*NREP
//           (head, part) rows are packed four to an MFMA; unused rows are zero.
//   D   <-> lane l accumulates, for each of its 8 code positions p, partial sums of output
//           column 8*(l%16)+p over its rows, one per A row; the parts are added at the end.
// NREP query heads of one kv head reuse the B registers.
// x*scale is formed once per (row, group) by the lane that loaded that scale (as in
// gemv_rows) and parked, already split, in the wave's LDS tile in A-operand order.
// block = (64, KW); grid = (splits, samples/NREP, M); dynamic LDS = KW * NM A tiles,
// NM = ceil(3*NREP/4).
// ---------------------------------------------------------------------------------------
typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// v_perm_b32 of two elements of one, two or four bytes.  Two-byte elements go in as they sit in their registers
// (as half-precision operands: an integer operand of 16 bits would be extended first): the selectors used here
// never pick a byte above the element, and written in C++ the compiler zero-extends a narrow value that lives
// across loop iterations again at every use (one v_and_b32 per element and k-block).
template <typename T>
__device__ __forceinline__ uint32_t perm_elems(T hi, T lo, uint32_t sel)
{
    if constexpr (sizeof(T) != 2 || !KVMIX_ROWS_RAW_PERM) {
        return __builtin_amdgcn_perm((uint32_t)hi, (uint32_t)lo, sel);
    } else {
        uint32_t r;
        asm("v_perm_b32 %0, %1, %2, %3" : "=v"(r) : "v"(__builtin_bit_cast(_Float16, hi)), "v"(__builtin_bit_cast(_Float16, lo)), "s"(sel));
        return r;
    }
}

template <int BITS>
struct CodeElem;
template <>
struct CodeElem<4> {
    using type = uint32_t;
};
template <>
struct CodeElem<2> {
    using type = uint16_t;
};
template <>
struct CodeElem<1> {
    using type = uint8_t;
};
template <>
struct CodeElem<30> {
    using type = uint32_t;
};

// B operand of field f of a byte that sits in the low byte of both halves of t (everything else zero).
// The mask keeps the fields 0..f, not f alone: the accumulator then holds the sum over fields 0..f (field j
// counting 2^(j*BITS)-fold) and the kernels' last step takes the difference of neighbouring accumulators.
// For the top field that is the whole byte and no instruction at all (measured at B = 16, T = 8k: p.V 4-bit
// 55.4 -> 53.7 us, 2-bit 36.7 -> 35.0; q.K^T 64.9 -> 63.4 and 40.0 -> 39.3).  The differences cost accuracy
// of the order of one fp32 rounding of the larger sum, far inside the tolerance of the fp32 accumulation.
template <int BITS>
__device__ __forceinline__ uint32_t field_operand(uint32_t t, int f)
{
    constexpr int FPB = 8 / BITS;
    if (f == FPB - 1) return t;
    return t & (((1u << (BITS * (f + 1))) - 1u) * 0x00010001u);
}
// the sum of field f alone from the accumulated sums of a byte's fields (cur: fields 0..f, prev: 0..f-1)
__device__ __forceinline__ float field_sum(float cur, float prev, int f)
{
    return f > 0 ? cur - prev : cur;
}
// The same two with the low fields moved up in their byte (p.V kernels).  The matrix cores align the four
// products of a sum by their operands' exponent fields, which all byte patterns share, so a pattern with leading
// zeros leaves that many fewer bits for a sum its product dominates -- a row of probabilities with one large entry
// (measured with a probe: one product with a subnormal operand exact, four off by up to 2^-17 of their sum while
// the accumulator is the smaller addend; once it dominates, the sum is exact and rounded to nearest.  With the
// fields in place a 2-bit p.V carries 18 bits of a dominant product, a 4-bit one 20, which shows where the code
// term and the zero term of an output cancel).
#ifndef KVMIX_ROWS_FIELDS_TOP
#define KVMIX_ROWS_FIELDS_TOP 1
#endif
// bits the fields 0..f are moved up by: the fields of the low nibble by four, so that one shifted copy of the
// register serves them all and no operand of a dominant product has more than three leading zeros (1-bit codes;
// two for 2-bit codes, none for 4-bit codes) where in place it has up to seven (six, four)
template <int BITS>
__device__ __forceinline__ constexpr int field_shift(int f)
{
    return BITS * (f + 1) <= 4 ? 4 : 0;
}
template <int BITS>
__device__ __forceinline__ uint32_t field_operand_top(uint32_t t, int f)
{
    constexpr int FPB = 8 / BITS;
    if (f == FPB - 1) return t;
    const int sh = field_shift<BITS>(f);
    const uint32_t mask = ((1u << (BITS * (f + 1))) - 1u) * 0x00010001u;
    return sh > 0 ? (t << sh) & (mask << sh) : t & mask;
}
// sum of field f alone, counting 2^(BITS * f + field_shift(f))-fold
template <int BITS>
__device__ __forceinline__ float field_sum_top(float cur, float prev, int f)
{
    if (f == 0) return cur;
    const int d = field_shift<BITS>(f - 1) - field_shift<BITS>(f);  // prev counts 2^d-fold against cur
    return fmaf(prev, -1.0f / (float)(1 << d), cur);
}
// bit offset field f of a byte counts with
template <int BITS>
__device__ __forceinline__ constexpr int field_offset_top(int f)
{
    return BITS * f + field_shift<BITS>(f);
}

// bf16 parts x*scale*2^90 is split into: three (24 significant bits hold the product of two fp16 exactly).  One
// query head: its three rows fit one MFMA.  Four heads per pass: twelve rows, three MFMAs per B operand.
// KVMIX_HEADS_PARTS = 2 (measurement only; p.V kernel) rounds the second part to nearest instead -- every product off
// by up to 2^-17 of itself, eight rows, two MFMAs per B operand, a third of the staging gone: 2-bit p.V at B = 16,
// 32 / 8 heads, T = 32768 70 -> 55 us.  Not shipped: where the code term and the zero term of an output nearly cancel
// (a peaked probability row on a value near zero) that error took a 4-bit case at K = 128 from 0.65 to 1.4 times the
// GEMV tolerance (tests/test_gpu_gemv.py holds the case).
// (What the matrix cores keep of a sum of such products, and what the p.V kernels do about it: field_operand_top.)
#ifndef KVMIX_HEADS_PARTS
#define KVMIX_HEADS_PARTS 3
#endif
constexpr int rows_mfma_parts(int nrep) { return nrep > 1 ? KVMIX_HEADS_PARTS : 3; }   // p.V
constexpr int cols_mfma_parts(int) { return 3; }                                        // q.K^T
constexpr int mfma_sets(int parts, int nrep) { return (parts * nrep + 3) / 4; }
constexpr int rows_mfma_sets(int nrep) { return mfma_sets(rows_mfma_parts(nrep), nrep); }
constexpr int cols_mfma_sets(int nrep) { return mfma_sets(cols_mfma_parts(nrep), nrep); }
// v (= x*scale*2^90) as NP bf16, part i in the high half of part[i]: all but the last by truncation (the
// remainders are exact); the last holds what is left exactly when NP = 3 and is rounded to nearest otherwise
// (a carry into the exponent is the next power of two, as it should be; v is far from overflow)
template <int NP>
__device__ __forceinline__ void split_bf16_parts(float v, uint32_t *part)
{
#pragma unroll
    for (int i = 0; i + 1 < NP; i++) {
        part[i] = __float_as_uint(v) & 0xffff0000u;
        v -= __uint_as_float(part[i]);
    }
    part[NP - 1] = NP >= 3 ? __float_as_uint(v) : __float_as_uint(v) + 0x8000u;
}
// the sum over the parts' accumulators of head h at code position p
template <int NP, int NM, int NPOS>
__device__ __forceinline__ float parts_sum(const f32x4_t (&acc)[NM][NPOS], int h, int p)
{
    float s = acc[(NP * h) / 4][p][(NP * h) % 4];
#pragma unroll
    for (int i = 1; i < NP; i++) s += acc[(NP * h + i) / 4][p][(NP * h + i) % 4];
    return s;
}
constexpr int kRowsMfmaTile = (32 * 17 + 1) * 4 + 4;  // bf16 elements of one A tile (32 skewed rows), 8-byte multiple

constexpr int kRowsMfmaWaves = 16;  // waves per block at most (register budget of 128 per lane)

template <int BITS, int NREP, int DEPTH>
__global__ void __launch_bounds__(64 * (NREP > 1 ? kRowsHeadsWaves : kRowsMfmaWaves))
    __attribute__((amdgpu_waves_per_eu(NREP > 1 ? kMfmaHeadsOcc : 4))) gemv_rows_mfma(GemvArgs a)
{
    // BITS = 30: dense 3-bit stream, a lane's 8 codes are 3 bytes
    using Elem = typename CodeElem<BITS>::type;
    constexpr int EB = BITS == 30 ? 3 : BITS;   // bytes of a lane's 8 codes
    constexpr int FB = BITS == 30 ? 3 : BITS;   // bits of a code
    constexpr int LPR = 4;             // groups per row (N = 128)
    constexpr int EPR = 16;            // lanes (8-code elements) per row
    constexpr int RL = kWave / EPR;    // rows per load instruction (4)
    constexpr int RKB = 4 * RL;        // rows per k-block (16)
    constexpr int CH = 128;            // rows per chunk: 512 scales = one 128-bit load per lane
    constexpr int KB = CH / RKB;       // k-blocks per chunk (8)
    constexpr int AT = kRowsMfmaTile;  // bf16 elements of one A tile
    constexpr int NP = rows_mfma_parts(NREP); // bf16 parts of x*scale
    constexpr int NM = rows_mfma_sets(NREP);  // MFMAs per B operand
    constexpr int NPOS = 8;            // code positions per lane
    constexpr int FPB = 8 / FB;        // whole fields per byte window

    extern __shared__ float lds[];
    const int lane = threadIdx.x;
    const int wy = threadIdx.y;
    const int KW = blockDim.y;
    uint16_t *atile = reinterpret_cast<uint16_t *>(lds) + wy * (NM * AT);
    float *red = lds;  // [KW][NREP][128], reuses the A tiles after the streaming loop
    const int rs = lane / EPR;
    const int wi = lane % EPR;
    int64_t split, hg;
    xcd_swizzled_block(split, hg, a.heads_per_kv > NREP);
    const int64_t sample0 = hg * NREP;
    const int64_t m = blockIdx.z;
    const int64_t kv = sample0 / a.heads_per_kv;
    const int64_t kbeg = split * a.rows_per_split;
    const int64_t kend = kbeg + a.rows_per_split < a.K ? kbeg + a.rows_per_split : a.K;

    const uint16_t *xp = reinterpret_cast<const uint16_t *>(a.x) + sample0 * a.x_bs + m * a.x_rs;
    // dense 3-bit: a group is three aligned words; lane j of the group's four loads word
    // min(j, 2), and its 24 bits [24j, 24j+24) are cut out of two neighbours' words in compute()
    // (a dword load at byte 3j instead -- no exchange between lanes -- was measured slower: 33 against 28 us)
    const uint8_t *cp = reinterpret_cast<const uint8_t *>(a.code + kv * a.c_bs) +
                        (BITS == 30 ? (wi / 4) * 12 + (wi % 4 < 2 ? wi % 4 : 2) * 4 : wi * EB);
    [[maybe_unused]] const uint32_t sh3 = (uint32_t)(24 * (wi % 4)) % 32u;
    const uint16_t *sp = reinterpret_cast<const uint16_t *>(a.scale) + kv * a.s_bs;
    const uint16_t *zp = reinterpret_cast<const uint16_t *>(a.zero) + kv * a.s_bs;

    f32x4_t acc[NM][NPOS];
    float zacc[NREP][LPR];
#pragma unroll
    for (int q = 0; q < NM; q++) {
#pragma unroll
        for (int p = 0; p < NPOS; p++) acc[q][p] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int h = 0; h < NREP; h++) {
#pragma unroll
        for (int g = 0; g < LPR; g++) zacc[h][g] = 0.f;
    }
    // staging: this lane owns elements [8*lane, 8*lane+8) of the chunk's [128][4] scale array,
    // i.e. rows 2*lane and 2*lane+1, all four groups.  Row r of a chunk is k-slot (r%16)/4 of
    // A-lanes  (r%4)*16 + 4*g + i  in k-block r/16.
    // A tile: one 8-byte cell (4 k-slots) per (k-block t, lane); the 16 cells of the lanes with
    // the same (t, lane/16) form a row of 17 cells' pitch, and the rows of k-blocks 4..7 are
    // shifted by one more cell.  With that skew the 2-byte staging stores of a wave (same
    // cell column, 32 different rows) fall into 32 different LDS banks, and a wave's 8-byte
    // operand reads stay conflict-free.
    auto cell = [](int t, int l) { return ((4 * t + l / EPR) * 17 + (l % EPR)) * 4 + (t >> 2) * 4; };
    const int row0 = 2 * lane;
    int aoff[2];  // bf16 index of (row0 + e, g = 0, i = 0)
#pragma unroll
    for (int e = 0; e < 2; e++) {
        const int r = row0 + e;
        aoff[e] = cell(r / RKB, (r % RL) * EPR) + (r % RKB) / RL;
    }

    // Chunks: CH rows each, handed round-robin to the block's waves.  A chunk that would cross
    // the end of the range is moved back to end exactly there (the host gives this kernel only
    // K >= CH): every address is then base + constant with no clamping, no load sits behind
    // a condition (which would make the compiler drain the load queue), and the rows such a
    // chunk repeats meet x == 0.  A chunk wholly past the end is all zeros.
    // The wave index is made scalar so that the loop is uniform control flow.
    const int ke32 = (int)kend;
    if (a.K < CH) return;  // (never launched so: a chunk longer than K would leave the operand; the same for every thread)
    const int stride = KW * CH;
    const int kfirst = (int)kbeg + __builtin_amdgcn_readfirstlane(wy) * CH;
    struct __attribute__((packed, aligned(2))) Half2x {
        uint16_t v[2];
    };
    // DEPTH chunks are in flight per wave: register set d holds chunk c with c % DEPTH == d
    Half8 s8[DEPTH], z8[DEPTH];
    Half2x xh[DEPTH][NREP];
    Elem w[DEPTH][KB][4];

    auto chunk_base = [&](int k0) { return k0 + CH <= ke32 ? k0 : max(ke32 - CH, 0); };
    auto load_small = [&](int d, int k0) {
        const uint32_t kr = (uint32_t)(chunk_base(k0) + row0);
        s8[d] = ld_stream<Half8>(sp + kr * LPR);
        z8[d] = ld_stream<Half8>(zp + kr * LPR);
#pragma unroll
        for (int h = 0; h < NREP; h++) xh[d][h] = *reinterpret_cast<const Half2x *>(xp + h * a.x_bs + kr);
    };
    auto load_codes = [&](int d, int k0, int t) {
        const uint8_t *base = cp + (uint32_t)(chunk_base(k0) + rs) * (EPR * EB);
#pragma unroll
        for (int k = 0; k < 4; k++)
            w[d][t][k] = ld_stream<Elem>(base + (t * RKB + RL * k) * (EPR * EB));
    };
    auto stage = [&](int d, int k0) {
        const int skip = k0 - chunk_base(k0);  // rows of this chunk that an earlier one covered
#pragma unroll
        for (int h = 0; h < NREP; h++) {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int q = e / LPR, g = e % LPR;
                const float xv = row0 + q >= skip ? h16_to_f32(xh[d][h].v[q]) : 0.f;
                zacc[h][g] = fmaf(xv, h16_to_f32(z8[d].v[e]), zacc[h][g]);
                // x * scale * 2^90, split into bf16 parts by truncation (three parts: exact)
                uint32_t part[NP];
                split_bf16_parts<NP>((xv * 1237940039285380274899124224.0f) * h16_to_f32(s8[d].v[e]), part);
#pragma unroll
                for (int pt = 0; pt < NP; pt++) {  // A row NP*h+pt: MFMA (NP*h+pt)/4, lanes 4g + (NP*h+pt)%4
                    const int ar = NP * h + pt;
                    atile[(ar / 4) * AT + aoff[q] + g * 16 + (ar % 4) * 4] = (uint16_t)(part[pt] >> 16);
                }
            }
        }
    };
    auto compute = [&](int d, int t) {
        bf16x4_t av[NM];
#pragma unroll
        for (int q = 0; q < NM; q++)
            av[q] = *reinterpret_cast<const bf16x4_t *>(atile + q * AT + cell(t, lane));
        if constexpr (BITS == 30) {
            // the lane's 24 bits hold code i at bit 3i.  Codes 0,1 are bits 0..5 of byte 0 and codes 6,7 bits
            // 2..7 of byte 2; codes 2,3 and 4,5 are bits 2..7 of byte 0 and bits 0..5 of byte 1 of the stream
            // shifted right by 4: one shift per row, and a field at bit offset o simply counts 2^o-fold
            // (offsets by code: 0 3 2 5 0 3 2 5).
            uint32_t v[4], u[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                // words (0,0,1,2) and (0,1,2,2) of the group for lanes 0..3, funnel-shifted; the second set is what the
                // lanes loaded (lane j holds word min(j, 2)), only the first has to come from the neighbours
                const uint32_t lo = __builtin_amdgcn_mov_dpp(w[d][t][k], 0x90, 0xf, 0xf, false);
                const uint32_t hi = w[d][t][k];
                v[k] = __builtin_amdgcn_alignbit(hi, lo, sh3);
                u[k] = v[k] >> 4;
            }
#pragma unroll
            for (int mm = 0; mm < 4; mm++) {
                // byte of the source register that holds the pair: v bytes 0 / 2, u bytes 0 / 1
                const bool from_u = mm == 1 || mm == 2;
                const uint32_t b = from_u ? (uint32_t)(mm - 1) : (mm == 0 ? 0u : 2u);
                const uint32_t sel = 0x0c000c00u | b | ((4u + b) << 16);
                const uint32_t *src = from_u ? u : v;
                const uint32_t t01 = __builtin_amdgcn_perm(src[1], src[0], sel);
                const uint32_t t23 = __builtin_amdgcn_perm(src[3], src[2], sel);
                // bit offset of the pair's first field in its byte: 0 or 2; a pair at 0 is moved up by two (see
                // field_operand_top: its first field would have five leading zeros)
                constexpr bool UP = KVMIX_ROWS_FIELDS_TOP;
                const uint32_t s01 = UP && mm % 2 == 0 ? t01 << 2 : t01, s23 = UP && mm % 2 == 0 ? t23 << 2 : t23;
                const int o0 = UP || mm % 2 != 0 ? 2 : 0;
#pragma unroll
                for (int f = 0; f < 2; f++) {
                    const uint32_t mask = 0x00070007u << (o0 + 3 * f);
                    const bf16x4_t bv = __builtin_bit_cast(bf16x4_t, make_uint2(s01 & mask, s23 & mask));
#pragma unroll
                    for (int q = 0; q < NM; q++)
                        acc[q][mm * 2 + f] =
                            __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av[q], bv, acc[q][mm * 2 + f], 0, 0, 0);
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < EB; b++) {
                // byte b of rows k and k+1 -> low bytes of the two halves
                const uint32_t sel = 0x0c000c00u | (uint32_t)b | ((uint32_t)(4 + b) << 16);
                const uint32_t t01 = perm_elems(w[d][t][1], w[d][t][0], sel);
                const uint32_t t23 = perm_elems(w[d][t][3], w[d][t][2], sel);
#pragma unroll
                for (int f = 0; f < FPB; f++) {
                    const bf16x4_t bv = __builtin_bit_cast(
                        bf16x4_t, KVMIX_ROWS_FIELDS_TOP ? make_uint2(field_operand_top<FB>(t01, f), field_operand_top<FB>(t23, f))
                                                        : make_uint2(field_operand<FB>(t01, f), field_operand<FB>(t23, f)));
#pragma unroll
                    for (int q = 0; q < NM; q++)
                        acc[q][b * FPB + f] =
                            __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av[q], bv, acc[q][b * FPB + f], 0, 0, 0);
                }
            }
        }
    };

    if (kfirst < ke32) {
        // (the first loads are issued in the loop's own order, each pinned in place: the wait
        // counts at the loop head must hold for the entry path too)
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            load_small(d, kfirst + d * stride);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < KB; t++) {
                load_codes(d, kfirst + d * stride, t);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // some A rows are never written: clear the tiles once -- behind the first loads, whose
        // latency covers it (every wave of a launch starts at the same time)
        for (int i = lane; i < NM * AT / 2; i += kWave) reinterpret_cast<uint32_t *>(atile)[i] = 0u;
        wave_lds_fence();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
        for (int k0 = kfirst; k0 < ke32; k0 += DEPTH * stride) {
#pragma unroll
            for (int d = 0; d < DEPTH; d++) {
                const int kc = k0 + d * stride, kn = kc + DEPTH * stride;
                stage(d, kc);
                wave_lds_fence();
                load_small(d, kn);
                // a k-block's registers are refilled right after use.  The scheduling barriers
                // pin the loads where they are written: left alone, the scheduler sinks them to
                // the end of the iteration and the next one starts by draining the queue.
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < KB; t++) {
                    compute(d, t);
                    load_codes(d, kn, t);
                    __builtin_amdgcn_sched_barrier(0);
                }
                wave_lds_fence();  // the next chunk overwrites the tile
            }
        }
    }

    // ---- reduce ---------------------------------------------------------------------------
    // zero term: zacc[h][g] summed over all lanes; a lane needs the sum of its own group
    float zterm[NREP];
#pragma unroll
    for (int h = 0; h < NREP; h++) {
        float z[LPR];
#pragma unroll
        for (int g = 0; g < LPR; g++) z[g] = zacc[h][g];
        scatter_reduce<LPR, 8, 0>(z, lane);  // lane bits 3, 2 = group of the lane's codes
        z[0] += __shfl_xor(z[0], 1);
        z[0] += __shfl_xor(z[0], 2);
        z[0] += __shfl_xor(z[0], 16);
        z[0] += __shfl_xor(z[0], 32);
        zterm[h] = z[0];
    }
    // code sums: the three parts meet; the 2^-133 of the bf16 patterns, the 2^90 and the
    // field's bit offset are undone; then the 4 row slots (lane bits 4, 5) are summed
    constexpr int NV = NREP * NPOS;
    float flat[NV];
#pragma unroll
    for (int h = 0; h < NREP; h++) {
        float sums[NPOS];
#pragma unroll
        for (int p = 0; p < NPOS; p++)
            sums[p] = parts_sum<NP>(acc, h, p);
#pragma unroll
        for (int p = 0; p < NPOS; p++) {
            // (bit offset code p's field counts with: dense 3-bit 2 5 2 5 2 5 2 5 -- in its byte 0 3 2 5 0 3 2 5, the pairs at
            // 0 moved up by two --, else see field_offset_top)
            const int off = BITS == 30 ? 3 * (p % 2) + (KVMIX_ROWS_FIELDS_TOP ? 2 : 2 * ((p / 2) % 2)) : (KVMIX_ROWS_FIELDS_TOP ? field_offset_top<FB>(p % FPB) : FB * (p % FPB));
            const float sum = BITS == 30 ? sums[p]
                              : KVMIX_ROWS_FIELDS_TOP ? field_sum_top<FB>(sums[p], sums[p > 0 ? p - 1 : 0], p % FPB)
                                                      : field_sum(sums[p], sums[p > 0 ? p - 1 : 0], p % FPB);
            flat[h * NPOS + p] = sum * __uint_as_float((uint32_t)(127 + 43 - off) << 23);
        }
    }
    __syncthreads();  // every wave is done with its A tile: the space becomes `red`
    constexpr int KEEP = NV / 4;
    const int first = scatter_reduce<NV, 16, 1>(flat, lane);
#pragma unroll
    for (int i = 0; i < KEEP; i++) {
        const int f = first + i;
        const int h = f / NPOS;
        float zt = zterm[0];
#pragma unroll
        for (int hh = 1; hh < NREP; hh++) zt = h == hh ? zterm[hh] : zt;
        red[(wy * NREP + h) * 128 + wi * NPOS + f % NPOS] = flat[i] + zt;
    }
    __syncthreads();
    for (int t = wy * kWave + lane; t < NREP * 128; t += KW * kWave) {
        const int h = t / 128, n = t % 128;
        float v = 0.f;
        for (int ww = 0; ww < KW; ww++) v += red[(ww * NREP + h) * 128 + n];
        if (a.splits == 1)
            a.out[(sample0 + h) * a.o_bs + m * a.o_rs + n] = __float2half_rn(v);
        else
            a.partial[(((sample0 + h) * a.M + m) * a.splits + split) * a.N + n] = v;
    }
}

// ---------------------------------------------------------------------------------------
// gemv_cols_mfma<BITS, NREP>   q.K^T shape, 1/2/4-bit codes: the matrix-core scheme of
// gemv_rows_mfma turned by 90 degrees.
//   A lane owns 8 consecutive codes (BITS bytes) of N in every row; a wave's tile is 512
//   codes = 16 quantization groups, the four lanes of an MFMA block are one group.  One load
//   instruction reads 64*BITS contiguous bytes of one row; the k-slots of an MFMA are four
//   consecutive rows.  All K rows are reduced inside the lane's accumulators, so nothing is
//   exchanged between lanes or waves except the zero term, and a lane stores its 8 outputs
//   with one 16-byte store.
//   Rows are walked in chunks of 32 (8 MFMA k-steps): the chunk's [32][16] scales and zeros
//   are one 128-bit load per lane each; the lane that loads a scale forms x*scale*2^90, splits
//   it into three bf16 and parks them in the wave's LDS tile in A-operand order (rows of 32
//   eight-byte cells at a pitch of 33: staging stores and operand reads are bank-conflict
//   free).  A chunk that would cross K is moved back to end at K and its repeated rows meet
//   x == 0 (the host gives this kernel K >= 32).  Loads rotate as in gemv_rows_mfma.
//   The last tile of a row is shifted left to end at N (N >= 512, a multiple of 32).
//   A wave walks `splits` tiles one after the other with the load pipeline running across
//   them.  block = (64, 2..4) waves on neighbouring tiles; grid = (tiles/(waves*splits),
//   samples/NREP, M), XCD-swizzled; dynamic LDS = waves * (NM tiles of kColsMfmaTile bf16 +
//   NREP*16 floats).
// ---------------------------------------------------------------------------------------
constexpr int kColsMfmaTile = 16 * 33 * 4;  // bf16 elements: 16 rows of 33 four-element cells

template <int BITS, int NREP>
__global__ void __launch_bounds__(64 * kColsWaves)
    __attribute__((amdgpu_waves_per_eu(NREP > 1 ? kMfmaHeadsOcc : 4))) gemv_cols_mfma(GemvArgs a)
{
    using Elem = typename CodeElem<BITS>::type;
    constexpr int CH = 32;             // rows per chunk
    constexpr int KB = CH / 4;         // MFMA k-steps per chunk
    constexpr int AT = kColsMfmaTile;
    constexpr int NP = cols_mfma_parts(NREP);
    constexpr int NM = cols_mfma_sets(NREP);
    constexpr int NPOS = 8;
    constexpr int FPB = 8 / BITS;
    constexpr int TG = 16;             // groups per tile

    extern __shared__ float lds[];
    const int lane = threadIdx.x;
    const int wy = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int nw = (int)blockDim.y;
    uint16_t *atile = reinterpret_cast<uint16_t *>(lds) + wy * (NM * AT + NREP * TG * 2);
    float *zl = reinterpret_cast<float *>(atile + NM * AT);  // [NREP][16] zero terms of a tile
    int64_t bx, hg;
    xcd_swizzled_block(bx, hg, true);
    const int64_t sample0 = hg * NREP;
    const int64_t m = blockIdx.z;
    const int64_t kv = sample0 / a.heads_per_kv;
    const int K = (int)a.K;
    const int ngroups = (int)(a.N / 32);
    // a.splits tiles per wave: tiles (bx*splits + j)*nw + wy, j = 0..splits-1 -- the block's
    // waves sit on neighbouring tiles at any time.  A tile past N is redirected to the last
    // one (recomputed, stored twice with identical values): uniform control flow, no branches.
    const int tpw = a.splits;
    const int tile0 = (int)bx * tpw * nw + wy;
    if (ngroups < TG || K < CH) return;  // (never launched so: a tile wider than the row, a chunk longer than K)
    if (tile0 * TG >= ngroups) return;  // (no block barrier below)
    const int nch = (K + CH - 1) / CH;
    const int items = tpw * nch;        // (tile, chunk) pairs of this wave, in order

    const uint16_t *xp = reinterpret_cast<const uint16_t *>(a.x) + sample0 * a.x_bs + m * a.x_rs;
    const Elem *cbase = reinterpret_cast<const Elem *>(a.code + kv * a.c_bs) + lane;
    const uint32_t c_re = (uint32_t)a.c_rs * (4 / BITS);  // row stride in elements
    const uint32_t s_rs = (uint32_t)a.s_rs;
    const int par = lane % 2;   // staging: row lane/2 of the chunk, groups 8*par .. 8*par+7
    const int srow = lane / 2;
    const uint16_t *sbase = reinterpret_cast<const uint16_t *>(a.scale) + kv * a.s_bs + 8 * par;
    const uint16_t *zbase = reinterpret_cast<const uint16_t *>(a.zero) + kv * a.s_bs + 8 * par;

    f32x4_t acc[NM][NPOS];
    float zacc[NREP][8];
    auto clear = [&]() {
#pragma unroll
        for (int q = 0; q < NM; q++) {
#pragma unroll
            for (int p = 0; p < NPOS; p++) acc[q][p] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int h = 0; h < NREP; h++) {
#pragma unroll
            for (int j = 0; j < 8; j++) zacc[h][j] = 0.f;
        }
    };
    clear();

    // cell of (k-step t, operand lane l): four bf16 k-slots
    auto cell = [](int t, int l) { return ((2 * t + l / 32) * 33 + l % 32) * 4; };
    // staged row srow is k-slot srow%4 of k-step srow/4; its group 8*par+j feeds lanes 4*(8*par+j)+i
    const int aoff = cell(srow / 4, 32 * par) + srow % 4;

    Half8 s8, z8;
    uint16_t xh[NREP];
    Elem w[KB][4];

    // item -> first group of its tile, first row of its chunk (moved back to end at K)
    auto tile_g0 = [&](int it) {
        const int g = (tile0 + (it / nch) * nw) * TG;
        return g + TG <= ngroups ? g : max(ngroups - TG, 0);
    };
    auto chunk_k0 = [&](int it) { return (it % nch) * CH; };
    auto chunk_base = [&](int k0) { return k0 + CH <= K ? k0 : max(K - CH, 0); };
    auto load_small = [&](int it) {
        const uint32_t d = (uint32_t)(chunk_base(chunk_k0(it)) + srow);
        const uint32_t off = d * s_rs + (uint32_t)tile_g0(it);
        s8 = ld_stream<Half8, false>(sbase + off);
        z8 = ld_stream<Half8, false>(zbase + off);
#pragma unroll
        for (int h = 0; h < NREP; h++) xh[h] = xp[h * a.x_bs + d];
    };
    auto load_codes = [&](int it, int t) {
        const Elem *base = cbase + ((uint32_t)(chunk_base(chunk_k0(it)) + 4 * t) * c_re + (uint32_t)tile_g0(it) * 4);
#pragma unroll
        for (int k = 0; k < 4; k++) w[t][k] = ld_stream<Elem, (KVMIX_COLS_NT_CODES && BITS >= 2)>(base + (uint32_t)k * c_re);
    };
    auto stage = [&](int it) {
        const int k0 = chunk_k0(it);
        const int skip = k0 - chunk_base(k0);  // rows of this chunk that an earlier one covered
#pragma unroll
        for (int h = 0; h < NREP; h++) {
            const float xv = srow >= skip ? h16_to_f32(xh[h]) : 0.f;
            const float x2 = xv * 1237940039285380274899124224.0f;  // 2^90
#pragma unroll
            for (int j = 0; j < 8; j++) {
                zacc[h][j] = fmaf(xv, h16_to_f32(z8.v[j]), zacc[h][j]);
                uint32_t part[NP];
                split_bf16_parts<NP>(x2 * h16_to_f32(s8.v[j]), part);  // (three parts: exact)
#pragma unroll
                for (int pt = 0; pt < NP; pt++) {  // A row NP*h+pt: MFMA (NP*h+pt)/4, lanes 4g + (NP*h+pt)%4
                    const int ar = NP * h + pt;
                    atile[(ar / 4) * AT + aoff + (4 * j + ar % 4) * 4] = (uint16_t)(part[pt] >> 16);
                }
            }
        }
    };
    auto compute = [&](int t) {
        bf16x4_t av[NM];
#pragma unroll
        for (int q = 0; q < NM; q++) av[q] = *reinterpret_cast<const bf16x4_t *>(atile + q * AT + cell(t, lane));
#pragma unroll
        for (int b = 0; b < BITS; b++) {
            const uint32_t sel = 0x0c000c00u | (uint32_t)b | ((uint32_t)(4 + b) << 16);
            const uint32_t t01 = __builtin_amdgcn_perm((uint32_t)w[t][1], (uint32_t)w[t][0], sel);
            const uint32_t t23 = __builtin_amdgcn_perm((uint32_t)w[t][3], (uint32_t)w[t][2], sel);
#pragma unroll
            for (int f = 0; f < FPB; f++) {
                const bf16x4_t bv =
                    __builtin_bit_cast(bf16x4_t, make_uint2(field_operand<BITS>(t01, f), field_operand<BITS>(t23, f)));
#pragma unroll
                for (int q = 0; q < NM; q++)
                    acc[q][b * FPB + f] =
                        __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av[q], bv, acc[q][b * FPB + f], 0, 0, 0);
            }
        }
    };
    struct __attribute__((packed, aligned(2))) Out8 {
        uint16_t v[8];
    };
    // a tile's K rows are done: zero terms through LDS, 8 outputs per lane and head, clear
    auto finish_tile = [&](int it) {
#pragma unroll
        for (int h = 0; h < NREP; h++) {
            float z[8];
#pragma unroll
            for (int j = 0; j < 8; j++) z[j] = zacc[h][j];
            const int first = scatter_reduce<8, 2, 1>(z, lane);  // lane bits 1..3
            z[0] += __shfl_xor(z[0], 16);
            z[0] += __shfl_xor(z[0], 32);
            zl[h * TG + 8 * par + first] = z[0];  // group 8*par+first (same value from 4 lanes)
        }
        wave_lds_fence();
        const int64_t col = (int64_t)tile_g0(it) * 32 + lane * 8;
#pragma unroll
        for (int h = 0; h < NREP; h++) {
            const float zt = zl[h * TG + lane / 4];
            Out8 o;
            float sums[NPOS];
#pragma unroll
            for (int p = 0; p < NPOS; p++)
                sums[p] = parts_sum<NP>(acc, h, p);
#pragma unroll
            for (int p = 0; p < NPOS; p++) {
                const float sum = field_sum(sums[p], sums[p > 0 ? p - 1 : 0], p % FPB);
                o.v[p] = f32_to_h16(fmaf(sum, __uint_as_float((uint32_t)(127 + 43 - BITS * (p % FPB)) << 23), zt));
            }
            uint16_t *op = reinterpret_cast<uint16_t *>(a.out) + (sample0 + h) * a.o_bs + m * a.o_rs + col;
            *reinterpret_cast<Out8 *>(op) = o;
        }
        wave_lds_fence();
        clear();
    };

    load_small(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < KB; t++) {
        load_codes(0, t);
        __builtin_amdgcn_sched_barrier(0);
    }
    // some A rows are never written: clear the tile once -- behind the first loads, whose latency
    // covers it (every wave of a launch starts at the same time)
    for (int i = lane; i < NM * AT / 2; i += kWave) reinterpret_cast<uint32_t *>(atile)[i] = 0u;
    wave_lds_fence();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
    for (int it = 0; it < items; it++) {
        const int nx = it + 1 < items ? it + 1 : it;  // (past the end: the same item again)
        stage(it);
        wave_lds_fence();
        load_small(nx);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < KB; t++) {
            compute(t);
            load_codes(nx, t);
            __builtin_amdgcn_sched_barrier(0);
        }
        wave_lds_fence();  // the next chunk overwrites the tile
        if (it % nch == nch - 1) finish_tile(it);
    }
}

// ---------------------------------------------------------------------------------------
// gemv_cols_mfma2<BITS, NTC, WIDE>   q.K^T, 4-, 2- or 1-bit codes, one query head per kv head: gemv_cols_mfma
// with several 8-code elements per lane, so that a wave reads longer contiguous pieces of a row and the launch
// needs fewer waves (measured: both the length of the pieces and the number of waves bound this shape).
// A row piece is cut into `HALVES` sub-pieces of 64 lanes x one load each; a quad of lanes holds one (4 bits) or
// two (2 bits, 1 bit) quantization groups per sub-piece, and each group of the quad is one MFMA set:
//   4 bits: the lane's dword of a sub-piece is element `lane` of its 256 bytes; a quad then holds all four elements
//   of ONE group, the set works on every lane's own register and nothing moves between lanes.
//   2 bits, 1 bit: the lane's dword / ushort is elements 2l and 2l+1 of the sub-piece; lanes 0,1 of a quad hold the
//   four elements of one group, lanes 2,3 those of the next.  The set of the first group takes the second elements
//   of lanes 0,1 to lanes 2,3 with a DPP quad permute, the set of the second group mirrors it.
//   Plain: 4 bits two sub-pieces (512 bytes), 2 bits one (256 bytes), 1 bit one (128 bytes): tile = 1024 codes = 32
//   groups, two sets.  WIDE: twice the sub-pieces: tile = 2048 codes = 64 groups, four sets, half as many waves with
//   twice the bytes in flight each (two waves per SIMD instead of three).
//   Per set the scheme is gemv_cols_mfma's: k = 4 channel rows, three exact bf16 parts of x*scale*2^90
//   as A.  Rows are walked in chunks of 16 (4 k-steps); the chunk's [16][groups] scales and zeros are one
//   128-bit load per lane and 32 groups each (plain: 64-byte pieces per row; WIDE: 128-byte pieces, 8 rows per
//   load).  LDS tile: per (k-step, set) a row of 64 eight-byte cells in four sub-rows at a pitch of 17 cells, rows
//   at a pitch of 74.
//   Loads go through buffer descriptors (row offsets in SGPRs); NTC: codes with the non-temporal hint.
//   block = (64, 2..4) waves on neighbouring tiles, or `ksplit` waves on ONE tile, each with a share
//   of the K rows (small launches); grid = (tiles/waves, samples, M), XCD-swizzled.
// ---------------------------------------------------------------------------------------
constexpr int kColsMfma2Row = 74 * 4;                   // bf16 elements per (k-step, set) row
constexpr int kColsMfma2Tile = 8 * kColsMfma2Row;       // 4 k-steps x 2 sets (plain); WIDE: twice that
constexpr int cols_mfma2_sets(bool wide) { return wide ? 4 : 2; }
constexpr int cols_mfma2_groups(bool wide) { return 16 * cols_mfma2_sets(wide); }   // groups of 32 codes per tile
constexpr size_t cols_mfma2_lds(bool wide)  // bytes per wave: the A tile + the tile's zero terms
{
    return (size_t)4 * cols_mfma2_sets(wide) * kColsMfma2Row * sizeof(uint16_t) + cols_mfma2_groups(wide) * sizeof(float);
}

// NTC: the codes are loaded non-temporally (the host asks for it while the launch is no more than a few rounds of
// resident waves: measured faster up to 8k waves, slower at 16k, where rows of neighbouring tiles meet in the L2)
template <int BITS, bool NTC, bool WIDE>
__global__ void __launch_bounds__(64 * kColsWaves) __attribute__((amdgpu_waves_per_eu(kMfma2Occ)))
gemv_cols_mfma2(GemvArgs a)
{
    static_assert(BITS == 4 || BITS == 2 || BITS == 1, "per sub-piece a dword (4, 2 bits) or a ushort (1 bit) per lane");
    constexpr int CH = 16;             // rows per chunk
    constexpr int KB = CH / 4;         // MFMA k-steps per chunk
    constexpr int NPOS = 8;
    constexpr int FPB = 8 / BITS;
    constexpr bool SPLIT = BITS == 4;  // a quad holds ONE group per sub-piece (else two, exchanged by DPP)
    constexpr int SPH = SPLIT ? 1 : 2;                       // sets (groups of a quad) per sub-piece
    constexpr int HALVES = (SPLIT ? 2 : 1) * (WIDE ? 2 : 1); // sub-pieces per row piece = registers per lane and row
    constexpr int NS = HALVES * SPH;                         // MFMA sets
    constexpr int TG = 16 * NS;                              // groups per tile
    constexpr int HB = BITS == 1 ? 128 : 256;                // bytes of a sub-piece
    constexpr int AT = KB * NS * kColsMfma2Row;              // bf16 elements of the A tile
    constexpr int NSZ = TG / 32;                             // 128-bit scale (and zero) loads per lane and chunk
    constexpr int UPR = TG / 8;                              // staging units (8 groups) per row
    static_assert(NS == cols_mfma2_sets(WIDE) && TG == cols_mfma2_groups(WIDE), "host-side sizes");

    extern __shared__ float lds[];
    const int lane = threadIdx.x;
    const int wy = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int nw = (int)blockDim.y;
    uint16_t *atile = reinterpret_cast<uint16_t *>(lds) + wy * (AT + TG * 2);
    float *zl = reinterpret_cast<float *>(atile + AT);  // [TG] zero terms of a tile
    int64_t bx, sample;
    xcd_swizzled_block(bx, sample, true);
    const int64_t m = blockIdx.z;
    const int64_t kv = sample / a.heads_per_kv;
    const int K = (int)a.K;
    const int ngroups = (int)(a.N / 32);
    // ks > 1 (small problems): ks neighbouring waves share a tile and slice its K rows
    // chunk-wise, which shortens each wave's chain of dependent loads; their sums meet in LDS
    const int ks = a.ksplit;
    const int slice = wy % ks;
    const int ntw = nw / ks;            // tiles a block works on at a time
    const int tile0 = (int)bx * ntw + wy / ks;   // one tile per wave
    if (ngroups < TG || K < CH) return;  // (never launched so: a tile wider than the row, a chunk longer than K; the same for every thread)
    if (tile0 * TG >= ngroups) {
        if (ks > 1) __syncthreads();    // (the one block barrier of finish_tile)
        return;
    }
    const int nch_all = (K + CH - 1) / CH;
    const int nch_slice = (nch_all + ks - 1) / ks;
    const int ch0 = slice * nch_slice;  // this wave's chunks: [ch0, ch0 + nch)
    const int nch = ch0 >= nch_all ? 0 : (ch0 + nch_slice <= nch_all ? nch_slice : nch_all - ch0);
    const int items = nch;

    const uint16_t *xp = reinterpret_cast<const uint16_t *>(a.x) + sample * a.x_bs + m * a.x_rs;
    // buffer descriptors of this (batch, kv-head) slice
    const uint32_t sz_bytes = slice_bytes(K, a.s_rs, ngroups, 2);
    const __amdgpu_buffer_rsrc_t crsrc = stream_rsrc(a.code + kv * a.c_bs, slice_bytes(K, a.c_rs, (int64_t)ngroups * BITS, 4));
    const __amdgpu_buffer_rsrc_t srsrc = stream_rsrc(a.scale + kv * a.s_bs, sz_bytes);
    const __amdgpu_buffer_rsrc_t zrsrc = stream_rsrc(a.zero + kv * a.s_bs, sz_bytes);
    const uint32_t c_rs = (uint32_t)a.c_rs, s_rs = (uint32_t)a.s_rs;
    // staging: unit u = lane + 64 i (i < NSZ) is row u / UPR of the chunk, groups 8 * (u % UPR) .. + 7
    // (u % UPR = lane % UPR for every i: a lane stages the same eight groups in NSZ rows)
    const int sub = lane % UPR;
    const uint32_t c_lane = (uint32_t)lane * (BITS == 1 ? 2u : 4u);                       // bytes, inside a sub-piece
    const uint32_t s_lane = 2u * ((uint32_t)(lane / UPR) * s_rs + 8u * (uint32_t)sub);    // bytes, unit i = 0
    const uint32_t s_step = 2u * (uint32_t)(kWave / UPR) * s_rs;                          // ... from unit i to i + 1
    const int j4 = lane % 4;    // position in the quad

    f32x4_t acc[NS][NPOS];
    float zacc[8];
    auto clear = [&]() {
#pragma unroll
        for (int q = 0; q < NS; q++) {
#pragma unroll
            for (int p = 0; p < NPOS; p++) acc[q][p] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < 8; j++) zacc[j] = 0.f;
    };
    clear();

    // cell (four bf16 k-slots) of (k-step t, set s, operand lane l)
    auto cell = [](int t, int s, int l) { return (NS * t + s) * kColsMfma2Row + ((l / 16) * 17 + l % 16) * 4; };
    // Group g = 8 * sub + jj of the tile is sub-piece g / (16 SPH); 4 bits: quad g % 16 of set g / 16; else quad
    // (g % 32) / 2 of set 2 (g / 32) + g % 2.  Its three parts go to operand lanes 4 quad + part.  Staged row r is
    // k-slot r % 4 of k-step r / 4.  With `sub` folded into a per-lane base, the 24 stores of a unit are base + constant.
    int aoff[NSZ];
#pragma unroll
    for (int i = 0; i < NSZ; i++) {
        const int srow = (lane + kWave * i) / UPR;
        aoff[i] = (SPLIT ? cell(srow / 4, sub / 2, 32 * (sub % 2)) : cell(srow / 4, 2 * (sub / 4), 16 * (sub % 4))) + srow % 4;
    }

    Half8 s8[NSZ], z8[NSZ];
    uint16_t xh[NSZ];
    uint32_t w[KB][4][HALVES];

    // the last tile of a row is moved back to end at N
    const int g_first = tile0 * TG + TG <= ngroups ? tile0 * TG : max(ngroups - TG, 0);
    auto tile_g0 = [&](int) { return g_first; };
    auto chunk_k0 = [&](int it) { return (ch0 + it) * CH; };
    auto chunk_base = [&](int k0) { return k0 + CH <= K ? k0 : max(K - CH, 0); };
    auto load_small = [&](int it) {
        const uint32_t d0 = (uint32_t)chunk_base(chunk_k0(it));
        const uint32_t off = 2u * (d0 * s_rs + (uint32_t)tile_g0(it));  // bytes, the same for every lane
#pragma unroll
        for (int i = 0; i < NSZ; i++) {
            s8[i] = ld_buffer<Half8, false>(srsrc, s_lane + (uint32_t)i * s_step, off);
            z8[i] = ld_buffer<Half8, false>(zrsrc, s_lane + (uint32_t)i * s_step, off);
            xh[i] = xp[d0 + (uint32_t)((lane + kWave * i) / UPR)];
        }
    };
    auto load_codes = [&](int it, int t) {
        // (a group of 32 codes is BITS words)
        const uint32_t base = 4u * ((uint32_t)(chunk_base(chunk_k0(it)) + 4 * t) * c_rs + (uint32_t)tile_g0(it) * BITS);
#pragma unroll
        for (int k = 0; k < 4; k++) {
#pragma unroll
            for (int h = 0; h < HALVES; h++) {
                if constexpr (BITS == 1)
                    w[t][k][h] = ld_buffer<uint16_t, (KVMIX_COLS_NT_CODES && NTC)>(crsrc, c_lane + (uint32_t)(h * HB), base + 4u * (uint32_t)k * c_rs);
                else
                    w[t][k][h] = ld_buffer<uint32_t, (KVMIX_COLS_NT_CODES && NTC)>(crsrc, c_lane + (uint32_t)(h * HB), base + 4u * (uint32_t)k * c_rs);
            }
        }
    };
    auto stage = [&](int it) {
        const int k0 = chunk_k0(it);
        const int skip = k0 - chunk_base(k0);  // rows of this chunk that an earlier one covered
#pragma unroll
        for (int i = 0; i < NSZ; i++) {
            const int srow = (lane + kWave * i) / UPR;
            const float xv = srow >= skip ? h16_to_f32(xh[i]) : 0.f;
            const float x2 = xv * 1237940039285380274899124224.0f;  // 2^90
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                zacc[jj] = fmaf(xv, h16_to_f32(z8[i].v[jj]), zacc[jj]);
                const float v0 = x2 * h16_to_f32(s8[i].v[jj]);  // split into three bf16 by truncation (exact)
                const uint32_t b0 = __float_as_uint(v0) & 0xffff0000u;
                const float v1 = v0 - __uint_as_float(b0);
                const uint32_t b1 = __float_as_uint(v1) & 0xffff0000u;
                const float v2 = v1 - __uint_as_float(b1);
                const uint32_t part[3] = {b0, b1, __float_as_uint(v2)};
#pragma unroll
                for (int pt = 0; pt < 3; pt++) {
                    if constexpr (SPLIT)  // operand lane 32 * (sub % 2) + 4 * jj + pt of set sub / 2
                        atile[aoff[i] + (((4 * jj + pt) / 16) * 17 + (4 * jj + pt) % 16) * 4] = (uint16_t)(part[pt] >> 16);
                    else                  // operand lane 16 * (sub % 4) + 4 * (jj / 2) + pt of set 2 * (sub / 4) + jj % 2
                        atile[aoff[i] + (jj % 2) * kColsMfma2Row + (4 * (jj / 2) + pt) * 4] = (uint16_t)(part[pt] >> 16);
                }
            }
        }
    };
    auto compute = [&](int t) {
        bf16x4_t av[NS];
#pragma unroll
        for (int s = 0; s < NS; s++) av[s] = *reinterpret_cast<const bf16x4_t *>(atile + cell(t, s, lane));
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const int h = s / SPH, s2 = s % SPH;  // sub-piece; which of the quad's groups in it
            // first group of the quad (s2 == 0): lanes 0,1 hold its elements 0,2 (their first) and lanes 2,3
            // take elements 1,3 (the second of lanes 0,1); the second group mirrors it for lanes 2,3
            uint32_t src[4];
            uint32_t hi = 0;  // 2 bits / 1 bit: byte offset (0 or 2 / 0 or 1) of the element inside the register
#pragma unroll
            for (int k = 0; k < 4; k++) {
                if constexpr (SPLIT) {
                    src[k] = w[t][k][h];
                } else {
                    src[k] = s2 == 0 ? __builtin_amdgcn_mov_dpp(w[t][k][h], 0x44, 0xf, 0xf, false)
                                     : __builtin_amdgcn_mov_dpp(w[t][k][h], 0xEE, 0xf, 0xf, false);
                }
            }
            if constexpr (BITS != 4) hi = (s2 == 0 ? j4 >= 2 : j4 < 2) ? (uint32_t)BITS : 0u;  // byte offset of the element
#pragma unroll
            for (int b = 0; b < BITS; b++) {
                const uint32_t sel = (0x0c000c00u | (uint32_t)b | ((uint32_t)(4 + b) << 16)) + hi * 0x00010001u;
                const uint32_t t01 = __builtin_amdgcn_perm(src[1], src[0], sel);
                const uint32_t t23 = __builtin_amdgcn_perm(src[3], src[2], sel);
#pragma unroll
                for (int f = 0; f < FPB; f++) {
                    const bf16x4_t bv =
                        __builtin_bit_cast(bf16x4_t, make_uint2(field_operand<BITS>(t01, f), field_operand<BITS>(t23, f)));
                    acc[s][b * FPB + f] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av[s], bv, acc[s][b * FPB + f], 0, 0, 0);
                }
            }
        }
    };
    struct __attribute__((packed, aligned(2))) Out8 {
        uint16_t v[8];
    };
    auto finish_tile = [&](int it) {
        // zero terms: zacc[jj] summed over the lanes with the same `sub`; group 8*sub+jj -> LDS
        float z[8];
#pragma unroll
        for (int jj = 0; jj < 8; jj++) z[jj] = zacc[jj];
        int first;
        if constexpr (UPR == 4) {
            first = scatter_reduce<8, 4, 1>(z, lane);  // lane bits 2..4
            z[0] += __shfl_xor(z[0], 32);
        } else {
            first = scatter_reduce<8, 8, 1>(z, lane);  // lane bits 3..5
        }
        zl[8 * sub + first] = z[0];
        float sum[NS][NPOS];
#pragma unroll
        for (int s = 0; s < NS; s++) {
#pragma unroll
            for (int p = 0; p < NPOS; p++) sum[s][p] = (acc[s][p][0] + acc[s][p][1]) + acc[s][p][2];
        }
        wave_lds_fence();
        if (ks > 1) {
            // slices 1.. park their sums in their own (now idle) A tile; slice 0 adds them up
            float *mine = reinterpret_cast<float *>(atile);
            if (slice > 0) {
#pragma unroll
                for (int s = 0; s < NS; s++) {
#pragma unroll
                    for (int p = 0; p < NPOS; p++) mine[(s * NPOS + p) * kWave + lane] = sum[s][p];
                }
            }
            __syncthreads();
            if (slice == 0) {
                for (int o = 1; o < ks; o++) {
                    const uint16_t *other_tile = atile + o * (AT + TG * 2);
                    const float *other = reinterpret_cast<const float *>(other_tile);
                    const float *ozl = reinterpret_cast<const float *>(other_tile + AT);
#pragma unroll
                    for (int s = 0; s < NS; s++) {
#pragma unroll
                        for (int p = 0; p < NPOS; p++) sum[s][p] += other[(s * NPOS + p) * kWave + lane];
                    }
                    if (lane < TG) zl[lane] += ozl[lane];
                }
                wave_lds_fence();
            }
        }
        if (slice == 0) {
            const int q = lane / 4;
            uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) + sample * a.o_bs + m * a.o_rs + (int64_t)tile_g0(it) * 32;
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const int h = s / SPH, s2 = s % SPH;
                // group of the tile / element (8 codes) of the tile that this lane's accumulators of set s belong to
                const float zt = SPLIT ? zl[16 * h + q] : zl[32 * h + 2 * q + s2];
                const int elem = SPLIT ? 64 * h + lane
                                       : 128 * h + 8 * q + (s2 == 0 ? ((j4 & 1) * 2 + (j4 >> 1)) : (4 + (j4 & 1) * 2 + (1 - (j4 >> 1))));
                Out8 o;
#pragma unroll
                for (int p = 0; p < NPOS; p++) {
                    const float v = field_sum(sum[s][p], sum[s][p > 0 ? p - 1 : 0], p % FPB);
                    o.v[p] = f32_to_h16(fmaf(v, __uint_as_float((uint32_t)(127 + 43 - BITS * (p % FPB)) << 23), zt));
                }
                *reinterpret_cast<Out8 *>(orow + elem * 8) = o;
            }
        }
        wave_lds_fence();
        clear();
    };

    if (nch == 0) {  // (a slice beyond the last chunk: only its zeros take part)
        finish_tile(0);
        return;
    }
    load_small(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < KB; t++) {
        load_codes(0, t);
        __builtin_amdgcn_sched_barrier(0);
    }
    // some A rows are never written: clear the tile once -- behind the first loads, whose latency
    // covers it (every wave of a launch starts at the same time)
    for (int i = lane; i < AT / 2; i += kWave) reinterpret_cast<uint32_t *>(atile)[i] = 0u;
    wave_lds_fence();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
    for (int it = 0; it < items; it++) {
        const int nx = it + 1 < items ? it + 1 : it;  // (past the end: the same item again)
        // The waves of a block read neighbouring pieces of the same rows: a barrier per chunk keeps them in step, so
        // that their requests for one row arrive together (measured at B = 16, T = 8k: 4 bits 63.0 -> 59.8 us,
        // 2 bits 38.7 -> 36.3).  Waves without a tile have left and do not count; sliced tiles (ks > 1) walk
        // different numbers of chunks and are left alone.
        if (ks == 1) __builtin_amdgcn_s_barrier();
        stage(it);
        wave_lds_fence();
        load_small(nx);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < KB; t++) {
            compute(t);
            load_codes(nx, t);
            __builtin_amdgcn_sched_barrier(0);
        }
        wave_lds_fence();  // the next chunk overwrites the tile
    }
    finish_tile(items - 1);
}

// The value phase of a matrix-core slab: out[128] += sum over the slab's NCH * 128 positions [t_first, ...) of
// p[position] * value[position][:], as gemv_rows_mfma does it (chunks of 128 rows, p * scale * 2^90 in three bf16
// parts as the A operand), with p taken from the wave's LDS row `pbuf` (position order, fp32) instead of an fp16
// vector in memory.  (m, l) of the slab and its 128 unnormalised outputs go to the workspace as slab `tile` of the
// row.  `atile`: the wave's A tile (kRowsMfmaTile bf16).
template <int VMODE, int NCH>
__device__ __forceinline__ void slab_value_phase(const AttnSlabArgs &a, int64_t kv, int64_t sample, int tile, int t_first,
                                                 uint16_t *atile, const float *pbuf, float slab_m, float slab_l)
{
    constexpr int NPOS = 8;
    constexpr int BITS = VMODE;
    using Elem = typename CodeElem<BITS>::type;
    constexpr int EB = BITS == 30 ? 3 : BITS, FB = BITS == 30 ? 3 : BITS;
    constexpr int LPR = 4, EPR = 16, RL = kWave / EPR, RKB = 4 * RL, CH = 128, KB = CH / RKB, FPB = 8 / FB;
    const int lane = threadIdx.x;
    const int rs = lane / EPR, wi = lane % EPR;
    const int t_end = t_first + NCH * 128;
    const uint8_t *cp = reinterpret_cast<const uint8_t *>(a.v_code + kv * a.vc_bs) +
                        (BITS == 30 ? (wi / 4) * 12 + (wi % 4 < 2 ? wi % 4 : 2) * 4 : wi * EB);
    [[maybe_unused]] const uint32_t sh3 = (uint32_t)(24 * (wi % 4)) % 32u;
    const uint16_t *sp = a.v_scale + kv * a.vsz_bs;
    const uint16_t *zp = a.v_zero + kv * a.vsz_bs;

    f32x4_t acc[NPOS];
    float zacc[LPR];
#pragma unroll
    for (int p = 0; p < NPOS; p++) acc[p] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < LPR; g++) zacc[g] = 0.f;
    auto cell = [](int t, int l) { return ((4 * t + l / EPR) * 17 + (l % EPR)) * 4 + (t >> 2) * 4; };
    const int row0 = 2 * lane;
    int aoff[2];
#pragma unroll
    for (int e = 0; e < 2; e++) {
        const int r = row0 + e;
        aoff[e] = cell(r / RKB, (r % RL) * EPR) + (r % RKB) / RL;
    }
    Half8 s8, z8;
    Elem w[KB][4];
    // (a chunk past the slab's end -- the prefetch of the last step -- is the last chunk again)
    auto chunk_base = [&](int k0) { return k0 + CH <= t_end ? k0 : max(t_end - CH, 0); };
    auto load_small = [&](int k0) {
        const uint32_t kr = (uint32_t)(chunk_base(k0) + row0);
        s8 = ld_stream<Half8>(sp + kr * LPR);
        z8 = ld_stream<Half8>(zp + kr * LPR);
    };
    auto load_codes = [&](int k0, int t) {
        const uint8_t *base = cp + (uint32_t)(chunk_base(k0) + rs) * (EPR * EB);
#pragma unroll
        for (int k = 0; k < 4; k++) w[t][k] = ld_stream<Elem>(base + (t * RKB + RL * k) * (EPR * EB));
    };
    auto stage = [&](int k0) {
        const float2 pv = *reinterpret_cast<const float2 *>(pbuf + (k0 - t_first) + row0);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int q = e / LPR, g = e % LPR;
            const float xv = q == 0 ? pv.x : pv.y;
            zacc[g] = fmaf(xv, h16_to_f32(z8.v[e]), zacc[g]);
            // p * scale * 2^90 in three bf16 parts by truncation (24 of the product's bits)
            const float v0 = (xv * 1237940039285380274899124224.0f) * h16_to_f32(s8.v[e]);
            const uint32_t b0 = __float_as_uint(v0) & 0xffff0000u;
            const float v1 = v0 - __uint_as_float(b0);
            const uint32_t b1 = __float_as_uint(v1) & 0xffff0000u;
            const float v2 = v1 - __uint_as_float(b1);
            const uint32_t part[3] = {b0, b1, __float_as_uint(v2)};
#pragma unroll
            for (int pt = 0; pt < 3; pt++) atile[aoff[q] + g * 16 + pt * 4] = (uint16_t)(part[pt] >> 16);
        }
    };
    auto compute = [&](int t) {
        const bf16x4_t av = *reinterpret_cast<const bf16x4_t *>(atile + cell(t, lane));
        if constexpr (BITS == 30) {
            uint32_t v[4], u[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t lo = __builtin_amdgcn_mov_dpp(w[t][k], 0x90, 0xf, 0xf, false);
                const uint32_t hi = w[t][k];  // (lane j holds word min(j, 2) of its group: the set (0,1,2,2))
                v[k] = __builtin_amdgcn_alignbit(hi, lo, sh3);
                u[k] = v[k] >> 4;
            }
#pragma unroll
            for (int mm = 0; mm < 4; mm++) {
                const bool from_u = mm == 1 || mm == 2;
                const uint32_t b = from_u ? (uint32_t)(mm - 1) : (mm == 0 ? 0u : 2u);
                const uint32_t sel = 0x0c000c00u | b | ((4u + b) << 16);
                const uint32_t *src = from_u ? u : v;
                const uint32_t t01 = __builtin_amdgcn_perm(src[1], src[0], sel);
                const uint32_t t23 = __builtin_amdgcn_perm(src[3], src[2], sel);
                constexpr bool UP = KVMIX_ROWS_FIELDS_TOP;  // (a pair at bit 0 is moved up by two, as in gemv_rows_mfma)
                const uint32_t s01 = UP && mm % 2 == 0 ? t01 << 2 : t01, s23 = UP && mm % 2 == 0 ? t23 << 2 : t23;
                const int o0 = UP || mm % 2 != 0 ? 2 : 0;
#pragma unroll
                for (int f = 0; f < 2; f++) {
                    const uint32_t mask = 0x00070007u << (o0 + 3 * f);
                    const bf16x4_t bv = __builtin_bit_cast(bf16x4_t, make_uint2(s01 & mask, s23 & mask));
                    acc[mm * 2 + f] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av, bv, acc[mm * 2 + f], 0, 0, 0);
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < EB; b++) {
                const uint32_t sel = 0x0c000c00u | (uint32_t)b | ((uint32_t)(4 + b) << 16);
                const uint32_t t01 = perm_elems(w[t][1], w[t][0], sel);
                const uint32_t t23 = perm_elems(w[t][3], w[t][2], sel);
#pragma unroll
                for (int f = 0; f < FPB; f++) {
                    const bf16x4_t bv = __builtin_bit_cast(
                        bf16x4_t, KVMIX_ROWS_FIELDS_TOP ? make_uint2(field_operand_top<FB>(t01, f), field_operand_top<FB>(t23, f))
                                                        : make_uint2(field_operand<FB>(t01, f), field_operand<FB>(t23, f)));
                    acc[b * FPB + f] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av, bv, acc[b * FPB + f], 0, 0, 0);
                }
            }
        }
    };

    load_small(t_first);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < KB; t++) {
        load_codes(t_first, t);
        __builtin_amdgcn_sched_barrier(0);
    }
    for (int i = lane; i < kRowsMfmaTile / 2; i += kWave) reinterpret_cast<uint32_t *>(atile)[i] = 0u;
    wave_lds_fence();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
    for (int k0 = t_first; k0 < t_end; k0 += CH) {
        stage(k0);
        wave_lds_fence();
        load_small(k0 + CH);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < KB; t++) {
            compute(t);
            load_codes(k0 + CH, t);
            __builtin_amdgcn_sched_barrier(0);
        }
        wave_lds_fence();
    }

    // zero term of the lane's group; code sums; the four row slots (lane bits 4, 5) meet
    float z[LPR];
#pragma unroll
    for (int g = 0; g < LPR; g++) z[g] = zacc[g];
    scatter_reduce<LPR, 8, 0>(z, lane);
    z[0] += __shfl_xor(z[0], 1);
    z[0] += __shfl_xor(z[0], 2);
    z[0] += __shfl_xor(z[0], 16);
    z[0] += __shfl_xor(z[0], 32);
    float sums[NPOS], flat[NPOS];
#pragma unroll
    for (int p = 0; p < NPOS; p++) sums[p] = (acc[p][0] + acc[p][1]) + acc[p][2];
#pragma unroll
    for (int p = 0; p < NPOS; p++) {
        const int off = BITS == 30 ? 3 * (p % 2) + (KVMIX_ROWS_FIELDS_TOP ? 2 : 2 * ((p / 2) % 2)) : (KVMIX_ROWS_FIELDS_TOP ? field_offset_top<FB>(p % FPB) : FB * (p % FPB));
        const float sum = BITS == 30 ? sums[p]
                          : KVMIX_ROWS_FIELDS_TOP ? field_sum_top<FB>(sums[p], sums[p > 0 ? p - 1 : 0], p % FPB)
                                                  : field_sum(sums[p], sums[p > 0 ? p - 1 : 0], p % FPB);
        flat[p] = sum * __uint_as_float((uint32_t)(127 + 43 - off) << 23);
    }
    const int first = scatter_reduce<NPOS, 16, 1>(flat, lane);  // two of the lane's eight columns are left
    float *wo = a.ws_o + ((int64_t)sample * a.slabs + tile) * 128 + wi * NPOS + first;
    wo[0] = flat[0] + z[0];
    wo[1] = flat[1] + z[0];
    if (lane == 0) {
        float *ml = a.ws_ml + ((int64_t)sample * a.slabs + tile) * 2;
        ml[0] = slab_m;
        ml[1] = slab_l;
    }
}

// ---------------------------------------------------------------------------------------
// attn_slab_mfma_body<KBITS, VMODE, COOP>   a tile of the single-pass decode step (attn_step_mfma below) over the
// quantized positions, on the matrix cores: 1024 positions of one query head (D = 128).
//   1. logits of the tile: the q.K^T tile of gemv_cols_mfma2, the sums kept in registers; each is rounded to fp16,
//      scaled by 1/sqrt(D) and masked as the reference does it.
//   2. slab maximum m, p = exp(logit - m) (fp32), their sum l; p goes to the wave's LDS row in position order.
//   3. p.V over the same positions, as gemv_rows_mfma does it (128-row chunks), with p taken from LDS instead of an
//      fp16 vector in memory.
//   (m, l) and the 128 unnormalised outputs go to the workspace as a slab of the row; the vector-ALU slabs over the
//   remaining positions (trailing blocks of the same launch) are further slabs and attn_fused_merge combines all.
//   The last tile of a row is moved back to end at `tokens`; the positions it shares with its neighbour get p = 0.
//   COOP = false: one wave per tile (slab = tile), block = (64, 4) waves on neighbouring tiles, no block barrier: a
//   wave without a tile simply leaves.  COOP = true: the block's four waves share ONE tile: wave w takes channel
//   rows [32 w, 32 w + 32) in step 1, the partial sums of all 1024 positions meet in LDS (two block barriers),
//   then wave w runs steps 2 and 3 on positions [256 w, 256 w + 256) as a slab of its own (four slabs per tile).
//   Dynamic LDS = 4 * kSlabLds bytes either way.
// ---------------------------------------------------------------------------------------
constexpr int kSlabKeyBytes = (kColsMfma2Tile * 2 + 32 * 4 + 15) / 16 * 16;  // A tile of the key phase + 32 zero terms
constexpr int kSlabLds = kSlabKeyBytes + 1024 * 4;                            // ... + the slab's probabilities
static_assert(kRowsMfmaTile * 2 <= kSlabKeyBytes, "the value phase's A tile reuses the key phase's space");

template <int KBITS, int VMODE, bool COOP>
__device__ __forceinline__ void attn_slab_mfma_body(const AttnSlabArgs &a, int64_t bx, int64_t sample, float *lds)
{
    static_assert(KBITS == 4 || KBITS == 2 || KBITS == 1, "key codes of 1, 2 or 4 bits");
    constexpr bool NTC = KBITS >= 2;  // (as gemv_cols_mfma2: a 1-bit row piece shares its lines with the neighbours')
    constexpr int NPOS = 8;
    constexpr int TG = 32;            // groups per tile

    const int lane = threadIdx.x;
    const int wy = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int nw = (int)blockDim.y;
    uint8_t *mine = reinterpret_cast<uint8_t *>(lds) + wy * kSlabLds;
    uint16_t *atile = reinterpret_cast<uint16_t *>(mine);
    float *pbuf = reinterpret_cast<float *>(mine + kSlabKeyBytes);  // [1024] probabilities of the slab
    const int64_t kv = sample / a.heads_per_kv;
    const int ngroups = (int)(a.tokens / 32);
    const int tile = COOP ? (int)bx : (int)bx * nw + wy;
    if (ngroups < TG) return;  // (never launched so: a slab longer than the row would leave the operands)
    if (tile * TG >= ngroups) return;  // (COOP: the whole block)
    const int g_first = tile * TG + TG <= ngroups ? tile * TG : max(ngroups - TG, 0);  // (the last tile ends at `tokens`)
    const int shift = tile * TG - g_first;                                     // its first groups are the neighbour's
    float slab_m, slab_l;

    // ---- 1. logits: gemv_cols_mfma2's tile ---------------------------------------------------------------
    {
        constexpr int BITS = KBITS;
        constexpr int CH = 16, KB = CH / 4, AT = kColsMfma2Tile, FPB = 8 / BITS, K = 128;
        constexpr int WL = BITS == 4 ? 2 : 1;
        constexpr bool SPLIT = BITS == 4;
        float *zl = reinterpret_cast<float *>(atile + AT);
        const uint16_t *xp = a.q + sample * a.q_bs;
        const uint32_t sz_bytes = slice_bytes(K, a.ksz_rs, ngroups, 2);
        const __amdgpu_buffer_rsrc_t crsrc = stream_rsrc(a.k_code + kv * a.kc_bs, slice_bytes(K, a.kc_rs, (int64_t)ngroups * BITS, 4));
        const __amdgpu_buffer_rsrc_t srsrc = stream_rsrc(a.k_scale + kv * a.ksz_bs, sz_bytes);
        const __amdgpu_buffer_rsrc_t zrsrc = stream_rsrc(a.k_zero + kv * a.ksz_bs, sz_bytes);
        const uint32_t c_rs = (uint32_t)a.kc_rs, s_rs = (uint32_t)a.ksz_rs;
        const int sub = lane % 4, srow = lane / 4, j4 = lane % 4;
        const uint32_t c_lane = SPLIT ? (uint32_t)lane * 4u : (uint32_t)lane * (2 * BITS);
        const uint32_t s_lane = 2u * ((uint32_t)srow * s_rs + 8u * (uint32_t)sub);

        f32x4_t acc[2][NPOS];
        float zacc[8];
#pragma unroll
        for (int q = 0; q < 2; q++) {
#pragma unroll
            for (int p = 0; p < NPOS; p++) acc[q][p] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < 8; j++) zacc[j] = 0.f;
        auto cell = [](int t, int s, int l) { return (2 * t + s) * kColsMfma2Row + ((l / 16) * 17 + l % 16) * 4; };
        const int aoff = SPLIT ? cell(srow / 4, sub / 2, 32 * (sub % 2)) + srow % 4 : cell(srow / 4, 0, 16 * sub) + srow % 4;

        Half8 s8, z8;
        uint16_t xh;
        uint32_t w[KB][4][WL];
        auto load_small = [&](int it) {
            const uint32_t d0 = (uint32_t)(it * CH);
            const uint32_t off = 2u * (d0 * s_rs + (uint32_t)g_first);
            s8 = ld_buffer<Half8, false>(srsrc, s_lane, off);
            z8 = ld_buffer<Half8, false>(zrsrc, s_lane, off);
            xh = xp[d0 + (uint32_t)srow];
        };
        auto load_codes = [&](int it, int t) {
            const uint32_t base = 4u * ((uint32_t)(it * CH + 4 * t) * c_rs + (uint32_t)g_first * BITS);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                if constexpr (BITS == 1) {
                    w[t][k][0] = ld_buffer<uint16_t, (KVMIX_COLS_NT_CODES && NTC)>(crsrc, c_lane, base + 4u * (uint32_t)k * c_rs);
                } else if constexpr (SPLIT) {
                    w[t][k][0] = ld_buffer<uint32_t, (KVMIX_COLS_NT_CODES && NTC)>(crsrc, c_lane, base + 4u * (uint32_t)k * c_rs);
                    w[t][k][1] = ld_buffer<uint32_t, (KVMIX_COLS_NT_CODES && NTC)>(crsrc, c_lane + 256u, base + 4u * (uint32_t)k * c_rs);
                } else {
                    w[t][k][0] = ld_buffer<uint32_t, (KVMIX_COLS_NT_CODES && NTC)>(crsrc, c_lane, base + 4u * (uint32_t)k * c_rs);
                }
            }
        };
        auto stage = [&]() {
            const float xv = h16_to_f32(xh);
            const float x2 = xv * 1237940039285380274899124224.0f;  // 2^90
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                zacc[jj] = fmaf(xv, h16_to_f32(z8.v[jj]), zacc[jj]);
                const float v0 = x2 * h16_to_f32(s8.v[jj]);  // split into three bf16 by truncation (exact)
                const uint32_t b0 = __float_as_uint(v0) & 0xffff0000u;
                const float v1 = v0 - __uint_as_float(b0);
                const uint32_t b1 = __float_as_uint(v1) & 0xffff0000u;
                const float v2 = v1 - __uint_as_float(b1);
                const uint32_t part[3] = {b0, b1, __float_as_uint(v2)};
#pragma unroll
                for (int pt = 0; pt < 3; pt++) {
                    if constexpr (SPLIT)
                        atile[aoff + (((4 * jj + pt) / 16) * 17 + (4 * jj + pt) % 16) * 4] = (uint16_t)(part[pt] >> 16);
                    else
                        atile[aoff + (jj % 2) * kColsMfma2Row + (4 * (jj / 2) + pt) * 4] = (uint16_t)(part[pt] >> 16);
                }
            }
        };
        auto compute = [&](int t) {
            const bf16x4_t av0 = *reinterpret_cast<const bf16x4_t *>(atile + cell(t, 0, lane));
            const bf16x4_t av1 = *reinterpret_cast<const bf16x4_t *>(atile + cell(t, 1, lane));
#pragma unroll
            for (int s = 0; s < 2; s++) {
                uint32_t src[4];
                uint32_t hi = 0;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    if constexpr (SPLIT) {
                        src[k] = w[t][k][s];
                    } else {
                        src[k] = s == 0 ? __builtin_amdgcn_mov_dpp(w[t][k][0], 0x44, 0xf, 0xf, false)
                                        : __builtin_amdgcn_mov_dpp(w[t][k][0], 0xEE, 0xf, 0xf, false);
                    }
                }
                if constexpr (BITS != 4) hi = (s == 0 ? j4 >= 2 : j4 < 2) ? (uint32_t)BITS : 0u;
#pragma unroll
                for (int b = 0; b < BITS; b++) {
                    const uint32_t sel = (0x0c000c00u | (uint32_t)b | ((uint32_t)(4 + b) << 16)) + hi * 0x00010001u;
                    const uint32_t t01 = __builtin_amdgcn_perm(src[1], src[0], sel);
                    const uint32_t t23 = __builtin_amdgcn_perm(src[3], src[2], sel);
#pragma unroll
                    for (int f = 0; f < FPB; f++) {
                        const bf16x4_t bv =
                            __builtin_bit_cast(bf16x4_t, make_uint2(field_operand<BITS>(t01, f), field_operand<BITS>(t23, f)));
                        acc[s][b * FPB + f] =
                            __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(s == 0 ? av0 : av1, bv, acc[s][b * FPB + f], 0, 0, 0);
                    }
                }
            }
        };

        constexpr int items = K / CH;
        // COOP: the block's four waves share the tile, each with a quarter of the 128 channel rows
        const int it0 = COOP ? wy * (items / kColsWaves) : 0, it1 = COOP ? it0 + items / kColsWaves : items;
        load_small(it0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < KB; t++) {
            load_codes(it0, t);
            __builtin_amdgcn_sched_barrier(0);
        }
        for (int i = lane; i < AT / 2; i += kWave) reinterpret_cast<uint32_t *>(atile)[i] = 0u;
        wave_lds_fence();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
        for (int it = it0; it < it1; it++) {
            const int nx = it + 1 < it1 ? it + 1 : it;
            // (as in gemv_cols_mfma2: the block's waves, on neighbouring tiles of the same rows, kept in step)
            if constexpr (!COOP && KVMIX_SLAB_BARRIER) __builtin_amdgcn_s_barrier();
            stage();
            wave_lds_fence();
            load_small(nx);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < KB; t++) {
                compute(t);
                load_codes(nx, t);
                __builtin_amdgcn_sched_barrier(0);
            }
            wave_lds_fence();
        }

        // zero terms of the 32 groups, then the logits of this lane's 16 positions
        {
            float z[8];
#pragma unroll
            for (int jj = 0; jj < 8; jj++) z[jj] = zacc[jj];
            const int first = scatter_reduce<8, 4, 1>(z, lane);
            z[0] += __shfl_xor(z[0], 32);
            zl[8 * sub + first] = z[0];
        }
        wave_lds_fence();
        const int q = lane / 4;
        const float *mrow = a.mask ? a.mask + (sample / a.heads) * a.mask_bs : nullptr;
        if constexpr (COOP) {
            // every wave has the sums of its rows for all 1024 positions: they meet in LDS (the waves' pbuf areas,
            // in position order), then wave w finishes positions [256 w, 256 w + 256) as a slab of its own
#pragma unroll
            for (int s = 0; s < 2; s++) {
                const int elem = SPLIT ? 64 * s + lane
                                       : 8 * q + (s == 0 ? ((j4 & 1) * 2 + (j4 >> 1)) : (4 + (j4 & 1) * 2 + (1 - (j4 >> 1))));
                float sums[NPOS], part[NPOS];
#pragma unroll
                for (int p = 0; p < NPOS; p++) sums[p] = (acc[s][p][0] + acc[s][p][1]) + acc[s][p][2];
#pragma unroll
                for (int p = 0; p < NPOS; p++) {
                    const float v = field_sum(sums[p], sums[p > 0 ? p - 1 : 0], p % FPB);
                    part[p] = v * __uint_as_float((uint32_t)(127 + 43 - BITS * (p % FPB)) << 23);
                }
                *reinterpret_cast<float4 *>(pbuf + elem * 8) = float4{part[0], part[1], part[2], part[3]};
                *reinterpret_cast<float4 *>(pbuf + elem * 8 + 4) = float4{part[4], part[5], part[6], part[7]};
            }
            __syncthreads();
            const uint8_t *base = reinterpret_cast<const uint8_t *>(lds);
            const int pos0 = 256 * wy + 4 * lane, grp = pos0 / 32;
            float4 d = float4{0.f, 0.f, 0.f, 0.f};
            float zt = 0.f;
#pragma unroll
            for (int w = 0; w < kColsWaves; w++) {
                const float4 v = *reinterpret_cast<const float4 *>(base + w * kSlabLds + kSlabKeyBytes + 4 * pos0);
                d.x += v.x, d.y += v.y, d.z += v.z, d.w += v.w;
                zt += reinterpret_cast<const float *>(base + w * kSlabLds + AT * 2)[grp];
            }
            __syncthreads();  // (the waves' areas are read; from here on pbuf is the wave's own 256 probabilities)
            const float dots[4] = {d.x + zt, d.y + zt, d.z + zt, d.w + zt};
            float xs[4];
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float lg = h16_to_f32(f32_to_h16(dots[j])) * a.inv_sqrt_d;
                if (mrow) lg = fmaxf(lg + mrow[(int64_t)g_first * 32 + pos0 + j], -3.4028234663852886e38f);
                xs[j] = grp >= shift ? lg : -INFINITY;
                mx = fmaxf(mx, xs[j]);
            }
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            float sum = 0.f, e[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                e[j] = xs[j] == -INFINITY ? 0.f : expf(xs[j] - mx);
                sum += e[j];
            }
            *reinterpret_cast<float4 *>(pbuf + 4 * lane) = float4{e[0], e[1], e[2], e[3]};
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
            wave_lds_fence();
            slab_value_phase<VMODE, 2>(a, kv, sample, tile * kColsWaves + wy, g_first * 32 + 256 * wy, atile, pbuf, mx, sum);
            return;
        }
        float x[2][NPOS];
        float mx = -INFINITY;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const int grp = SPLIT ? 16 * s + q : 2 * q + s;  // group of the tile these eight positions are in
            const int elem = SPLIT ? 64 * s + lane
                                   : 8 * q + (s == 0 ? ((j4 & 1) * 2 + (j4 >> 1)) : (4 + (j4 & 1) * 2 + (1 - (j4 >> 1))));
            const float zt = zl[grp];
            float sums[NPOS];
#pragma unroll
            for (int p = 0; p < NPOS; p++) sums[p] = (acc[s][p][0] + acc[s][p][1]) + acc[s][p][2];
#pragma unroll
            for (int p = 0; p < NPOS; p++) {
                const float v = field_sum(sums[p], sums[p > 0 ? p - 1 : 0], p % FPB);
                const float dot = fmaf(v, __uint_as_float((uint32_t)(127 + 43 - BITS * (p % FPB)) << 23), zt);
                float lg = h16_to_f32(f32_to_h16(dot)) * a.inv_sqrt_d;  // fp16 logit -> scaled, masked fp32 value
                if (mrow) lg = fmaxf(lg + mrow[(int64_t)g_first * 32 + elem * 8 + p], -3.4028234663852886e38f);
                x[s][p] = grp >= shift ? lg : -INFINITY;
                mx = fmaxf(mx, x[s][p]);
            }
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        float sum = 0.f;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const int elem = SPLIT ? 64 * s + lane
                                   : 8 * q + (s == 0 ? ((j4 & 1) * 2 + (j4 >> 1)) : (4 + (j4 & 1) * 2 + (1 - (j4 >> 1))));
#pragma unroll
            for (int p = 0; p < NPOS; p++) {
                const float e = x[s][p] == -INFINITY ? 0.f : expf(x[s][p] - mx);
                sum += e;
                pbuf[elem * 8 + p] = e;
            }
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
        slab_m = mx;
        slab_l = sum;
        wave_lds_fence();
    }

    // ---- 2. p.V over the slab's 1024 positions ------------------------------------------------------------
    slab_value_phase<VMODE, 8>(a, kv, sample, tile, g_first * 32, atile, pbuf, slab_m, slab_l);
}

// ---------------------------------------------------------------------------------------
// attn_slab_ref3_body<VMODE>   the same slab for keys in the reference's 3-bit words (11 codes and an own scale and
// zero per word): one wave = 128 words = 1408 positions of one query head (4 * lcm(11, 32): whole words of the keys
// and whole 128-row chunks of the values).
//   1. logits as gemv_cols3 computes them, one head per pass and no K slicing: a lane owns two words of every
//      channel row (8 + 4 + 4 bytes per row straight to registers, eight rows in flight), codes multiplied in as
//      fp32 bit patterns; the query, times 2^90, sits in the wave's LDS.
//   2. 3. as above, the value phase over eleven chunks.
//   `tokens` is a multiple of 352 here; the last tile is moved back to end there.
// ---------------------------------------------------------------------------------------
constexpr int kSlabRef3Words = 128;                       // words per tile and channel row
constexpr int kSlabRef3Tile = kSlabRef3Words * 11;        // positions per tile
constexpr int kSlabRef3ABytes = (kRowsMfmaTile * 2 + 15) / 16 * 16;
constexpr int kSlabRef3Lds = 128 * 4 + kSlabRef3ABytes + kSlabRef3Tile * 4;   // query, A tile of the value phase, probabilities

template <int VMODE, bool COOP>
__device__ __forceinline__ void attn_slab_ref3_body(const AttnSlabArgs &a, int64_t bx, int64_t sample, float *lds)
{
    constexpr int K = 128, U = 8, UPL = 2, VALS = 11, TW = kSlabRef3Words;
    const int lane = threadIdx.x;
    const int wy = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int nw = (int)blockDim.y;
    uint8_t *mine = reinterpret_cast<uint8_t *>(lds) + wy * kSlabRef3Lds;
    float *xs = reinterpret_cast<float *>(mine);                                  // [128] query * 2^90
    uint16_t *atile = reinterpret_cast<uint16_t *>(mine + K * 4);
    float *pbuf = reinterpret_cast<float *>(mine + K * 4 + kSlabRef3ABytes);      // [1408] probabilities of the slab
    const int64_t kv = sample / a.heads_per_kv;
    const int nwords = (int)(a.tokens / VALS);
    const int tile = COOP ? (int)bx : (int)bx * nw + wy;
    if (nwords < TW) return;  // (never launched so: a slab longer than the row would leave the operands)
    if (tile * TW >= nwords) return;  // (COOP: the whole block)
    const int w_first = tile * TW + TW <= nwords ? tile * TW : max(nwords - TW, 0);  // (the last tile ends at `tokens`)
    const int shift = tile * TW - w_first;                                             // its first words are the neighbour's
    float slab_m, slab_l;
    {
        const uint16_t *qp = a.q + sample * a.q_bs;
        for (int i = lane; i < K; i += kWave) xs[i] = h16_to_f32(qp[i]) * 1237940039285380274899124224.0f;  // 2^90
        wave_lds_fence();

        float acc[UPL][VALS], zsum[UPL];
#pragma unroll
        for (int j = 0; j < UPL; j++) {
            zsum[j] = 0.f;
#pragma unroll
            for (int i = 0; i < VALS; i++) acc[j][i] = 0.f;
        }
        struct __attribute__((packed, aligned(2))) Half2x {
            uint16_t v[UPL];
        };
        Words<UPL> cw[U];
        Half2x sw[U], zw[U];
        // uniform bases and 32-bit byte offsets per lane, one running offset per array (gemv_cols3's walk)
        const uint8_t *cb = reinterpret_cast<const uint8_t *>(a.k_code + kv * a.kc_bs);
        const uint8_t *sb = reinterpret_cast<const uint8_t *>(a.k_scale + kv * a.ksz_bs);
        const uint8_t *zb = reinterpret_cast<const uint8_t *>(a.k_zero + kv * a.ksz_bs);
        const uint32_t unit0 = (uint32_t)(w_first + lane * UPL);
        const uint32_t c_step = (uint32_t)a.kc_rs * 4u, s_step = (uint32_t)a.ksz_rs * 2u;
        // COOP: the block's four waves share the tile, each with a quarter of the 128 channel rows
        constexpr int steps = COOP ? K / U / kColsWaves : K / U;
        const int row0 = COOP ? wy * (K / kColsWaves) : 0;
        uint32_t co = unit0 * 4u + (uint32_t)row0 * c_step, so = unit0 * 2u + (uint32_t)row0 * s_step;
        auto next_row = [&](int u) {
            cw[u] = ld_stream<Words<UPL>, KVMIX_SLAB3_NT_CODES>(cb + co);
            sw[u] = ld_stream<Half2x, KVMIX_SLAB3_NT_SZ>(sb + so);
            zw[u] = ld_stream<Half2x, KVMIX_SLAB3_NT_SZ>(zb + so);
            co += c_step;
            so += s_step;
        };
        float xr[U];
        auto compute_row = [&](int u) {
            const float xv = xr[u];
#pragma unroll
            for (int j = 0; j < UPL; j++) {
                const half2_t sz = __builtin_bit_cast(half2_t, (uint32_t)sw[u].v[j] | ((uint32_t)zw[u].v[j] << 16));
                // (a masked field of the word is code * 2^(offset - 149) as an fp32 pattern: see gemv_cols3)
                const uint32_t w = cw[u].v[j], hi = w >> 24;
                float f[VALS];
#pragma unroll
                for (int i = 0; i < 8; i++) f[i] = __uint_as_float(w & (7u << (3 * i)));
                f[8] = __uint_as_float(hi & 0x07u);
                f[9] = __uint_as_float(hi & 0x38u);
                f[10] = __uint_as_float(hi & 0xC0u);
                zsum[j] = fmaf(xv, (float)sz.y, zsum[j]);
                const float mq = fmaf(xv, (float)sz.x, 0.f);
#pragma unroll
                for (int i = 0; i < VALS; i++) acc[j][i] = fmaf(mq, f[i], acc[j][i]);
            }
        };
#pragma unroll
        for (int u = 0; u < U; u++) {
            next_row(u);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll 1
        for (int st = 0; st < steps - 1; st++) {
#pragma unroll
            for (int u = 0; u < U; u++) xr[u] = xs[row0 + st * U + u];
            __builtin_amdgcn_sched_barrier(0);
            // the block's waves -- neighbouring tiles of the same rows -- stay in step: a row piece does not end on a
            // cache line, and the line two tiles share is then fetched from memory once (measured, 2-bit values, us:
            // B = 8 72.2 -> 68.6, B = 16 141.2 -> 134.2).  A wave whose tile lies past the row has left: the barrier
            // counts the waves that remain
            if constexpr (!COOP && KVMIX_SLAB3_BARRIER) __builtin_amdgcn_s_barrier();
#pragma unroll
            for (int u = 0; u < U; u++) {
                compute_row(u);
                next_row(u);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) xr[u] = xs[row0 + (steps - 1) * U + u];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; u++) compute_row(u);

        // the logits of this lane's 22 positions: fp16 rounding, 1/sqrt(D), mask as in the reference
        const float *mrow = a.mask ? a.mask + (sample / a.heads) * a.mask_bs + (int64_t)w_first * VALS : nullptr;
        if constexpr (COOP) {
            // the waves' sums over their rows meet in LDS (the waves' pbuf areas, in position order); then wave w
            // finishes three of the tile's eleven 128-position chunks as a slab of its own: chunks 3 w .. 3 w + 2,
            // the last wave chunks 8 .. 10 with chunk 8 (wave 2's) at probability 0
#pragma unroll
            for (int j = 0; j < UPL; j++) {
#pragma unroll
                for (int i = 0; i < VALS; i++)
                    pbuf[(lane * UPL + j) * VALS + i] = fmaf(acc[j][i], cols3_out_scale(i), zsum[j] * kCols3ZeroDown);
            }
            __syncthreads();
            constexpr int CHW = 3, SPAN = CHW * 128, PER = SPAN / kWave;  // positions per wave, per lane
            const int begin = wy < kColsWaves - 1 ? SPAN * wy : kSlabRef3Tile - SPAN;  // first position of the wave's chunks
            const int own = SPAN * wy;                                                  // ... of the positions it owns
            const uint8_t *base = reinterpret_cast<const uint8_t *>(lds) + K * 4 + kSlabRef3ABytes;
            float xv[PER];
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < PER; r++) {
                const int pos = begin + r * kWave + lane;
                float dot = 0.f;
#pragma unroll
                for (int w = 0; w < kColsWaves; w++) dot += reinterpret_cast<const float *>(base + w * kSlabRef3Lds)[pos];
                float lg = h16_to_f32(f32_to_h16(dot)) * a.inv_sqrt_d;
                if (mrow) lg = fmaxf(lg + mrow[pos], -3.4028234663852886e38f);
                xv[r] = pos >= own && pos / VALS >= shift ? lg : -INFINITY;
                mx = fmaxf(mx, xv[r]);
            }
            __syncthreads();  // (the waves' areas are read; from here on pbuf is the wave's own 384 probabilities)
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            float sum = 0.f;
#pragma unroll
            for (int r = 0; r < PER; r++) {
                const float e = xv[r] == -INFINITY ? 0.f : expf(xv[r] - mx);
                sum += e;
                pbuf[r * kWave + lane] = e;
            }
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
            wave_lds_fence();
            slab_value_phase<VMODE, CHW>(a, kv, sample, tile * kColsWaves + wy, w_first * VALS + begin, atile, pbuf, mx, sum);
            return;
        }
        float x[UPL][VALS];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < UPL; j++) {
            const int wj = lane * UPL + j;  // word of the tile
#pragma unroll
            for (int i = 0; i < VALS; i++) {
                const float dot = fmaf(acc[j][i], cols3_out_scale(i), zsum[j] * kCols3ZeroDown);
                float lg = h16_to_f32(f32_to_h16(dot)) * a.inv_sqrt_d;
                if (mrow) lg = fmaxf(lg + mrow[wj * VALS + i], -3.4028234663852886e38f);
                x[j][i] = wj >= shift ? lg : -INFINITY;
                mx = fmaxf(mx, x[j][i]);
            }
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < UPL; j++) {
#pragma unroll
            for (int i = 0; i < VALS; i++) {
                const float e = x[j][i] == -INFINITY ? 0.f : expf(x[j][i] - mx);
                sum += e;
                pbuf[(lane * UPL + j) * VALS + i] = e;
            }
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
        slab_m = mx;
        slab_l = sum;
        wave_lds_fence();
    }
    slab_value_phase<VMODE, kSlabRef3Tile / 128>(a, kv, sample, tile, w_first * VALS, atile, pbuf, slab_m, slab_l);
}

// The launch of a large single-pass step: blocks [0, mfma_blocks) are the matrix-core tiles above (mfma_nx blocks per
// query head, XCD-swizzled), the rest are slabs of the vector-ALU kind (fused_slab.h, 8 lanes per key row = 256
// threads) over the positions the tiles do not cover: the fp16 tails, and quantized positions where keys and values
// are quantized to different lengths.  One launch instead of two; attn_fused_merge follows.
// KBITS: 1, 2, 4, or 3 = the reference's 3-bit words (tiles of 1408 positions).  block = (64, 4); dynamic LDS = step_lds(KBITS).
constexpr size_t step_lds(int k_mode)
{
    const size_t tiles = (size_t)kColsWaves * (k_mode == 3 ? kSlabRef3Lds : kSlabLds);
    const size_t slab = fused::SlabCfg<8>::lds_floats(1) * sizeof(float);
    return tiles > slab ? tiles : slab;
}
template <int KBITS, int VMODE, bool COOP>
__global__ void __launch_bounds__(64 * kColsWaves) __attribute__((amdgpu_waves_per_eu(kMfma2Occ)))
attn_step_mfma(AttnSlabArgs m, fused::FusedArgs f, unsigned mfma_blocks, unsigned mfma_nx)
{
    extern __shared__ float lds[];
    if (blockIdx.x < mfma_blocks) {
        // consecutive logical blocks on one XCD (xcd_swizzled_block, for a part of a one-dimensional grid; the XCD
        // of a block is its index in the whole launch modulo 8, and the tiles come first)
        const int64_t n = mfma_blocks, l = blockIdx.x;
        const int64_t xcd = l % kXcds, slot = l / kXcds, per = n / kXcds, rem = n % kXcds;
        const int64_t j = xcd * per + (xcd < rem ? xcd : rem) + slot;
        if constexpr (KBITS == 3)
            attn_slab_ref3_body<VMODE, COOP>(m, j % mfma_nx, j / mfma_nx, lds);
        else
            attn_slab_mfma_body<KBITS, VMODE, COOP>(m, j % mfma_nx, j / mfma_nx, lds);
    } else {
        fused::attn_fused_slab_body<1, 8>(f, (int64_t)blockIdx.x - mfma_blocks, (int64_t)gridDim.x - mfma_blocks,
                                          (int)(threadIdx.y * kWave + threadIdx.x), lds);
    }
}

__global__ void __launch_bounds__(256) reduce_splits(GemvArgs a)
{
    const int64_t sample = blockIdx.y;
    const int64_t m = blockIdx.z;
    const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= a.N) return;
    const float *p = a.partial + (sample * a.M + m) * a.splits * a.N + n;
    float v = 0.f;
    for (int s = 0; s < a.splits; s++) v += p[(int64_t)s * a.N];
    a.out[sample * a.o_bs + m * a.o_rs + n] = __float2half_rn(v);
}

// ---------------------------------------------------------------------------------------
// gemv_generic: one thread per packed unit (one word; three words for the dense stream),
// serial over K, the group of a unit is the group of its first code
// (dequantization_gemv_cuda.cu:23-24).
// ---------------------------------------------------------------------------------------
template <int MODE>
struct GenericCfg {
    static constexpr int VALS = MODE == 30 ? 32 : (MODE == 3 ? 11 : 32 / MODE);
    static constexpr int THREADS = VALS == 32 ? 256 : 512;  // (THREADS * (VALS + 1) floats of LDS stay under 64 KB)
};

// A block covers UB = 2^ub_log2 units; when that is fewer than the block has threads, the
// remaining factor KS = THREADS / UB slices K: thread (unit, slice) walks rows slice, slice + KS, ...
// and the slices are summed through LDS.  Short rows (few quantized tokens) would otherwise leave
// a handful of threads per output row walking all of K one after the other.
template <int MODE>
__global__ void __launch_bounds__(GenericCfg<MODE>::THREADS) gemv_generic(GemvArgs a, int ub_log2)
{
    constexpr int BITS = MODE == 30 ? 3 : MODE;
    constexpr int VALS = GenericCfg<MODE>::VALS;
    constexpr int THREADS = GenericCfg<MODE>::THREADS;
    constexpr int WORDS = MODE == 30 ? 3 : 1;
    extern __shared__ float red[];  // [THREADS][VALS + 1] when K is sliced
    const int tid = threadIdx.x;
    const int UB = 1 << ub_log2, KS = THREADS >> ub_log2;
    const int ul = tid & (UB - 1), slice = tid >> ub_log2;
    const int64_t u = (int64_t)blockIdx.x * UB + ul;
    const int64_t units = a.N / VALS;
    const bool live = u < units;
    const int64_t sample = blockIdx.y;
    const int64_t m = blockIdx.z;
    const int64_t kv = sample / a.heads_per_kv;
    const int64_t grp = (u * VALS) / a.group;
    const __half *xp = a.x + sample * a.x_bs + m * a.x_rs;
    const uint32_t *cp = a.code + kv * a.c_bs + u * WORDS;
    const __half *sp = a.scale + kv * a.s_bs + grp;
    const __half *zp = a.zero + kv * a.s_bs + grp;
    float acc[VALS];
#pragma unroll
    for (int i = 0; i < VALS; i++) acc[i] = 0.f;
    float zsum = 0.f;
    if (live) {
#pragma unroll 4
        for (int64_t k = slice; k < a.K; k += KS) {
            uint32_t w[WORDS];
#pragma unroll
            for (int t = 0; t < WORDS; t++) w[t] = cp[k * a.c_rs + t];
            const float xv = __half2float(xp[k]);
            const float qs = xv * __half2float(sp[k * a.s_rs]);
            zsum = fmaf(xv, __half2float(zp[k * a.s_rs]), zsum);
            if constexpr (MODE == 30) {
                accumulate_unit<30>(w, qs, acc);
            } else if constexpr (MODE == 3) {
                accumulate_unit<3>(w, qs, acc);
            } else {
#pragma unroll
                for (int i = 0; i < VALS; i++)
                    acc[i] = fmaf(qs, (float)((w[0] >> (i * BITS)) & ((1u << BITS) - 1u)), acc[i]);
            }
        }
    }
    __half *orow = a.out + sample * a.o_bs + m * a.o_rs;
    if (KS == 1) {  // (the same for every thread of the grid)
        if (live) {
#pragma unroll
            for (int i = 0; i < VALS; i++) orow[u * VALS + i] = __float2half_rn(fmaf(acc[i], Fmt<MODE>::OUT_SCALE, zsum));
        }
        return;
    }
    float *mine = red + tid * (VALS + 1);
#pragma unroll
    for (int i = 0; i < VALS; i++) mine[i] = acc[i];
    mine[VALS] = zsum;
    __syncthreads();
    for (int o = tid; o < UB * VALS; o += THREADS) {
        const int ul2 = o / VALS, i = o % VALS;
        const int64_t u2 = (int64_t)blockIdx.x * UB + ul2;
        if (u2 >= units) continue;
        float sum = 0.f, z = 0.f;
        for (int sl = 0; sl < KS; sl++) {
            const float *r = red + (sl * UB + ul2) * (VALS + 1);
            sum += r[i];
            z += r[VALS];
        }
        orow[u2 * VALS + i] = __float2half_rn(fmaf(sum, Fmt<MODE>::OUT_SCALE, z));
    }
}

// --------------------------- host side ---------------------------

// kvmix_quantized_gemv_plan: the dispatch below runs as usual, but every launch is recorded instead of made
static thread_local kvmix_gemv_plan_t *t_plan = nullptr;

static void plan_record(const dim3 &grid, const dim3 &block, size_t lds, const char *fmt, ...)
{
    kvmix_gemv_plan_t *p = t_plan;
    if (p->launches++ > 0) return;  // (a second launch is the split-K reduction: counted, not described)
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(p->kernel, sizeof(p->kernel), fmt, ap);
    va_end(ap);
    p->grid[0] = grid.x, p->grid[1] = grid.y, p->grid[2] = grid.z;
    p->block[0] = block.x, p->block[1] = block.y, p->block[2] = block.z;
    p->lds_bytes = lds;
}

// launch `kernel(args)` -- or, while a plan is being recorded, note its name (a printf format and its
// arguments: the template parameters) and geometry
#define KVMIX_LAUNCH(kernel, grid, block, lds, st, args, ...)              \
    do {                                                                   \
        if (t_plan)                                                        \
            plan_record(grid, block, lds, __VA_ARGS__);                    \
        else                                                               \
            hipLaunchKernelGGL(kernel, grid, block, lds, st, args);       \
    } while (0)

// Every tiled kernel moves the last tile of a row back so that it ends at N: a tile wider than the row would
// start before the row.  The dispatch never picks such a kernel; each launcher checks it all the same, launches
// nothing when the tile does not fit, and the entry point then reports the shape -- so that a change of the
// dispatch rules cannot turn into an access outside the operands.
static thread_local int t_refused = KVMIX_OK;
static bool tile_fits(int64_t units, int64_t tile_units)
{
    if (units >= tile_units) return true;
    t_refused = KVMIX_ERR_SHAPE;
    return false;
}

static bool rows_shape_ok(int64_t N) { return N == 64 || N == 128 || N == 256; }

struct RowsPlan {
    int waves;   // waves per block
    int splits;  // blocks along K
    int64_t rows_per_split;
};

// How gemv_rows covers K for `batch_rows` = samples*M independent outputs.
// (blocks of at most four waves are the multi-head kernels, which hold two waves per SIMD:
// they get half as many waves, again one resident round)
static RowsPlan plan_rows(int64_t batch_rows, int64_t K, int64_t N, int max_waves)
{
    const int64_t target = max_waves <= kRowsHeadsWaves ? kTargetWaves / kHeadsWaveDiv : kTargetWaves;
    RowsPlan p{4, 1, K > 0 ? K : 1};
    if (!rows_shape_ok(N) || batch_rows <= 0 || K <= 0) return p;
    const int64_t chunk = 512 / (N / 32);            // rows one wave takes per step
    const int64_t chunks = (K + chunk - 1) / chunk;  // units of parallelism along K
    int64_t want = (target + batch_rows - 1) / batch_rows;  // waves wanted per output row
    if (want > chunks) want = chunks;
    // a wave's start-up and the reduction at its end are paid per wave: with fewer than about eight
    // chunks per wave, fewer and longer-lived waves are faster (measured at B = 8, T = 8k: 16 -> 8
    // waves per row, 2-bit p.V 22.2 -> 20.3 us), as long as two waves per SIMD remain
    {
        const int64_t by_chunks = (chunks + kRowsChunksPerWave - 1) / kRowsChunksPerWave;
        const int64_t by_waves = (target / 2 + batch_rows - 1) / batch_rows;
        const int64_t lean = by_chunks > by_waves ? by_chunks : by_waves;
        if (lean < want) want = lean;
    }
    if (want < 1) want = 1;
    // blocks of 5, 6 or 7 waves are slower than blocks of 4 or 8 (four SIMDs per CU, and a launch a little larger
    // than the resident waves).  Measured at T = 8k, 2 / 4 bits, us: 28 x 32 rows, 5 -> 4 waves: 76.1 -> 59.7 / 104.5 ->
    // 90.8; 24 x 32 rows, 6 -> 4: 53.2 -> 49.0 / 79.6 -> 75.6; 20 x 32 rows, 7 -> 4: 49.1 -> 46.7 / 69.0 -> 66.6; 12 x 32
    // rows, 6 waves 38.1 / 45.6 against 8 waves 33.6 / 43.2.  Up to the next multiple of four while all waves of the
    // launch stay resident (four per SIMD), else down
    if (want > 4 && want < max_waves && want % 4 != 0) {
        const int64_t up = (want + 3) / 4 * 4;
        want = batch_rows * up <= target ? up : want / 4 * 4;
    }
#ifdef KVMIX_EXPERIMENT
    if (const char *e = getenv("KVMIX_DBG_ROWS_WAVES")) want = atoll(e);
#endif
    int64_t waves = want < max_waves ? want : max_waves;
    if (waves < 4) waves = 4;  // the block epilogue wants 128+ threads; idle waves are cheap
    int64_t splits = (want + waves - 1) / waves;
    // a second block per output row brings the reduce_splits launch with it: not worth it while
    // one block's waves get at most kRowsSingleBlockChunks chunks each
    if (splits > 1 && chunks <= waves * kRowsSingleBlockChunks) splits = 1;
    if (splits > 64) splits = 64;
    int64_t rps = (K + splits - 1) / splits;
    rps = (rps + chunk - 1) / chunk * chunk;
    splits = (K + rps - 1) / rps;
    p.waves = (int)waves;
    p.splits = (int)(splits < 1 ? 1 : splits);
    p.rows_per_split = rps;
    return p;
}

// query heads one block of gemv_rows / gemv_cols serves from a single pass over the packed data
static int heads_per_block(int heads_per_kv) { return heads_per_kv % 4 == 0 ? 4 : 1; }

// which p.V kernel a problem gets, and the most waves one of its blocks may have
// (gemv_rows_mfma: N = 128, dense code rows, at least one whole 128-row chunk)
static bool rows_use_mfma(int mode, int64_t N, int64_t K, int64_t c_rs)
{
    return (mode == 1 || mode == 2 || mode == 4 || mode == 30) && N == 128 && K >= 128 &&
           c_rs == N * (mode == 30 ? 3 : mode) / 32;
}
static int rows_max_waves(bool mfma, int nrep)
{
    return nrep > 1 ? kRowsHeadsWaves : (mfma ? kRowsMfmaWaves : kRowsMaxWaves);
}

template <int MODE, int NREP>
static void launch_rows_n(GemvArgs &a, int64_t samples, hipStream_t st)
{
    // (a block's LDS is waves * NREP * (512 + N) floats)
    const bool mfma = rows_use_mfma(MODE, a.N, a.K, a.c_rs);
    const RowsPlan p = plan_rows(samples / NREP * a.M, a.K, a.N, rows_max_waves(mfma, NREP));
    a.splits = p.splits;
    a.rows_per_split = p.rows_per_split;
    const dim3 grid((unsigned)a.splits, (unsigned)(samples / NREP), (unsigned)a.M), block(kWave, p.waves);
    if (mfma) {
        if (!tile_fits(a.K, 128)) return;  // (a chunk past the end is moved back to end at K)
        // one A tile per wave and MFMA set; the block reduction (waves*NREP*128 floats) reuses it
        const size_t lds = (size_t)p.waves * rows_mfma_sets(NREP) * kRowsMfmaTile * sizeof(uint16_t);
        constexpr int DEPTH = 1;  // chunks in flight per wave (deeper costs occupancy and was slower)
        if (lds > 64 * 1024 && !t_plan) {
            // above the default per-block limit: raise it for this kernel, once per device
            // (the attribute is idempotent: two threads that both find the flag clear set it twice)
            static std::atomic<bool> raised[kMaxDevices];
            int dev = 0;
            if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices ||
                !raised[dev].load(std::memory_order_acquire)) {
                (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_rows_mfma<MODE, NREP, DEPTH>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
                if (dev >= 0 && dev < kMaxDevices) raised[dev].store(true, std::memory_order_release);
            }
        }
        KVMIX_LAUNCH((gemv_rows_mfma<MODE, NREP, DEPTH>), grid, block, lds, st, a, "gemv_rows_mfma<%d,%d,%d>", MODE, NREP, DEPTH);
        if (a.splits > 1) {
            const dim3 g2((unsigned)((a.N + 255) / 256), (unsigned)samples, (unsigned)a.M);
            KVMIX_LAUNCH(reduce_splits, g2, dim3(256), 0, st, a, "reduce_splits");
        }
        return;
    }
    const size_t lds = sizeof(float) * (size_t)p.waves * (size_t)NREP * (size_t)(512 + a.N);
    switch (a.N / 32) {
    case 2: KVMIX_LAUNCH((gemv_rows<MODE, 2, NREP>), grid, block, lds, st, a, "gemv_rows<%d,2,%d>", MODE, NREP); break;
    case 4: KVMIX_LAUNCH((gemv_rows<MODE, 4, NREP>), grid, block, lds, st, a, "gemv_rows<%d,4,%d>", MODE, NREP); break;
    default: KVMIX_LAUNCH((gemv_rows<MODE, 8, NREP>), grid, block, lds, st, a, "gemv_rows<%d,8,%d>", MODE, NREP); break;
    }
    if (a.splits > 1) {
        const dim3 g2((unsigned)((a.N + 255) / 256), (unsigned)samples, (unsigned)a.M);
        KVMIX_LAUNCH(reduce_splits, g2, dim3(256), 0, st, a, "reduce_splits");
    }
}

template <int MODE>
static void launch_rows(GemvArgs &a, int64_t samples, hipStream_t st)
{
    if (heads_per_block(a.heads_per_kv) == 4)
        launch_rows_n<MODE, 4>(a, samples, st);
    else
        launch_rows_n<MODE, 1>(a, samples, st);
}

// waves per block for a kernel whose waves each take one of `slots` tiles of an output row:
// the count (2..4) that leaves the fewest launched waves without a tile
static int pick_waves_per_block(int64_t slots)
{
    int wpb = kColsWaves;
    int64_t idle = (slots + wpb - 1) / wpb * wpb - slots;
    for (int w = kColsWaves - 1; w >= 2 && idle > 0; w--) {
        const int64_t i = (slots + w - 1) / w * w - slots;
        if (i < idle) {
            idle = i;
            wpb = w;
        }
    }
    return slots < wpb ? (int)slots : wpb;
}


// units one lane owns in gemv_cols: enough for a 128-bit code load per lane and row
template <int MODE>
struct ColsUpl {
    static constexpr int value = MODE == 3 ? 4 : 1;
};

template <int MODE, int RQ, int UPL>
static void launch_cols_cfg(const GemvArgs &a, int64_t samples, hipStream_t st)
{
    constexpr int VALS = Fmt<MODE>::VALS;
    constexpr int TU = (kWave / RQ) * UPL;
    const int64_t units = a.N / VALS;
    if (!tile_fits(units, TU)) return;
    const int64_t tiles = (units + TU - 1) / TU;
    const int wpb = pick_waves_per_block(tiles);
    const dim3 grid((unsigned)((tiles + wpb - 1) / wpb), (unsigned)samples, (unsigned)a.M);
    KVMIX_LAUNCH((gemv_cols<MODE, RQ, UPL>), grid, dim3(kWave, wpb), 0, st, a, "gemv_cols<%d,%d,%d>", MODE, RQ, UPL);
}

// smallest tile (in units) any gemv_cols configuration of this mode needs
template <int MODE>
static int64_t cols_min_units()
{
    // (reference 3-bit format: gemv_cols3 with two words per lane and two row sections)
    return MODE == 3 ? 64 : 16 * ColsUpl<MODE>::value;
}


template <int RQ, int UPL, int NREP>
static void launch_cols3_cfg(GemvArgs &a, int64_t samples, hipStream_t st, int ks = 1)
{
    constexpr int TU = (kWave / RQ) * UPL;
    const int64_t units = a.N / 11;
    if (!tile_fits(units, TU)) return;
    const int64_t tiles = (units + TU - 1) / TU;
    constexpr int U = NREP > 1 ? kCols3HeadsU : kCols3U;  // rows in flight per lane
    a.ksplit = ks;
    if (ks > 1) {
        // one tile per block: its ks waves slice K and leave their sums behind the x vector in LDS
        const dim3 grid((unsigned)tiles, (unsigned)(samples / NREP), (unsigned)a.M);
        const size_t lds = sizeof(float) * ((size_t)NREP * (size_t)(a.K + 1) + (size_t)ks * NREP * UPL * 11 * kWave);
        KVMIX_LAUNCH((gemv_cols3<RQ, UPL, U, NREP>), grid, dim3(kWave, ks), lds, st, a, "gemv_cols3<%d,%d,%d,%d>", RQ, UPL, U, NREP);
        return;
    }
    const int wpb = pick_waves_per_block(tiles);
    const dim3 grid((unsigned)((tiles + wpb - 1) / wpb), (unsigned)(samples / NREP), (unsigned)a.M);
    KVMIX_LAUNCH((gemv_cols3<RQ, UPL, U, NREP>), grid, dim3(kWave, wpb), sizeof(float) * (size_t)NREP * (size_t)(a.K + 1), st,
                 a, "gemv_cols3<%d,%d,%d,%d>", RQ, UPL, U, NREP);
}

// (gemv_cols_mfma: whole 512-code tiles, at least one whole 32-row chunk)
static bool cols_use_mfma(int mode, int64_t N, int64_t K)
{
    return (mode == 1 || mode == 2 || mode == 4) && N >= 512 && K >= 32;
}

template <int BITS, int NREP>
static void launch_cols_mfma(GemvArgs &a, int64_t samples, hipStream_t st)
{
    if (!tile_fits(a.N / 32, 16) || !tile_fits(a.K, 32)) return;  // a 512-code tile, a 32-row chunk
    const int64_t tiles = (a.N / 32 + 15) / 16;
    const int64_t batch = samples / NREP * a.M;
    // tiles per wave: as many as still leave one resident round of waves (4 per SIMD, 2 for
    // the multi-head kernel); a wave that walks several tiles pays its start-up once
    const int64_t target = NREP > 1 ? kTargetWaves / 2 : kTargetWaves;
    int64_t tpw = batch * tiles / target;
    tpw = tpw < 1 ? 1 : (tpw > 8 ? 8 : tpw);
    const int64_t slots = (tiles + tpw - 1) / tpw;  // waves per output row
    const int wpb = pick_waves_per_block(slots);
    a.splits = (int)tpw;
    const dim3 grid((unsigned)((slots + wpb - 1) / wpb), (unsigned)(samples / NREP), (unsigned)a.M);
    const size_t lds = (size_t)wpb * (cols_mfma_sets(NREP) * kColsMfmaTile * sizeof(uint16_t) + NREP * 16 * sizeof(float));
    KVMIX_LAUNCH((gemv_cols_mfma<BITS, NREP>), grid, dim3(kWave, wpb), lds, st, a, "gemv_cols_mfma<%d,%d>", BITS, NREP);
}

template <int BITS, bool NTC, bool WIDE>
static void launch_cols_mfma2_nt(GemvArgs &a, int64_t samples, hipStream_t st)
{
    constexpr int TG = cols_mfma2_groups(WIDE);  // groups of 32 codes per tile
    if (!tile_fits(a.N / 32, TG) || !tile_fits(a.K, 16)) return;  // a whole tile, a 16-row chunk
    const int64_t tiles = (a.N / 32 + TG - 1) / TG;
    const int64_t batch = samples * a.M;
    // one tile per wave (several tiles per wave, so that one round of resident waves covers the problem, were
    // measured slower at every size).  Few tiles: 2 or 4 waves per tile, each with a share of the K rows (chunks of 16)
    const int64_t chunks = (a.K + 15) / 16;
    int ks = 1;
    while (!WIDE && ks < kColsWaves && batch * tiles * ks * 2 <= kMfma2KsplitWaves && chunks >= ks * 4) ks *= 2;
    a.ksplit = ks;
    a.splits = 1;
    const size_t lds_wave = cols_mfma2_lds(WIDE);
    if (ks > 1) {
        const dim3 grid((unsigned)tiles, (unsigned)samples, (unsigned)a.M);  // one tile per block of ks waves
        KVMIX_LAUNCH((gemv_cols_mfma2<BITS, NTC, WIDE>), grid, dim3(kWave, ks), ks * lds_wave, st, a, "gemv_cols_mfma2<%d,%d,%d>", BITS,
                     (int)NTC, (int)WIDE);
        return;
    }
    const int wpb = pick_waves_per_block(tiles);
    const dim3 grid((unsigned)((tiles + wpb - 1) / wpb), (unsigned)samples, (unsigned)a.M);
    KVMIX_LAUNCH((gemv_cols_mfma2<BITS, NTC, WIDE>), grid, dim3(kWave, wpb), wpb * lds_wave, st, a, "gemv_cols_mfma2<%d,%d,%d>", BITS,
                 (int)NTC, (int)WIDE);
}

// Whether a launch takes the wide tiles (2048 codes per wave, two waves per SIMD) instead of the plain ones (1024
// codes, three waves per SIMD): where the plain tiles would need more than one round of resident waves, the wide
// ones get by with half as many waves that each keep twice the bytes in flight.  Measured, one library against
// the other in one run (plain -> wide, us): T = 8k, B = 16: 4 bits 58.6 -> 56.5, 2 bits 40.2 -> 39.5; B = 24: 92.8 ->
// 90.3, 71.4 -> 68.3; B = 32: 130.1 -> 124.9, 84.9 -> 84.2; B = 8 at T = 16k, 2 bits: 37.5 -> 35.0.  Behind where
// one round of plain tiles covers the launch (B = 12: 44.4 -> 49.2, 29.2 -> 32.1) and on short rows (T = 4k, B = 64:
// 136.6 -> 141.7, 88.0 -> 88.9).
static bool cols_mfma2_wide(int bits, int64_t batch, int64_t N)
{
#ifdef KVMIX_EXPERIMENT
    if (const char *e = getenv("KVMIX_DBG_WIDE")) return atoi(e) != 0 && N >= 2048;
#endif
    (void)bits;
    const int64_t plain_tiles = (N / 32 + 31) / 32;
    return N >= kMfma2WideMinCodes && batch * plain_tiles > (int64_t)kMfma2ResidentWaves;
}

template <int BITS>
static void launch_cols_mfma2(GemvArgs &a, int64_t samples, hipStream_t st)
{
    // non-temporal code loads: 2 and 4 bits (a wave's 1-bit row piece is 128 bytes and shares its cache lines
    // with the neighbours'), and only while the launch is at most three rounds of resident waves
    const int64_t tiles = (a.N / 32 + 31) / 32;
    const bool nt = BITS >= 2 && samples * a.M * tiles <= 3 * (int64_t)kMfma2ResidentWaves;
    const bool wide = cols_mfma2_wide(BITS, samples * a.M, a.N);
    if (wide) {
        if (nt) launch_cols_mfma2_nt<BITS, true, true>(a, samples, st);
        else launch_cols_mfma2_nt<BITS, false, true>(a, samples, st);
    } else {
        if (nt) launch_cols_mfma2_nt<BITS, true, false>(a, samples, st);
        else launch_cols_mfma2_nt<BITS, false, false>(a, samples, st);
    }
}

int plan_attn_slab_mfma(int k_mode, bool coop, int64_t tokens, int64_t samples, int64_t tail_blocks, unsigned grid[3],
                        unsigned block[3])
{
    const int64_t tile = k_mode == 3 ? kSlabRef3Tile : 1024, unit = k_mode == 3 ? 352 : 32;
    const int64_t tiles = (tokens + tile - 1) / tile;
    if (tokens < tile || tokens % unit != 0 || samples <= 0 || tail_blocks < 0) return KVMIX_ERR_SHAPE;
    // blocks per query head: of four tiles, or (coop) one tile shared by the block's four waves
    const int64_t nx = coop ? tiles : (tiles + kColsWaves - 1) / kColsWaves;
    if (nx * samples + tail_blocks > 0x7fffffff) return KVMIX_ERR_SHAPE;
    grid[0] = (unsigned)(nx * samples + tail_blocks), grid[1] = 1, grid[2] = 1;
    block[0] = kWave, block[1] = kColsWaves, block[2] = 1;
    return KVMIX_OK;
}

int launch_attn_step_mfma(const AttnSlabArgs &a, const fused::FusedArgs &f, int k_bits, bool coop, int v_mode, int64_t samples,
                          int64_t tail_blocks, hipStream_t stream)
{
    unsigned g[3], b[3];
    const int prc = plan_attn_slab_mfma(k_bits, coop, a.tokens, samples, tail_blocks, g, b);
    if (prc != KVMIX_OK) return prc;
    const dim3 grid(g[0]), block(b[0], b[1]);
    const unsigned mfma_blocks = (unsigned)(g[0] - tail_blocks), mfma_nx = (unsigned)(mfma_blocks / samples);
    const size_t lds = step_lds(k_bits);
#define KVMIX_SLAB(KB_, VM_)                                                                                   \
    if (coop)                                                                                                  \
        hipLaunchKernelGGL((attn_step_mfma<KB_, VM_, true>), grid, block, lds, stream, a, f, mfma_blocks, mfma_nx); \
    else                                                                                                       \
        hipLaunchKernelGGL((attn_step_mfma<KB_, VM_, false>), grid, block, lds, stream, a, f, mfma_blocks, mfma_nx)
#define KVMIX_SLAB_V(KB_)                          \
    switch (v_mode) {                              \
    case 1: KVMIX_SLAB(KB_, 1); break;             \
    case 2: KVMIX_SLAB(KB_, 2); break;             \
    case 4: KVMIX_SLAB(KB_, 4); break;             \
    case 30: KVMIX_SLAB(KB_, 30); break;           \
    default: return KVMIX_ERR_UNSUPPORTED;         \
    }
    switch (k_bits) {
    case 1: KVMIX_SLAB_V(1) break;
    case 2: KVMIX_SLAB_V(2) break;
    case 3: KVMIX_SLAB_V(3) break;
    case 4: KVMIX_SLAB_V(4) break;
    default: return KVMIX_ERR_UNSUPPORTED;
    }
#undef KVMIX_SLAB_V
#undef KVMIX_SLAB
    return launch_status();
}

// gemv_cols3 with one head per pass: where tiles of 256 words with one wave each, every wave walking all 128 channel
// rows, lay exactly one block on every CU -- 224 to 256 output rows of three or four tiles, the block = the tiles
// of a row -- or exactly three blocks of four waves, they are ahead of the K-sliced 128-word tiles (which put 6 to
// 24 waves on every SIMD): the waves stream 1 KiB pieces of a row and nothing queues.  Measured (us, K-sliced ->
// whole rows): B = 8, T = 8192 (256 rows x 3 tiles): 36.3 -> 32.7; T = 7500: 33.6 -> 29.8; T = 8576: 36.8 -> 34.2;
// T = 11264 (4 tiles): 50.3 -> 43.0; B = 7: 33.3 -> 30.7; three blocks per CU: B = 8, T = 32768: 146.5 -> 138.7; B = 24,
// T = 11264: 147.1 -> 140.0.  One block more than the CUs and the launch takes two rounds: B = 9, T = 8192 (288
// rows): 39.1 -> 57.7, B = 10: 43.9 -> 58.8; fewer rows leave CUs idle: B = 6: 28.7 -> 30.3; other wave counts lose 2 to
// 7 % (B = 16, T = 8192: 68.9 -> 71.6; B = 6, T = 32768: 108.6 -> 115.8).  Tiles of 192 words (three per lane), which
// would put a wave on every SIMD at 256 rows x 733 words, lose to the 12- and 6-byte loads they need (32.8 -> 39.1);
// so does a fourth wave per block that takes the last quarter of the channel rows of all three tiles and hands its
// sums over in LDS (33.7 -> 36.6).
static bool cols3_whole_rows(int64_t units, int64_t rows)
{
    if (units < 513) return false;
    const int64_t tiles = (units + 255) / 256;
    if (tiles <= 4) return rows >= 224 && rows <= 256;
    return tiles % 4 == 0 && rows * (tiles / 4) >= 736 && rows * (tiles / 4) <= 768;
}

template <int MODE>
static void launch_cols(GemvArgs &a, int64_t samples, hipStream_t st)
{
    if constexpr (MODE == 1 || MODE == 2 || MODE == 4) {
        // two-element matrix-core kernel: measured faster than gemv_cols and gemv_cols_mfma up to
        // one resident round of waves (B = 16 at T = 8k); beyond that gemv_cols streams better
        const int64_t tiles2 = (a.N / 32 + 31) / 32;
        // ... and at any batch while a row holds no more than two of gemv_cols' 2048-code tiles (T = 4k,
        // B = 64: 2-bit 111 -> 88 us, 4-bit 133 -> 127 us; at T = 5k gemv_cols is ahead again)
        // 1 bit: only beyond the range of the one-element kernel (which, with its several tiles per
        // wave, is ahead up to one resident round of waves: B = 16, T = 4k: 19.6 against 22.7 us);
        // there, and for rows of up to two of gemv_cols' tiles, it replaces gemv_cols (B = 64, T = 4k:
        // 110 -> 87 us; at T = 8k gemv_cols stays ahead)
        const bool one_bit_ok = MODE != 1 || (a.N <= 2 * 2048 &&
                                              samples * a.M * ((a.N / 32 + 31) / 32) >= (int64_t)kMfma1MaxWaves);
        // ... and with the wide tiles (rows of kMfma2WideMinCodes codes and more): 4 bits up to kMfma2WideMaxWaves of
        // them (beyond, gemv_cols is ahead: T = 8k, B = 20: 73.0 against 79.2 us, B = 48: 173 against 191), 2 bits at
        // any batch (gemv_cols -> wide tiles, us: T = 8k, B = 20: 57.8 -> 53.6, B = 24: 69.3 -> 60.0, B = 32: 85.2 -> 79.8,
        // B = 64: 169.7 -> 159.2; T = 16k, B = 12: 66.1 -> 59.3; T = 32k, B = 8: 78.1 -> 71.9)
        int64_t wide_max = kMfma2WideMaxWaves;
#ifdef KVMIX_EXPERIMENT
        if (const char *e = getenv("KVMIX_DBG_WIDE_MAX")) wide_max = atoll(e);
#endif
        const bool wide_range = MODE != 1 && a.N >= kMfma2WideMinCodes &&
                                (MODE == 2 || samples * a.M * ((a.N / 32 + 63) / 64) <= wide_max);
        if (one_bit_ok && heads_per_block(a.heads_per_kv) == 1 && a.N >= 1024 && a.K >= 16 &&
            (MODE == 1 || samples * a.M * tiles2 <= (int64_t)kMfma2MaxWaves || wide_range || a.N <= 2 * 2048)) {
            launch_cols_mfma2<MODE>(a, samples, st);
            return;
        }
    }
    if constexpr (MODE == 1 || MODE == 2 || MODE == 4) {
        // Matrix-core kernel: always for GQA (the query heads of a kv head share one pass over
        // the codes); for one head per kv head only when the problem is small enough that
        // gemv_cols would have to cut its tiles down to 256-byte row pieces anyway -- measured,
        // gemv_cols with 512-byte pieces streams faster than either kernel with 256-byte ones.
        if (cols_use_mfma(MODE, a.N, a.K)) {
            const int64_t units = a.N / 32, batch = samples * a.M;
            if (heads_per_block(a.heads_per_kv) == 4) {
                launch_cols_mfma<MODE, 4>(a, samples, st);
                return;
            }
            if (batch * ((units + 31) / 32) < (int64_t)kMfma1MaxWaves) {
                launch_cols_mfma<MODE, 1>(a, samples, st);
                return;
            }
        }
    }
    if constexpr (MODE == 3) {
        // reference 3-bit format: register-streaming kernel; the widest tile (256, 128 or 64
        // words per wave) that still gives the chip enough waves and fits into N
        const int64_t units = a.N / 11, batch = samples * a.M;
        auto waves = [&](int64_t tu) { return batch * ((units + tu - 1) / tu); };
        bool force_wide = false;
#ifdef KVMIX_EXPERIMENT
        if (const char *e = getenv("KVMIX_DBG_COLS3_WIDE")) force_wide = atoi(e) == 1 && units >= 256;
#endif
        if (heads_per_block(a.heads_per_kv) == 4 && a.K <= 2048)  // GQA: four query heads per pass over the
            launch_cols3_cfg<2, 2, 4>(a, samples, st);              // words (their x rows must fit into LDS)
        else if (force_wide || cols3_whole_rows(units, batch))
            launch_cols3_cfg<1, 4, 1>(a, samples, st);
        else if (units >= 128 && 2 * ((units + 127) / 128) * 128 <= 3 * units && a.K >= 64 &&
                 a.K <= 4096 && (waves(128) * 4 <= 1024 || waves(128) * 4 >= 2304))
            // tiles of 128 words (512 bytes of codes per row), each shared by four waves that slice K: measured
            // ahead of the one-wave-per-tile configurations below (T = 2.3k..32k, B = 1..128: by 2..35 %) with
            // streaming loads: longer pieces per row, shorter chains of loads per wave.  Not where that makes
            // between one and two waves per SIMD (measured behind there), nor where the last tile, moved back
            // to end at N, would mostly repeat its neighbour.
            launch_cols3_cfg<2, 4, 1>(a, samples, st, 4);
        else if (units >= 256 && waves(256) >= kCols3WideWaves)
            launch_cols3_cfg<1, 4, 1>(a, samples, st);
        else if (units >= 128 && waves(128) >= kCols3MinWaves)
            launch_cols3_cfg<2, 4, 1>(a, samples, st);
        else
            launch_cols3_cfg<2, 2, 1>(a, samples, st);
    } else {
    // more row sections per wave = more, narrower waves: take the widest tile that still
    // gives the chip enough waves and fits into N
    constexpr int VALS = Fmt<MODE>::VALS;
    constexpr int UPL = ColsUpl<MODE>::value;
    const int64_t units = a.N / VALS;
    const int64_t batch = samples * a.M;
    int rq = 4;
    if (batch * ((units + 64 * UPL - 1) / (64 * UPL)) >= kTargetWaves)
        rq = 1;
    else if (batch * ((units + 32 * UPL - 1) / (32 * UPL)) >= kTargetWaves)
        rq = 2;
    while (rq < 4 && units < (64 / rq) * UPL) rq *= 2;  // the tile must fit into N
    if (rq == 4)
        launch_cols_cfg<MODE, 4, UPL>(a, samples, st);
    else if (rq == 2)
        launch_cols_cfg<MODE, 2, UPL>(a, samples, st);
    else
        launch_cols_cfg<MODE, 1, UPL>(a, samples, st);
    }
}

template <int MODE>
static void launch_generic(GemvArgs &a, int64_t samples, hipStream_t st)
{
    constexpr int VALS = GenericCfg<MODE>::VALS;
    constexpr int THREADS = GenericCfg<MODE>::THREADS;
    const int64_t units = a.N / VALS;
    int ub_log2 = 0;
    while ((1 << ub_log2) < THREADS && (1 << ub_log2) < units) ub_log2++;
    const int ub = 1 << ub_log2;
    const size_t lds = ub < THREADS ? (size_t)THREADS * (VALS + 1) * sizeof(float) : 0;
    const dim3 grid((unsigned)((units + ub - 1) / ub), (unsigned)samples, (unsigned)a.M);
    if (t_plan)
        plan_record(grid, dim3(THREADS), lds, "gemv_generic<%d>", MODE);
    else
        hipLaunchKernelGGL(gemv_generic<MODE>, grid, dim3(THREADS), lds, st, a, ub_log2);
}

}  // namespace kvmix

using namespace kvmix;

extern "C" size_t kvmix_gemv_workspace_bytes(int64_t samples, int64_t M, int64_t K, int64_t N)
{
    if (samples <= 0 || M <= 0 || K <= 0 || N <= 0) return 0;
    if (samples > 65535 || M > 65535) return 0;  // (goes out in parts of more than 30000 rows each: never split)
    // the split count depends on the kernel and on how many query heads share a block (which
    // this query does not know): size for the largest of the possible plans
    const RowsPlan p1 = plan_rows(samples * M, K, N, kRowsMaxWaves);
    const RowsPlan p8 = plan_rows(samples * M, K, N, kRowsMfmaWaves);
    const RowsPlan p4 = plan_rows((samples + 3) / 4 * M, K, N, kRowsHeadsWaves);
    int splits = p1.splits > p4.splits ? p1.splits : p4.splits;
    splits = p8.splits > splits ? p8.splits : splits;
    return splits > 1 ? (size_t)(samples * M) * (size_t)splits * (size_t)N * sizeof(float) : 0;
}

// Workspace of kvmix_quantized_gemv_static: the split-K partial sums of the p.V kernels.  Every
// device the library runs on holds its own copy of this array until the process ends.  In host
// code the name stands for the symbol, not for device memory: the address on a device comes from
// hipGetSymbolAddress (static_scratch below) and only that pointer is handed to kernels.
static __device__ __align__(256) unsigned char scratch[KVMIX_GEMV_STATIC_SCRATCH_BYTES];

// the array's address on the current device, looked up once per device; nullptr on failure
static void *static_scratch()
{
    static std::mutex lock;
    static void *ptr[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> hold(lock);
    if (!ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        ptr[dev] = p;
    }
    return ptr[dev];
}

static int quantized_gemv(int group, const void *x, int64_t x_batch_stride,
                          int64_t x_row_stride, const uint32_t *code,
                          int64_t code_batch_stride, int64_t code_row_stride,
                          const void *scale, const void *zero, int64_t sz_batch_stride,
                          int64_t sz_row_stride, int bits, int fmt, int64_t samples,
                          int heads_per_kv, int64_t M, int64_t K, int64_t N, void *out,
                          int64_t out_batch_stride, int64_t out_row_stride, void *workspace,
                          size_t workspace_bytes, bool workspace_is_static, kvmix_stream_t stream);

extern "C" int kvmix_quantized_gemv(int group, const void *x, int64_t x_batch_stride,
                                    int64_t x_row_stride, const uint32_t *code,
                                    int64_t code_batch_stride, int64_t code_row_stride,
                                    const void *scale, const void *zero, int64_t sz_batch_stride,
                                    int64_t sz_row_stride, int bits, int fmt, int64_t samples,
                                    int heads_per_kv, int64_t M, int64_t K, int64_t N, void *out,
                                    int64_t out_batch_stride, int64_t out_row_stride, void *workspace,
                                    size_t workspace_bytes, kvmix_stream_t stream)
{
    return quantized_gemv(group, x, x_batch_stride, x_row_stride, code, code_batch_stride, code_row_stride, scale,
                          zero, sz_batch_stride, sz_row_stride, bits, fmt, samples, heads_per_kv, M, K, N, out,
                          out_batch_stride, out_row_stride, workspace, workspace_bytes, false, stream);
}

extern "C" int kvmix_quantized_gemv_static(int group, const void *x, int64_t x_batch_stride,
                                           int64_t x_row_stride, const uint32_t *code,
                                           int64_t code_batch_stride, int64_t code_row_stride,
                                           const void *scale, const void *zero, int64_t sz_batch_stride,
                                           int64_t sz_row_stride, int bits, int fmt, int64_t samples,
                                           int heads_per_kv, int64_t M, int64_t K, int64_t N, void *out,
                                           int64_t out_batch_stride, int64_t out_row_stride,
                                           kvmix_stream_t stream)
{
    // (the arguments are checked first, as in kvmix_quantized_gemv; the buffer is looked up only by a call whose
    // plan splits K, so q.K^T products and unsplit batches never touch the lock or the symbol)
    return quantized_gemv(group, x, x_batch_stride, x_row_stride, code, code_batch_stride, code_row_stride, scale,
                          zero, sz_batch_stride, sz_row_stride, bits, fmt, samples, heads_per_kv, M, K, N, out,
                          out_batch_stride, out_row_stride, nullptr, 0, true, stream);
}

static int quantized_gemv(int group, const void *x, int64_t x_batch_stride,
                          int64_t x_row_stride, const uint32_t *code,
                          int64_t code_batch_stride, int64_t code_row_stride,
                          const void *scale, const void *zero, int64_t sz_batch_stride,
                          int64_t sz_row_stride, int bits, int fmt, int64_t samples,
                          int heads_per_kv, int64_t M, int64_t K, int64_t N, void *out,
                          int64_t out_batch_stride, int64_t out_row_stride, void *workspace,
                          size_t workspace_bytes, bool workspace_is_static, kvmix_stream_t stream)
{
    if (fmt != KVMIX_FMT_REF && fmt != KVMIX_FMT_DENSE3) return KVMIX_ERR_FORMAT;
    if (bits != 1 && bits != 2 && bits != 3 && bits != 4) return KVMIX_ERR_BITS;
    if (fmt == KVMIX_FMT_DENSE3 && bits != 3) return KVMIX_ERR_FORMAT;
    if (heads_per_kv <= 0 || samples < 0 || samples % heads_per_kv != 0) return KVMIX_ERR_HEADS;
    const bool ref3 = bits == 3 && fmt == KVMIX_FMT_REF;
    if (ref3 && group != 11) return KVMIX_ERR_GROUP3;
    if (M < 0 || K < 0 || N < 0 || group <= 0) return KVMIX_ERR_SHAPE;
    if (N % group != 0) return KVMIX_ERR_STEPS_GROUP;
    const int mode = ref3 ? 3 : (bits == 3 ? 30 : bits);
    const int64_t unit_vals = mode == 30 ? 32 : (mode == 3 ? 11 : 32 / bits);
    const int64_t unit_words = mode == 30 ? 3 : 1;
    if (N % unit_vals != 0) return KVMIX_ERR_STEPS_WORD;
    // a packed unit must not straddle two groups (the reference would silently use the
    // first group's scale for the whole word)
    if (group % unit_vals != 0) return KVMIX_ERR_UNSUPPORTED;
    if (samples == 0 || M == 0 || N == 0) return KVMIX_OK;
    if (!t_plan) {
        if (!out) return KVMIX_ERR_NULL;
        if (K > 0 && (!x || !code || !scale || !zero)) return KVMIX_ERR_NULL;
    }
    const int64_t words = N / unit_vals * unit_words, groups = N / group;
    if (code_row_stride < words || sz_row_stride < groups || x_row_stride < K || out_row_stride < N)
        return KVMIX_ERR_SHAPE;
    // the built-in buffer: the documented bound, not the launch plan's exact need -- what is refused depends on
    // the sizes only
    if (workspace_is_static && kvmix_gemv_workspace_bytes(samples, M, K, N) > KVMIX_GEMV_STATIC_SCRATCH_BYTES)
        return KVMIX_ERR_STATIC_SCRATCH;
    // grid.y / grid.z hold at most 65535 blocks: a larger batch goes out as several launches of nearly equal
    // size over whole kv heads (and whole groups of M rows), one after the other on the stream.  (Each part
    // then still has more than 30000 output rows, which no kernel splits over blocks: no workspace.)
    if (heads_per_kv > 65535) return KVMIX_ERR_SHAPE;
    if (samples > 65535 || M > 65535) {
        const int64_t kvs = samples / heads_per_kv, kv_max = 65535 / heads_per_kv;
        const int64_t sparts = (kvs + kv_max - 1) / kv_max, mparts = (M + 65534) / 65535;
        const int64_t kv_step = (kvs + sparts - 1) / sparts, mstep = (M + mparts - 1) / mparts;
        for (int64_t m0 = 0; m0 < M; m0 += mstep) {
            for (int64_t kv0 = 0; kv0 < kvs; kv0 += kv_step) {
                const int64_t s0 = kv0 * heads_per_kv, nkv = kvs - kv0 < kv_step ? kvs - kv0 : kv_step;
                const int64_t nm = M - m0 < mstep ? M - m0 : mstep;
                const int rc = quantized_gemv(
                    group, x ? (const __half *)x + s0 * x_batch_stride + m0 * x_row_stride : nullptr, x_batch_stride,
                    x_row_stride, code ? code + kv0 * code_batch_stride : nullptr, code_batch_stride, code_row_stride,
                    scale ? (const __half *)scale + kv0 * sz_batch_stride : nullptr,
                    zero ? (const __half *)zero + kv0 * sz_batch_stride : nullptr, sz_batch_stride, sz_row_stride, bits,
                    fmt, nkv * heads_per_kv, heads_per_kv, nm, K, N,
                    out ? (__half *)out + s0 * out_batch_stride + m0 * out_row_stride : nullptr, out_batch_stride,
                    out_row_stride, workspace, workspace_bytes, workspace_is_static, stream);
                if (rc != KVMIX_OK) return rc;
            }
        }
        return KVMIX_OK;
    }

    GemvArgs a;
    a.x = (const __half *)x;
    a.code = code;
    a.scale = (const __half *)scale;
    a.zero = (const __half *)zero;
    a.out = (__half *)out;
    a.partial = (float *)workspace;
    a.x_bs = x_batch_stride;
    a.x_rs = x_row_stride;
    a.c_bs = code_batch_stride;
    a.c_rs = code_row_stride;
    a.s_bs = sz_batch_stride;
    a.s_rs = sz_row_stride;
    a.o_bs = out_batch_stride;
    a.o_rs = out_row_stride;
    a.K = K;
    a.N = N;
    a.M = M;
    a.heads_per_kv = heads_per_kv;
    a.group = group;
    a.splits = 1;
    a.ksplit = 1;
    a.rows_per_split = K > 0 ? K : 1;
    hipStream_t st = (hipStream_t)stream;

    // the fast kernels index one (batch, kv-head) slice with 32-bit offsets
    const bool small = K < (1 << 30) && N < (1 << 30) && (K + 1) * code_row_stride < (1ll << 30) &&
                       (K + 1) * sz_row_stride < (1ll << 30);
    const bool fast_group = small && (ref3 ? true : group == 32);
    // gemv_rows reads a chunk's scale/zero as one flat array: rows must be contiguous
    const bool rows_ok = fast_group && !ref3 && rows_shape_ok(N) && sz_row_stride == N / 32 && K >= 8;
    // gemv_cols needs one whole wave tile of group units along N
    const int64_t min_units = mode == 3 ? cols_min_units<3>() : cols_min_units<4>();
    // (gemv_cols3 keeps x for all K rows in LDS)
    const bool cols_ok = fast_group && K > 0 && N / (ref3 ? 11 : 32) >= min_units && (!ref3 || K <= 8192);
    // p.V shape: few columns, many rows.  q.K^T shape: the opposite.
    const bool use_rows = rows_ok && (K >= 2 * N || !cols_ok);

#define KVMIX_DISPATCH(fn)                                   \
    switch (mode) {                                          \
    case 1: fn<1>(a, samples, st); break;                    \
    case 2: fn<2>(a, samples, st); break;                    \
    case 3: fn<3>(a, samples, st); break;                    \
    case 4: fn<4>(a, samples, st); break;                    \
    default: fn<30>(a, samples, st); break;                  \
    }

    t_refused = KVMIX_OK;
    if (use_rows) {
        const int nrep = heads_per_block(heads_per_kv);
        const RowsPlan p = plan_rows(samples / nrep * M, K, N,
                                     rows_max_waves(rows_use_mfma(mode, N, K, code_row_stride), nrep));
        if (p.splits > 1 && !t_plan) {
            const size_t need = (size_t)(samples * M) * (size_t)p.splits * (size_t)N * sizeof(float);
            if (workspace_is_static) {
                if (need > KVMIX_GEMV_STATIC_SCRATCH_BYTES) return KVMIX_ERR_STATIC_SCRATCH;
                a.partial = (float *)static_scratch();
                if (!a.partial) return KVMIX_ERR_STATIC_LOOKUP;
            } else if (!workspace || workspace_bytes < need) {
                return KVMIX_ERR_WORKSPACE;
            }
        }
        switch (mode) {
        case 1: launch_rows<1>(a, samples, st); break;
        case 2: launch_rows<2>(a, samples, st); break;
        case 4: launch_rows<4>(a, samples, st); break;
        default: launch_rows<30>(a, samples, st); break;
        }
    } else if (cols_ok) {
        KVMIX_DISPATCH(launch_cols)
    } else {
        KVMIX_DISPATCH(launch_generic)
    }
#undef KVMIX_DISPATCH
    if (t_refused != KVMIX_OK) return t_refused;  // (a launcher found its kernel's tile wider than the problem)
    if (t_plan) {
        t_plan->splits = a.splits;
        t_plan->ksplit = a.ksplit;
        return KVMIX_OK;
    }
    return launch_status();
}

extern "C" int kvmix_quantized_gemv_plan(int group, int bits, int fmt, int64_t samples, int heads_per_kv, int64_t M,
                                         int64_t K, int64_t N, int64_t code_row_stride, int64_t sz_row_stride,
                                         kvmix_gemv_plan_t *plan)
{
    if (!plan) return KVMIX_ERR_NULL;
    *plan = kvmix_gemv_plan_t{};
    t_plan = plan;
    // contiguous slices: the batch strides only enter the kernels, not the dispatch
    const int rc = quantized_gemv(group, nullptr, M * K, K, nullptr, K * code_row_stride, code_row_stride, nullptr, nullptr,
                                  K * sz_row_stride, sz_row_stride, bits, fmt, samples, heads_per_kv, M, K, N, nullptr, M * N,
                                  N, nullptr, 0, false, nullptr);
    t_plan = nullptr;
    return rc;
}
