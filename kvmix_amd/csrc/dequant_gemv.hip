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
// term is one fma per (k, group) instead of one per element, and the first needs one
// int->float conversion and one fma per element.  All accumulation is fp32.
//
// Kernels
//   gemv_cols   q.K^T shape (K = head_dim small, N = tokens large).  A lane owns one
//               quantization group of N (32 codes, or one 11-code word in the reference's
//               3-bit format) and walks down the K rows: no cross-lane reduction at all.
//               The K rows are split over the waves of the block, partials meet in LDS.
//               x (the query) is staged in LDS as fp32.
//   gemv_rows   p.V shape (K = tokens large, N = head_dim small).  A lane owns one group
//               of one row; a wave covers 64/(N/32) rows per load.  Per-lane fp32
//               accumulators, butterfly reduction across the row lanes, LDS across waves,
//               split-K across blocks with fp32 partials in the workspace.
//   gemv_generic  any shape/group: one thread per packed word, serial over K.
//   reduce_splits sums the split-K partials and stores fp16.

#include "kvmix_common.h"

namespace kvmix {

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
};

// MODE: 1, 2, 4 = reference layout with that many bits (group 32 in the fast kernels),
//       3 = the reference's 3-bit layout (11 codes per word, group 11),
//       30 = dense 3-bit stream (32 codes in 3 words, group 32).
template <int MODE>
struct Fmt {
    static constexpr int BITS = MODE == 30 ? 3 : MODE;
    static constexpr int VALS = MODE == 3 ? 11 : 32;                  // codes per group unit
    static constexpr int WORDS = MODE == 3 ? 1 : (MODE == 30 ? 3 : MODE);  // words per group unit
};

// 4-byte-aligned vector of W words: lets the compiler use one wide load where rows are
// only dword aligned (global memory tolerates dword-aligned wide loads on gfx9).
template <int W>
struct __attribute__((packed, aligned(4))) Words {
    uint32_t v[W];
};

// acc[i] += qs * code_i for the VALS codes held in w[]; qs = x_k * scale_k.
template <int MODE>
__device__ __forceinline__ void accumulate_unit(const uint32_t *w, float qs, float *acc)
{
    if constexpr (MODE == 4) {
        const float qs16 = qs * 0.0625f;  // exact: the high nibble is read as 16*code
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t lo = w[j] & 0x0F0F0F0Fu, hi = w[j] & 0xF0F0F0F0u;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                acc[8 * j + 2 * b] = fmaf(qs, (float)((lo >> (8 * b)) & 0xffu), acc[8 * j + 2 * b]);
                acc[8 * j + 2 * b + 1] = fmaf(qs16, (float)((hi >> (8 * b)) & 0xffu), acc[8 * j + 2 * b + 1]);
            }
        }
    } else if constexpr (MODE == 2) {
        const float q1 = qs, q4 = qs * 0.25f, q16 = qs * 0.0625f, q64 = qs * 0.015625f;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t m0 = w[j] & 0x03030303u, m1 = w[j] & 0x0C0C0C0Cu, m2 = w[j] & 0x30303030u,
                           m3 = w[j] & 0xC0C0C0C0u;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                float *a = acc + 16 * j + 4 * b;
                a[0] = fmaf(q1, (float)((m0 >> (8 * b)) & 0xffu), a[0]);
                a[1] = fmaf(q4, (float)((m1 >> (8 * b)) & 0xffu), a[1]);
                a[2] = fmaf(q16, (float)((m2 >> (8 * b)) & 0xffu), a[2]);
                a[3] = fmaf(q64, (float)((m3 >> (8 * b)) & 0xffu), a[3]);
            }
        }
    } else if constexpr (MODE == 1) {
        float qv[8];
        qv[0] = qs;
#pragma unroll
        for (int s = 1; s < 8; s++) qv[s] = qv[s - 1] * 0.5f;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const uint32_t m = w[0] & (0x01010101u << s);
#pragma unroll
            for (int b = 0; b < 4; b++)
                acc[8 * b + s] = fmaf(qv[s], (float)((m >> (8 * b)) & 0xffu), acc[8 * b + s]);
        }
    } else if constexpr (MODE == 3) {
#pragma unroll
        for (int i = 0; i < 10; i++) acc[i] = fmaf(qs, (float)((w[0] >> (3 * i)) & 7u), acc[i]);
        acc[10] = fmaf(qs, (float)(w[0] >> 30), acc[10]);
    } else {  // dense 3-bit stream over three words
        const uint64_t lo = (uint64_t)w[0] | ((uint64_t)w[1] << 32);
        const uint64_t hi = (uint64_t)w[1] | ((uint64_t)w[2] << 32);
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const int bit = 3 * i;
            const uint32_t c = bit < 32 ? (uint32_t)(lo >> bit) & 7u : (uint32_t)(hi >> (bit - 32)) & 7u;
            acc[i] = fmaf(qs, (float)c, acc[i]);
        }
    }
}

// ---------------------------------------------------------------------------------------
// gemv_cols: lanes along N (one group per lane), waves split K.  blockDim = (64, KW).
// grid = (ceil(groups/64), samples, M).  Dynamic LDS: K floats (x) + KW*VALS*64 floats.
// ---------------------------------------------------------------------------------------
template <int MODE>
__global__ void __launch_bounds__(256) gemv_cols(GemvArgs a)
{
    using F = Fmt<MODE>;
    constexpr int VALS = F::VALS, WORDS = F::WORDS;
    extern __shared__ float lds[];
    float *xs = lds;
    float *red = lds + ((a.K + 63) & ~(int64_t)63);

    const int lane = threadIdx.x;
    const int wy = threadIdx.y;
    const int KW = blockDim.y;
    const int64_t sample = blockIdx.y;
    const int64_t m = blockIdx.z;
    const int64_t kv = sample / a.heads_per_kv;
    const int64_t ngroups = a.N / VALS;
    const int64_t G = (int64_t)blockIdx.x * kWave + lane;
    const bool active = G < ngroups;

    const __half *xp = a.x + sample * a.x_bs + m * a.x_rs;
    for (int64_t k = wy * kWave + lane; k < a.K; k += KW * kWave) xs[k] = __half2float(xp[k]);
    __syncthreads();

    float acc[VALS];
#pragma unroll
    for (int i = 0; i < VALS; i++) acc[i] = 0.f;
    float zsum = 0.f;

    if (active) {
        const int64_t kper = (a.K + KW - 1) / KW;
        const int64_t k0 = wy * kper;
        const int64_t k1 = k0 + kper < a.K ? k0 + kper : a.K;
        const uint32_t *cp = a.code + kv * a.c_bs + G * WORDS + k0 * a.c_rs;
        const __half *sp = a.scale + kv * a.s_bs + G + k0 * a.s_rs;
        const __half *zp = a.zero + kv * a.s_bs + G + k0 * a.s_rs;
#pragma unroll 4
        for (int64_t k = k0; k < k1; k++) {
            const Words<WORDS> w = *reinterpret_cast<const Words<WORDS> *>(cp);
            const float s = __half2float(*sp);
            const float z = __half2float(*zp);
            const float xv = xs[k];
            zsum = fmaf(xv, z, zsum);
            accumulate_unit<MODE>(w.v, xv * s, acc);
            cp += a.c_rs;
            sp += a.s_rs;
            zp += a.s_rs;
        }
    }
#pragma unroll
    for (int i = 0; i < VALS; i++) acc[i] += zsum;

    __half *op = a.out + sample * a.o_bs + m * a.o_rs + G * VALS;
    if (KW == 1) {
        if (active) {
#pragma unroll
            for (int i = 0; i < VALS; i++) op[i] = __float2half_rn(acc[i]);
        }
        return;
    }
    // cross-wave reduction: red[wy][i][lane]
#pragma unroll
    for (int i = 0; i < VALS; i++) red[(wy * VALS + i) * kWave + lane] = acc[i];
    __syncthreads();
    if (!active) return;
    for (int i = wy; i < VALS; i += KW) {
        float r = 0.f;
        for (int w = 0; w < KW; w++) r += red[(w * VALS + i) * kWave + lane];
        op[i] = __float2half_rn(r);
    }
}

// ---------------------------------------------------------------------------------------
// gemv_rows: lanes along (row, group); LPR = N/32 lanes per row; blockDim = (64, KW).
// grid = (splits, samples, M).  Static LDS: KW * N floats.
// ---------------------------------------------------------------------------------------
template <int MODE, int LPR>
__global__ void __launch_bounds__(256) gemv_rows(GemvArgs a)
{
    using F = Fmt<MODE>;
    constexpr int VALS = F::VALS, WORDS = F::WORDS;
    static_assert(VALS == 32, "gemv_rows handles 32-code groups");
    constexpr int RPW = kWave / LPR;  // rows per wave per step
    constexpr int KWMAX = 4;
    __shared__ float red[KWMAX][LPR * VALS];

    const int lane = threadIdx.x;
    const int wy = threadIdx.y;
    const int KW = blockDim.y;
    const int r = lane / LPR;
    const int j = lane % LPR;
    const int64_t sample = blockIdx.y;
    const int64_t m = blockIdx.z;
    const int64_t kv = sample / a.heads_per_kv;
    const int64_t kbeg = (int64_t)blockIdx.x * a.rows_per_split;
    const int64_t kend = kbeg + a.rows_per_split < a.K ? kbeg + a.rows_per_split : a.K;

    const __half *xp = a.x + sample * a.x_bs + m * a.x_rs;
    const uint32_t *cp = a.code + kv * a.c_bs + j * WORDS;
    const __half *sp = a.scale + kv * a.s_bs + j;
    const __half *zp = a.zero + kv * a.s_bs + j;

    float acc[VALS];
#pragma unroll
    for (int i = 0; i < VALS; i++) acc[i] = 0.f;
    float zsum = 0.f;

#pragma unroll 4
    for (int64_t kt = kbeg + wy * RPW; kt < kend; kt += KW * RPW) {
        const int64_t k = kt + r;
        if (k < kend) {
            const Words<WORDS> w = *reinterpret_cast<const Words<WORDS> *>(cp + k * a.c_rs);
            const float s = __half2float(sp[k * a.s_rs]);
            const float z = __half2float(zp[k * a.s_rs]);
            const float xv = __half2float(xp[k]);
            zsum = fmaf(xv, z, zsum);
            accumulate_unit<MODE>(w.v, xv * s, acc);
        }
    }
#pragma unroll
    for (int i = 0; i < VALS; i++) {
        float v = acc[i] + zsum;
#pragma unroll
        for (int off = LPR; off < kWave; off <<= 1) v += __shfl_xor(v, off);
        acc[i] = v;
    }
    if (r == 0) {
#pragma unroll
        for (int i = 0; i < VALS; i++) red[wy][j * VALS + i] = acc[i];
    }
    __syncthreads();
    const int t = wy * kWave + lane;
    if (t < LPR * VALS) {
        float v = 0.f;
        for (int w = 0; w < KW; w++) v += red[w][t];
        if (a.splits == 1)
            a.out[sample * a.o_bs + m * a.o_rs + t] = __float2half_rn(v);
        else
            a.partial[((sample * a.M + m) * a.splits + blockIdx.x) * a.N + t] = v;
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
__global__ void __launch_bounds__(256) gemv_generic(GemvArgs a)
{
    constexpr int BITS = MODE == 30 ? 3 : MODE;
    constexpr int VALS = MODE == 30 ? 32 : (MODE == 3 ? 11 : 32 / BITS);
    constexpr int WORDS = MODE == 30 ? 3 : 1;
    const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t units = a.N / VALS;
    if (u >= units) return;
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
    for (int64_t k = 0; k < a.K; k++) {
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
    __half *op = a.out + sample * a.o_bs + m * a.o_rs + u * VALS;
#pragma unroll
    for (int i = 0; i < VALS; i++) op[i] = __float2half_rn(acc[i] + zsum);
}

// --------------------------- host side ---------------------------

constexpr int kRowsKW = 4;          // waves per block in gemv_rows
constexpr int kColsKW = 4;          // waves per block in gemv_cols
constexpr int64_t kTargetBlocks = 1024;  // ~4 blocks of 4 waves on each of 256 CUs
constexpr int64_t kColsMaxK = 4096;

static bool rows_shape_ok(int64_t N) { return N == 64 || N == 128 || N == 256; }

// split-K factor of gemv_rows for a problem (same function sizes the workspace)
static int choose_splits(int64_t batch_rows, int64_t K, int64_t N)
{
    if (!rows_shape_ok(N) || batch_rows <= 0) return 1;
    const int64_t lpr = N / 32;
    const int64_t tile = (int64_t)kRowsKW * (kWave / lpr);  // rows one block covers per step
    int64_t want = (kTargetBlocks + batch_rows - 1) / batch_rows;
    int64_t most = (K + 2 * tile - 1) / (2 * tile);  // at least two steps per block
    if (most < 1) most = 1;
    if (want > most) want = most;
    if (want > 256) want = 256;
    return (int)(want < 1 ? 1 : want);
}

template <int MODE>
static void launch_rows(const GemvArgs &a, int64_t samples, hipStream_t st)
{
    const dim3 grid((unsigned)a.splits, (unsigned)samples, (unsigned)a.M), block(kWave, kRowsKW);
    switch (a.N / 32) {
    case 2: hipLaunchKernelGGL((gemv_rows<MODE, 2>), grid, block, 0, st, a); break;
    case 4: hipLaunchKernelGGL((gemv_rows<MODE, 4>), grid, block, 0, st, a); break;
    default: hipLaunchKernelGGL((gemv_rows<MODE, 8>), grid, block, 0, st, a); break;
    }
    if (a.splits > 1) {
        const dim3 g2((unsigned)((a.N + 255) / 256), (unsigned)samples, (unsigned)a.M);
        hipLaunchKernelGGL(reduce_splits, g2, dim3(256), 0, st, a);
    }
}

template <int MODE>
static void launch_cols(const GemvArgs &a, int64_t samples, hipStream_t st)
{
    constexpr int VALS = Fmt<MODE>::VALS;
    const int64_t groups = a.N / VALS;
    const dim3 grid((unsigned)((groups + kWave - 1) / kWave), (unsigned)samples, (unsigned)a.M);
    const int kw = a.K >= 4 * kColsKW ? kColsKW : 1;
    const size_t lds = sizeof(float) * (size_t)(((a.K + 63) & ~(int64_t)63) + (kw > 1 ? kw * VALS * kWave : 0));
    hipLaunchKernelGGL(gemv_cols<MODE>, grid, dim3(kWave, kw), lds, st, a);
}

template <int MODE>
static void launch_generic(const GemvArgs &a, int64_t samples, hipStream_t st)
{
    constexpr int VALS = MODE == 30 ? 32 : (MODE == 3 ? 11 : 32 / MODE);
    const int64_t units = a.N / VALS;
    const dim3 grid((unsigned)((units + 255) / 256), (unsigned)samples, (unsigned)a.M);
    hipLaunchKernelGGL(gemv_generic<MODE>, grid, dim3(256), 0, st, a);
}

}  // namespace kvmix

using namespace kvmix;

extern "C" size_t kvmix_gemv_workspace_bytes(int64_t samples, int64_t M, int64_t K, int64_t N)
{
    if (samples <= 0 || M <= 0 || K <= 0 || N <= 0) return 0;
    const int splits = choose_splits(samples * M, K, N);
    return splits > 1 ? (size_t)(samples * M) * (size_t)splits * (size_t)N * sizeof(float) : 0;
}

extern "C" int kvmix_quantized_gemv(int group, const void *x, int64_t x_batch_stride,
                                    int64_t x_row_stride, const uint32_t *code,
                                    int64_t code_batch_stride, int64_t code_row_stride,
                                    const void *scale, const void *zero, int64_t sz_batch_stride,
                                    int64_t sz_row_stride, int bits, int fmt, int64_t samples,
                                    int heads_per_kv, int64_t M, int64_t K, int64_t N, void *out,
                                    int64_t out_batch_stride, int64_t out_row_stride, void *workspace,
                                    size_t workspace_bytes, kvmix_stream_t stream)
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
    if (!out) return KVMIX_ERR_NULL;
    if (K > 0 && (!x || !code || !scale || !zero)) return KVMIX_ERR_NULL;
    const int64_t words = N / unit_vals * unit_words, groups = N / group;
    if (code_row_stride < words || sz_row_stride < groups || x_row_stride < K || out_row_stride < N)
        return KVMIX_ERR_SHAPE;
    if (samples > 65535 * 16 || M > 65535) return KVMIX_ERR_SHAPE;

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
    a.rows_per_split = K;
    hipStream_t st = (hipStream_t)stream;
    if (samples > 65535) return KVMIX_ERR_SHAPE;  // grid.y limit

    const bool fast_group = ref3 ? true : group == 32;
    const bool rows_ok = fast_group && !ref3 && rows_shape_ok(N);
    const bool cols_ok = fast_group && K <= kColsMaxK;
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

    if (use_rows) {
        a.splits = choose_splits(samples * M, K, N);
        if (a.splits > 1) {
            const size_t need = (size_t)(samples * M) * (size_t)a.splits * (size_t)N * sizeof(float);
            if (!workspace || workspace_bytes < need) return KVMIX_ERR_WORKSPACE;
        }
        const int64_t tile = (int64_t)kRowsKW * (kWave / (N / 32));
        int64_t rps = (K + a.splits - 1) / a.splits;
        rps = (rps + tile - 1) / tile * tile;
        a.rows_per_split = rps;
        a.splits = (int)((K + rps - 1) / rps);
        if (a.splits < 1) a.splits = 1;
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
    return launch_status();
}
