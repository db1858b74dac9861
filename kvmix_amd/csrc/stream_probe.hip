// Streaming-read probe: what a kernel that only reads (no arithmetic beyond an xor that keeps the
// loads alive) reaches on this GPU for the two access patterns of the GEMV kernels.  It is the
// ceiling the measured kernels are compared with; nothing in the operators calls it.
//
//   pattern 0, "slab":  every block owns a contiguous slab of the buffer, its waves take 64*BPL*U-byte
//                       chunks of it round-robin (the p.V kernels: a (batch, head) slice of value codes
//                       is one contiguous run of token rows);
//   pattern 1, "rows":  the buffer is [slices][rows][row_bytes]; a wave owns a column piece of
//                       64*BPL bytes and walks it down all rows of its slice, U rows in flight (the
//                       q.K^T kernels: a channel row per head dimension, `rows` = 128).
// BPL = bytes per lane and load instruction (4, 8, 16), U = load instructions in flight per wave,
// NT = non-temporal loads.
#include "kvmix_common.h"

namespace kvmix {

template <int BPL>
struct ProbeVec;
template <>
struct ProbeVec<4> {
    using type = uint32_t;
};
template <>
struct ProbeVec<8> {
    using type = uint2;
};
template <>
struct ProbeVec<16> {
    using type = uint4;
};

template <int BPL, bool NT>
__device__ __forceinline__ uint32_t probe_load(const uint8_t *p)
{
    using V = typename ProbeVec<BPL>::type;
    if constexpr (BPL == 4) {
        return NT ? __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p))
                  : *reinterpret_cast<const uint32_t *>(p);
    } else if constexpr (BPL == 8) {
        const uint32_t *q = reinterpret_cast<const uint32_t *>(p);
        if constexpr (NT) {
            typedef uint32_t u2 __attribute__((ext_vector_type(2)));
            const u2 v = __builtin_nontemporal_load(reinterpret_cast<const u2 *>(p));
            return v.x ^ v.y;
        } else {
            const V v = *reinterpret_cast<const V *>(q);
            return v.x ^ v.y;
        }
    } else {
        if constexpr (NT) {
            typedef uint32_t u4 __attribute__((ext_vector_type(4)));
            const u4 v = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p));
            return v.x ^ v.y ^ v.z ^ v.w;
        } else {
            const V v = *reinterpret_cast<const V *>(p);
            return v.x ^ v.y ^ v.z ^ v.w;
        }
    }
}

template <int BPL, int U, bool NT>
__global__ void __launch_bounds__(1024) probe_slab(const uint8_t *buf, int64_t slab_bytes, uint32_t *sink)
{
    constexpr int64_t CHUNK = (int64_t)kWave * BPL * U;
    const int lane = threadIdx.x, wy = threadIdx.y, W = blockDim.y;
    const uint8_t *base = buf + (int64_t)blockIdx.x * slab_bytes + lane * BPL;
    const int64_t chunks = slab_bytes / CHUNK;
    uint32_t acc = 0;
    for (int64_t c = wy; c < chunks; c += W) {
        const uint8_t *q = base + c * CHUNK;
        uint32_t v[U];
#pragma unroll
        for (int i = 0; i < U; i++) v[i] = probe_load<BPL, NT>(q + (int64_t)i * kWave * BPL);
#pragma unroll
        for (int i = 0; i < U; i++) acc ^= v[i];
    }
    if (acc == 0x12345678u) sink[0] = acc;  // (never true for the buffers the bench fills: keeps the loads)
}

template <int BPL, int U, bool NT>
__global__ void __launch_bounds__(256) probe_rows(const uint8_t *buf, int64_t rows, int64_t row_bytes, int64_t pieces,
                                                  uint32_t *sink)
{
    // grid.x = ceil(pieces / waves per block), grid.y = slices
    const int lane = threadIdx.x;
    int64_t piece = (int64_t)blockIdx.x * blockDim.y + threadIdx.y;
    if (piece >= pieces) return;
    int64_t col = piece * (kWave * BPL);
    if (col + kWave * BPL > row_bytes) col = row_bytes - kWave * BPL;  // the last piece is moved back to end at the row's end
    const uint8_t *base = buf + (int64_t)blockIdx.y * rows * row_bytes + col + lane * BPL;
    uint32_t acc = 0;
    for (int64_t r = 0; r + U <= rows; r += U) {
        uint32_t v[U];
#pragma unroll
        for (int i = 0; i < U; i++) v[i] = probe_load<BPL, NT>(base + (r + i) * row_bytes);
#pragma unroll
        for (int i = 0; i < U; i++) acc ^= v[i];
    }
    if (acc == 0x12345678u) sink[0] = acc;
}

// pattern 2: pattern 1 with 16 rows in flight and 8 bytes per lane, plus what the q.K^T kernels read beside
// the codes: per 16 rows one 16-byte load per lane from each of two side arrays [slices][rows][side_row_bytes]
// (lane = row lane/4 of the 16, bytes 64*piece + 16*(lane%4) of it: 64-byte pieces per row and wave).
template <bool NT, bool NT_SIDE>
__global__ void __launch_bounds__(256) probe_rows_side(const uint8_t *buf, const uint8_t *side0, const uint8_t *side1,
                                                       int64_t rows, int64_t row_bytes, int64_t side_row_bytes,
                                                       int64_t pieces, int swizzle, uint32_t *sink)
{
    constexpr int BPL = 8, U = 16;
    const int lane = threadIdx.x;
    int64_t bx = blockIdx.x, by = blockIdx.y;
    if (swizzle & 1) {  // consecutive logical blocks on one XCD (blocks go to the 8 XCDs round-robin in launch order)
        const int64_t nx = gridDim.x, n = nx * (int64_t)gridDim.y;
        const int64_t l = by * nx + bx;
        const int64_t xcd = l % 8, slot = l / 8, per = n / 8, rem = n % 8;
        const int64_t j = xcd * per + (xcd < rem ? xcd : rem) + slot;
        bx = j % nx;
        by = j / nx;
    }
    int64_t piece = bx * blockDim.y + threadIdx.y;
    if (piece >= pieces) return;
    int64_t col = piece * (kWave * BPL);
    if (col + kWave * BPL > row_bytes) col = row_bytes - kWave * BPL;
    int64_t scol = piece * 64;
    if (scol + 64 > side_row_bytes) scol = side_row_bytes - 64;
    const uint8_t *base = buf + by * rows * row_bytes + col + lane * BPL;
    const int64_t soff = by * rows * side_row_bytes + (lane / 4) * side_row_bytes + scol + (lane % 4) * 16;
    uint32_t acc = 0;
    if (swizzle & 2) {
        // the q.K^T kernels' order of issue: the side loads of a chunk of 16 rows one chunk ahead, the code loads
        // in four steps of four rows, each step refilled right after it was consumed (loads pinned in place)
        typedef uint32_t u2 __attribute__((ext_vector_type(2)));
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        u2 v[U];
        u4 s0, s1;
        uint32_t dummy[4] = {1, 2, 3, 4};
        typedef float f4x __attribute__((ext_vector_type(4)));
        f4x macc = {0.f, 0.f, 0.f, 0.f};
        const int alu = swizzle >> 4;
        auto ld2 = [&](int64_t r) {
            const int64_t rr = r < rows ? r : rows - 1;
            if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const u2 *>(base + rr * row_bytes));
            else return *reinterpret_cast<const u2 *>(base + rr * row_bytes);
        };
        auto ldside = [&](int64_t r) {
            const int64_t rr = r < rows ? r : rows - 16;
            s0 = *reinterpret_cast<const u4 *>(side0 + soff + rr * side_row_bytes);
            s1 = *reinterpret_cast<const u4 *>(side1 + soff + rr * side_row_bytes);
        };
        ldside(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < U; i++) v[i] = ld2(i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
        for (int64_t r = 0; r < rows; r += U) {
            acc ^= s0.x ^ s0.y ^ s0.z ^ s0.w ^ s1.x ^ s1.y ^ s1.z ^ s1.w;
            __builtin_amdgcn_sched_barrier(0);
            ldside(r + U);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < 4; t++) {
#pragma unroll
                for (int i = 0; i < 4; i++) acc ^= v[4 * t + i].x ^ v[4 * t + i].y;
                // synthetic arithmetic on the loaded data: `alu` rounds of 8 vector-ALU operations and one
                // 4x4x4 matrix-core operation per step (the real kernels: about 100 and 16 per step)
                for (int a = 0; a < alu; a++) {
                    typedef short bf4 __attribute__((ext_vector_type(4)));
                    typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        dummy[i] = (dummy[i] ^ v[4 * t + i].x) * 0x9E3779B1u;
                        dummy[i] += v[4 * t + i].y >> 3;
                    }
                    const bf4 av = __builtin_bit_cast(bf4, make_uint2(dummy[0], dummy[1]));
                    const bf4 bv = __builtin_bit_cast(bf4, make_uint2(dummy[2] & 0x000f000fu, dummy[3] & 0x000f000fu));
                    macc = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av, bv, macc, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 4; i++) v[4 * t + i] = ld2(r + U + 4 * t + i);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        acc ^= dummy[0] ^ dummy[1] ^ dummy[2] ^ dummy[3] ^ __float_as_uint(macc[0] + macc[1] + macc[2] + macc[3]);
        if (acc == 0x12345678u) sink[0] = acc;
        return;
    }
    for (int64_t r = 0; r + U <= rows; r += U) {
        uint32_t v[U + 2];
        v[U] = probe_load<16, NT_SIDE>(side0 + soff + r * side_row_bytes);
        v[U + 1] = probe_load<16, NT_SIDE>(side1 + soff + r * side_row_bytes);
#pragma unroll
        for (int i = 0; i < U; i++) v[i] = probe_load<BPL, NT>(base + (r + i) * row_bytes);
#pragma unroll
        for (int i = 0; i < U + 2; i++) acc ^= v[i];
    }
    if (acc == 0x12345678u) sink[0] = acc;
}

template <int BPL, int U, bool NT>
static void probe_launch(int pattern, const uint8_t *buf, int64_t a0, int64_t a1, int64_t a2, int blocks_or_slices,
                         int waves, uint32_t *sink, hipStream_t st)
{
    if (pattern == 0) {
        hipLaunchKernelGGL((probe_slab<BPL, U, NT>), dim3((unsigned)blocks_or_slices), dim3(kWave, waves), 0, st, buf, a0, sink);
    } else {
        const int64_t pieces = (a1 + kWave * BPL - 1) / (kWave * BPL);
        hipLaunchKernelGGL((probe_rows<BPL, U, NT>), dim3((unsigned)((pieces + waves - 1) / waves), (unsigned)blocks_or_slices),
                           dim3(kWave, waves), 0, st, buf, a0, a1, pieces, sink);
    }
}

}  // namespace kvmix

using namespace kvmix;

// pattern 0: a0 = slab bytes per block (a multiple of 64 * bytes_per_lane * in_flight), count = blocks;
//            reads count * a0 bytes.
// pattern 1: a0 = rows per slice (a multiple of in_flight), a1 = row bytes (a multiple of
//            bytes_per_lane, at least 64 * bytes_per_lane), count = slices; reads count * a0 * a1 bytes
//            (the last piece of a row overlaps its neighbour when a1 is not a multiple of 64 * bytes_per_lane).
extern "C" int kvmix_probe_stream_read(const void *buf, int pattern, int64_t a0, int64_t a1, int count, int waves,
                                       int bytes_per_lane, int in_flight, int flags, void *sink,
                                       kvmix_stream_t stream)
{
    if (!buf || !sink) return KVMIX_ERR_NULL;
    if (pattern == 2) {
        // (count, a0 and waves are checked like those of patterns 0 and 1: the kernel redirects rows past the end
        // to rows - 1 and rows - 16, and the grid is ceil(pieces / waves))
        // a0 = rows (multiple of 16), a1 = row bytes (multiple of 8, at least 512); side arrays of a1 / 8 bytes per
        // row follow the code array in buf; in_flight and bytes_per_lane are ignored
        const int64_t side_row = a1 / 8;
        if (count <= 0 || a0 < 16 || waves < 1 || waves > 4) return KVMIX_ERR_SHAPE;
        if (a0 % 16 != 0 || a1 % 8 != 0 || a1 < 512 || side_row < 64 || side_row % 2 != 0 || count > 65535)
            return KVMIX_ERR_SHAPE;
        const uint8_t *b = (const uint8_t *)buf;
        const uint8_t *s0 = b + (int64_t)count * a0 * a1, *s1 = s0 + (int64_t)count * a0 * side_row;
        const int64_t pieces = (a1 + 511) / 512;
        const dim3 grid((unsigned)((pieces + waves - 1) / waves), (unsigned)count), block(kWave, waves);
        hipStream_t st = (hipStream_t)stream;
        const size_t lds = (size_t)(flags >> 8) * 1024;
        if (lds > 64 * 1024) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&probe_rows_side<false, false>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&probe_rows_side<true, false>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&probe_rows_side<false, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&probe_rows_side<true, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
        switch (flags & 3) {
        case 0: hipLaunchKernelGGL((probe_rows_side<false, false>), grid, block, lds, st, b, s0, s1, a0, a1, side_row, pieces, ((flags >> 2) & 3) | (((flags >> 4) & 15) << 4), (uint32_t *)sink); break;
        case 1: hipLaunchKernelGGL((probe_rows_side<true, false>), grid, block, lds, st, b, s0, s1, a0, a1, side_row, pieces, ((flags >> 2) & 3) | (((flags >> 4) & 15) << 4), (uint32_t *)sink); break;
        case 2: hipLaunchKernelGGL((probe_rows_side<false, true>), grid, block, lds, st, b, s0, s1, a0, a1, side_row, pieces, ((flags >> 2) & 3) | (((flags >> 4) & 15) << 4), (uint32_t *)sink); break;
        default: hipLaunchKernelGGL((probe_rows_side<true, true>), grid, block, lds, st, b, s0, s1, a0, a1, side_row, pieces, ((flags >> 2) & 3) | (((flags >> 4) & 15) << 4), (uint32_t *)sink); break;
        }
        return launch_status();
    }
    if ((pattern != 0 && pattern != 1) || count <= 0 || a0 <= 0 || waves <= 0 || waves > (pattern == 0 ? 16 : 4))
        return KVMIX_ERR_SHAPE;
    if (bytes_per_lane != 4 && bytes_per_lane != 8 && bytes_per_lane != 16) return KVMIX_ERR_UNSUPPORTED;
    if (in_flight != 4 && in_flight != 8 && in_flight != 16) return KVMIX_ERR_UNSUPPORTED;
    if (pattern == 0 && a0 % ((int64_t)kWave * bytes_per_lane * in_flight) != 0) return KVMIX_ERR_SHAPE;
    if (pattern == 1 && (a0 % in_flight != 0 || a1 % bytes_per_lane != 0 || a1 < kWave * bytes_per_lane || count > 65535))
        return KVMIX_ERR_SHAPE;
    const uint8_t *b = (const uint8_t *)buf;
    uint32_t *s = (uint32_t *)sink;
    hipStream_t st = (hipStream_t)stream;
#define KVMIX_PROBE(BPL_, U_)                                                                           \
    if (bytes_per_lane == BPL_ && in_flight == U_) {                                                    \
        if (flags & KVMIX_PROBE_NT)                                                               \
            probe_launch<BPL_, U_, true>(pattern, b, a0, a1, 0, count, waves, s, st);                   \
        else                                                                                            \
            probe_launch<BPL_, U_, false>(pattern, b, a0, a1, 0, count, waves, s, st);                  \
    }
    KVMIX_PROBE(4, 4) KVMIX_PROBE(4, 8) KVMIX_PROBE(4, 16)
    KVMIX_PROBE(8, 4) KVMIX_PROBE(8, 8) KVMIX_PROBE(8, 16)
    KVMIX_PROBE(16, 4) KVMIX_PROBE(16, 8) KVMIX_PROBE(16, 16)
#undef KVMIX_PROBE
    return launch_status();
}
