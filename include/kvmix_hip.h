/*
 * kvmix_hip.h -- C ABI of libkvmix_hip.so: the KVmix KV-cache hot path on gfx950.
 *
 * Plain C: device pointers, sizes, strides, a hipStream_t passed as void*.  No
 * torch types.  Every call validates its arguments on the host, enqueues its
 * kernels on `stream` and returns without synchronising.  Return value 0 is
 * success; negative values are the KVMIX_ERR_* codes below (kvmix_strerror()
 * gives the text, which for argument errors is the reference's TORCH_CHECK text).
 * Calls on different streams or from different threads are independent: the library's
 * only process-wide state is set up once per device under a lock or an atomic flag (a
 * kernel attribute, the address of kvmix_quantized_gemv_static's buffer) and never
 * changes afterwards.  The one exception is the content of that buffer, see there.
 *
 * Packed formats (`fmt`):
 *   KVMIX_FMT_REF    the reference's layout.  bits 1/2/4: 32/bits codes per
 *                    uint32, code i at bit i*bits.  bits 3: eleven codes per
 *                    uint32 -- ten 3-bit codes at bits 0..29 and an eleventh
 *                    clamped to 0..3 at bits 30..31 -- and the group is 11
 *                    (quant_cuda/csrc/quantization_cuda.cu:573-584,617-621).
 *   KVMIX_FMT_DENSE3 extension with no counterpart in the reference: 3-bit
 *                    codes as a little-endian bit stream, 32 codes in three
 *                    consecutive uint32, any group that is a multiple of 32.
 */
#ifndef KVMIX_HIP_H
#define KVMIX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KVMIX_OK 0
#define KVMIX_ERR_BITS (-1)        /* bits not in {1,2,3,4} */
#define KVMIX_ERR_GROUP3 (-2)      /* bits == 3 (reference format) needs group 11 */
#define KVMIX_ERR_STEPS_GROUP (-3) /* last dimension not divisible by the group */
#define KVMIX_ERR_STEPS_WORD (-4)  /* last dimension not divisible by codes per word */
#define KVMIX_ERR_HEADS (-5)       /* query heads not divisible by kv heads */
#define KVMIX_ERR_DTYPE (-6)       /* dtype tag not KVMIX_F16 / KVMIX_F32 */
#define KVMIX_ERR_NULL (-7)        /* null pointer with a non-empty problem */
#define KVMIX_ERR_SHAPE (-8)       /* negative size or a stride smaller than the row it spans */
#define KVMIX_ERR_UNSUPPORTED (-9) /* group / word combination the packed layout cannot express */
#define KVMIX_ERR_FORMAT (-10)     /* unknown fmt */
#define KVMIX_ERR_WORKSPACE (-11)  /* workspace smaller than kvmix_gemv_workspace_bytes() */
#define KVMIX_ERR_LAUNCH (-12)     /* hipGetLastError() after a launch was not hipSuccess */
#define KVMIX_ERR_STATIC_SCRATCH (-13) /* kvmix_quantized_gemv_static: problem beyond the built-in buffer */
#define KVMIX_ERR_STATIC_LOOKUP (-14)  /* kvmix_quantized_gemv_static: the built-in buffer's address could not be obtained */

#define KVMIX_F16 0
#define KVMIX_F32 1

#define KVMIX_FMT_REF 0
#define KVMIX_FMT_DENSE3 1
/* quantizer only, bits == 3: the reference's value-append kernel packs the eleventh code
 * of a word with the plain shift 10*3 after clamping to 0..7, so only its low two bits
 * survive (quantization_cuda.cu:282-289 with j == 10; the reference calls this branch
 * "placeholder logic", :463).  Kept so process_value_quantization_cuda stays literal. */
#define KVMIX_FMT_REF3_WRAP 2

/* how the returned scale is rounded (the codes always use (max-min)/qmax):
 *   KVMIX_SCALE_RECIPROCAL  (max-min) * fp32(1/qmax) -- what the reference's
 *        one-shot quantizer returns, because quantization_cuda.cu:711 divides a
 *        tensor by an integer scalar through ATen's CUDA kernel, which multiplies
 *        by the scalar's reciprocal;
 *   KVMIX_SCALE_DIVIDE      (max-min) / qmax -- what the reference's append
 *        kernels store (quantization_cuda.cu:49-51,149-151,234). */
#define KVMIX_SCALE_RECIPROCAL 0
#define KVMIX_SCALE_DIVIDE 1

typedef void *kvmix_stream_t; /* hipStream_t */

int kvmix_version(void);
const char *kvmix_strerror(int code);

/*
 * Group quantize + bit-pack along the last dimension.
 * Replaces quantize_pack_last_dim_cuda (quant_cuda/csrc/quantization_cuda.h:23-28,
 * quantization_cuda.cu:631-721) and, through the strides, the "new" half of
 * process_key_quantization_cuda / process_value_quantization_cuda
 * (quantization_cuda.h:4-21, quantization_cuda.cu:298-537).
 *
 *   x      [outer, inner, steps]  fp16 or fp32 (x_dtype), unit stride along steps,
 *          element strides x_outer_stride / x_inner_stride
 *   code   [outer, inner, steps/vpw] uint32 words, word strides code_*_stride
 *   scale, zero  [outer, inner, steps/group], same dtype as x, element strides sz_*_stride
 *
 * Keys (grouped per channel along tokens):  outer = B*Hkv, inner = D, steps = n.
 * Values (grouped per token along head_dim): outer = B*Hkv, inner = n, steps = D.
 * Writing at an offset into a larger pre-allocated cache is done by offsetting the
 * output pointers and passing the cache's strides.
 */
int kvmix_quant_pack_last_dim(const void *x, int x_dtype, int64_t outer, int64_t inner, int64_t steps,
                              int64_t x_outer_stride, int64_t x_inner_stride, int group, int bits,
                              int fmt, int scale_mode, uint32_t *code, int64_t code_outer_stride,
                              int64_t code_inner_stride, void *scale, void *zero,
                              int64_t sz_outer_stride, int64_t sz_inner_stride, kvmix_stream_t stream);

/*
 * Key quantizer that reads the token-major fp16 tail directly and writes the
 * channel-major packed layout, i.e. quantize_pack_last_dim_cuda applied to
 * `tail[:, :, :n, :].transpose(2, 3).contiguous()` without materialising the
 * transpose (the call site is models/modeling_llama_KVmix.py:131-133).
 *
 *   k      [outer, n, D] fp16, unit stride along D, element strides k_outer_stride / k_token_stride
 *   code   [outer, D, n/vpw]; scale, zero [outer, D, n/group] fp16
 * group must be 32 (bits 1/2/4, or 3 with KVMIX_FMT_DENSE3) or 11 (bits 3, KVMIX_FMT_REF).
 */
int kvmix_quant_pack_key_tokens(const void *k, int64_t outer, int64_t n, int64_t D,
                                int64_t k_outer_stride, int64_t k_token_stride, int group, int bits,
                                int fmt, int scale_mode, uint32_t *code, int64_t code_outer_stride,
                                int64_t code_inner_stride, void *scale, void *zero,
                                int64_t sz_outer_stride, int64_t sz_inner_stride, kvmix_stream_t stream);

/*
 * Both flushes of one decode step in a single launch: the key tail through
 * kvmix_quant_pack_key_tokens and the value tail through kvmix_quant_pack_last_dim
 * (fp16 input), same arguments, same results bit for bit.  The reference issues the two
 * quantizers back to back from models/modeling_llama_KVmix.py:119-160; each is a small,
 * latency-bound launch, so one launch for both costs about what either costs alone.
 * Both halves are validated before anything is launched.  When a half is empty or the
 * value half is not the group-32 fp16 case, the call falls back to separate launches.
 */
typedef struct kvmix_key_flush {
    const void *k;              /* [outer, n, D] fp16 */
    int64_t outer, n, D;
    int64_t k_outer_stride, k_token_stride;
    int group, bits, fmt, scale_mode;
    uint32_t *code;             /* [outer, D, n/vpw] */
    int64_t code_outer_stride, code_inner_stride;
    void *scale, *zero;         /* [outer, D, n/group] fp16 */
    int64_t sz_outer_stride, sz_inner_stride;
} kvmix_key_flush_t;

typedef struct kvmix_value_flush {
    const void *x;              /* [outer, inner, steps] fp16 */
    int64_t outer, inner, steps;
    int64_t x_outer_stride, x_inner_stride;
    int group, bits, fmt, scale_mode;
    uint32_t *code;             /* [outer, inner, steps/vpw] */
    int64_t code_outer_stride, code_inner_stride;
    void *scale, *zero;         /* [outer, inner, steps/group] fp16 */
    int64_t sz_outer_stride, sz_inner_stride;
} kvmix_value_flush_t;

int kvmix_quant_pack_kv_flush(const kvmix_key_flush_t *key, const kvmix_value_flush_t *value,
                              kvmix_stream_t stream);

/*
 * The flushes of several layers (or caches) at once: `count` (key, value) pairs as arrays of descriptor pointers,
 * eight pairs to a launch, the results those of kvmix_quant_pack_kv_flush on each pair, bit for bit.  In the
 * reference every layer flushes inside its own forward (models/modeling_llama_KVmix.py:119-167), but what a layer
 * flushes in a decode step are the OLDEST tokens of its fp16 tail (`key_states_full[:, :, :to_quantize_length]`,
 * lines 122-127, 152-156) -- tokens of earlier steps -- and how many follows from the tail's length alone: the
 * flushes of all layers of a step can be issued together before its first layer runs.  A flush is a latency-bound
 * launch of about 10 us whatever its size; eight layers in one launch take about as long as two alone.
 * All pairs are validated before anything is launched; a pair that kvmix_quant_pack_kv_flush would run as separate
 * launches (an empty half, a value half that is not the group-32 fp16 case) is run so here too.
 */
int kvmix_quant_pack_kv_flush_batch(const kvmix_key_flush_t *const *keys, const kvmix_value_flush_t *const *values,
                                    int count, kvmix_stream_t stream);

/*
 * Fused dequantize + matrix-vector product over the packed cache.
 * Replaces quantized_gemm (quant_cuda/csrc/dequantization_gemv_cuda.h:22-29,
 * dequantization_gemv_cuda.cu:7-248):
 *
 *   out[s, m, n] = fp16( sum_k fp32(x[s, m, k]) *
 *                        ( fp32(scale[s', k, grp(n)]) * code[s', k, n] + fp32(zero[s', k, grp(n)]) ) )
 *   s' = s / heads_per_kv,   grp(n) = n / group,   fp32 accumulation.
 *
 *   x      [samples, M, K] fp16     (samples = B * query heads)
 *   code   [samples/heads_per_kv, K, N/vpw] uint32, read in the stored layout (no transpose copy)
 *   scale, zero [samples/heads_per_kv, K, N/group] fp16
 *   out    [samples, M, N] fp16
 * All strides are in elements of the respective array; rows are unit-stride.
 *
 * q.K^T is the case K = head_dim, N = quantized tokens (code = key codes [.., D, Tq/vpw]);
 * p.V is the case K = quantized tokens, N = head_dim (code = value codes [.., Tq, D/vpw]).
 * The reference kernel only produces row m = 0 (it ignores blockIdx.z); rows m >= 1 are
 * computed here with the same formula.
 *
 * workspace: device scratch of at least kvmix_gemv_workspace_bytes() bytes for the same
 * sizes (may be NULL when that returns 0).  Its contents are undefined afterwards.
 */
size_t kvmix_gemv_workspace_bytes(int64_t samples, int64_t M, int64_t K, int64_t N);

int kvmix_quantized_gemv(int group, const void *x, int64_t x_batch_stride, int64_t x_row_stride,
                         const uint32_t *code, int64_t code_batch_stride, int64_t code_row_stride,
                         const void *scale, const void *zero, int64_t sz_batch_stride,
                         int64_t sz_row_stride, int bits, int fmt, int64_t samples, int heads_per_kv,
                         int64_t M, int64_t K, int64_t N, void *out, int64_t out_batch_stride,
                         int64_t out_row_stride, void *workspace, size_t workspace_bytes,
                         kvmix_stream_t stream);

/*
 * Which kernel a kvmix_quantized_gemv call of these sizes is dispatched to, without launching
 * anything and without a GPU (no counterpart in the reference; for tests that pin the dispatch of
 * the benchmark shapes, and for reading profiles).  code_row_stride / sz_row_stride as in the call
 * (words / elements between two rows of one slice).  kernel: the kernel's name with its template
 * arguments; grid, block, lds_bytes: its launch geometry; splits: blocks along K of a p.V kernel
 * (more than one brings the reduction launch) or tiles a q.K^T wave walks; ksplit: waves that
 * share a q.K^T tile; launches: kernel launches of the call (0: nothing to do).
 * Returns the code kvmix_quantized_gemv would return for these sizes.
 */
typedef struct kvmix_gemv_plan {
    char kernel[64];
    unsigned grid[3], block[3];
    uint64_t lds_bytes;
    int splits, ksplit, launches;
} kvmix_gemv_plan_t;
int kvmix_quantized_gemv_plan(int group, int bits, int fmt, int64_t samples, int heads_per_kv, int64_t M,
                              int64_t K, int64_t N, int64_t code_row_stride, int64_t sz_row_stride,
                              kvmix_gemv_plan_t *plan);

/*
 * kvmix_quantized_gemv for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments minus the workspace, same kernels, same results bit for bit: the split-K partial
 * sums go to a buffer of KVMIX_GEMV_STATIC_SCRATCH_BYTES that is part of the library's device
 * image (every device the library runs on holds it until the process ends).  The call allocates
 * and frees nothing.  The arguments are checked as in kvmix_quantized_gemv (same codes); then a problem whose
 * kvmix_gemv_workspace_bytes() exceeds the buffer is refused with KVMIX_ERR_STATIC_SCRATCH before anything is
 * launched.  Only a call whose plan splits K looks the buffer up (KVMIX_ERR_STATIC_LOOKUP if the device does not
 * give its address).  The buffer covers every q.K^T product
 * and every p.V product with N <= 128 (at most 1.06 MiB of partial sums, reached near 120 output
 * rows of 128k tokens; launches of 1024 and more output rows need none); with N = 256 a few shapes
 * around 120 output rows of 64k and more tokens need up to 2.11 MiB and are refused.
 * All calls on one device share the buffer: two calls that overlap on one device (different
 * streams, or threads) race on it; calls on one stream are ordered and safe.  Nothing in the
 * buffer has to start at zero (every partial sum is written before it is read).  The first call
 * on a device looks the buffer's address up (hipGetSymbolAddress): make it outside a capture.
 */
#define KVMIX_GEMV_STATIC_SCRATCH_BYTES (2u << 20)
int kvmix_quantized_gemv_static(int group, const void *x, int64_t x_batch_stride, int64_t x_row_stride,
                                const uint32_t *code, int64_t code_batch_stride, int64_t code_row_stride,
                                const void *scale, const void *zero, int64_t sz_batch_stride,
                                int64_t sz_row_stride, int bits, int fmt, int64_t samples, int heads_per_kv,
                                int64_t M, int64_t K, int64_t N, void *out, int64_t out_batch_stride,
                                int64_t out_row_stride, kvmix_stream_t stream);

/*
 * One decode step of attention over the packed cache and its fp16 residual tails: what
 * LlamaAttention_KVmix.forward does between RoPE and the output projection once the cache is up to
 * date (models/modeling_llama_KVmix.py:68-75,180-211; Mistral twin: models/modeling_mistral_KVmix.py
 * :114-121,217-262), on the caller's stream:
 *
 *   logits = cat(fp16 q.K^T over the quantized keys, fp16 q.K_tail^T) / sqrt(D)  (+ mask, clamped to
 *            the lowest finite fp32), softmax in fp32, probabilities rounded to fp16;
 *   out    = fp16(p.V over the quantized values) + fp16(p_tail . V_tail)
 *
 * The two quantized products are kvmix_quantized_gemv launches; the tail products and the softmax
 * are two small kernels, so a step is four or five launches instead of the reference's dozen.
 *
 *   q        [samples, D] fp16 (samples = B * query heads, one row per head), row stride q_stride
 *   k_..., v_...  the packed operands exactly as kvmix_quantized_gemv takes them (keys [.., D, Tk/vpw],
 *            values [.., Tv, D/vpw]); k_tokens / v_tokens = Tk / Tv may be 0
 *   k_tail, v_tail  [samples / heads_per_kv, slots, D] fp16 windows of the residual tails, of which
 *            the first *_tail_len slots hold tokens.  If *_tail_len_dev is not NULL the length is
 *            read from that device location when the kernel runs (a step replayed from a captured
 *            graph) and *_tail_len is ignored.
 *   mask     optional fp32 [samples / heads, width] added to the scaled logits (row = batch element)
 *   probs    [samples, width] fp16, width = max(k_tokens + k_tail_slots, v_tokens + v_tail_slots):
 *            out: the probabilities (position i of a row is token i; slots past a tail's length are 0)
 *   out      [samples, D] fp16
 * With host-side lengths, k_tokens + k_tail_len must equal v_tokens + v_tail_len.
 * workspace: at least kvmix_decode_attention_workspace_bytes() bytes of device scratch.
 */
typedef struct kvmix_decode_attn {
    const void *q;              /* [samples, D] fp16 */
    int64_t q_stride;           /* elements between two rows of q */
    const uint32_t *k_code;     /* [samples / heads_per_kv, D, k_tokens / vpw] */
    int64_t k_code_batch_stride, k_code_row_stride;
    const void *k_scale, *k_zero; /* [samples / heads_per_kv, D, k_tokens / k_group] fp16 */
    int64_t k_sz_batch_stride, k_sz_row_stride;
    int k_bits, k_fmt, k_group;
    int64_t k_tokens;           /* quantized key tokens (0: none, the k_ pointers are not read) */
    const uint32_t *v_code;     /* [samples / heads_per_kv, v_tokens, D / vpw] */
    int64_t v_code_batch_stride, v_code_row_stride;
    const void *v_scale, *v_zero; /* [samples / heads_per_kv, v_tokens, D / v_group] fp16 */
    int64_t v_sz_batch_stride, v_sz_row_stride;
    int v_bits, v_fmt, v_group;
    int64_t v_tokens;           /* quantized value tokens */
    const void *k_tail;         /* [samples / heads_per_kv, k_tail_slots, D] fp16 */
    int64_t k_tail_batch_stride, k_tail_token_stride, k_tail_slots, k_tail_len;
    const int64_t *k_tail_len_dev; /* NULL, or where the live length is read when the kernels run */
    const void *v_tail;         /* [samples / heads_per_kv, v_tail_slots, D] fp16 */
    int64_t v_tail_batch_stride, v_tail_token_stride, v_tail_slots, v_tail_len;
    const int64_t *v_tail_len_dev;
    const float *mask;          /* NULL, or [samples / heads, width] fp32 */
    int64_t mask_stride;
    int64_t samples;            /* batch * query heads */
    int heads;                  /* query heads per batch element (the mask is per batch element) */
    int heads_per_kv;           /* query heads that share one kv head */
    int64_t D;                  /* head dimension, a multiple of 8 */
    void *probs;                /* [samples, width] fp16, out */
    int64_t probs_stride;
    void *out;                  /* [samples, D] fp16, out */
    int64_t out_stride;
} kvmix_decode_attn_t;

size_t kvmix_decode_attention_workspace_bytes(const kvmix_decode_attn_t *step);
int kvmix_decode_attention(const kvmix_decode_attn_t *step, void *workspace, size_t workspace_bytes,
                           kvmix_stream_t stream);

/*
 * The same step in one pass over the positions: every block computes the logits of one slab of
 * positions, keeps exp(logit - slab maximum) on chip and multiplies it into the values of the same
 * positions; a second small kernel merges the slabs (two launches, no logits or probabilities in
 * memory).  It takes the same descriptor; `probs` and `probs_stride` are ignored (no probabilities
 * are returned).  It follows models/modeling_llama_KVmix.py:68-75,180-211 up to the softmax (fp16
 * logits, 1/sqrt(D), mask, clamp) but not the reference's roundings after it: probabilities are not
 * rounded to fp16 and the quantized and tail halves of the output are not rounded separately, so the
 * result differs from kvmix_decode_attention's by up to about 2^-10 of the largest value magnitude.
 * Steps whose keys (1, 2 or 4 bits, or the reference's 3-bit words) and values are both quantized over at least
 * one tile of 1024 positions (1408 with those words), with dense value rows, run the positions quantized on both
 * sides on the matrix cores -- a wave per tile, or the four waves of a block per tile when the step has few tiles:
 * logits, slab softmax and the product with the values of the same positions -- and the rest (the fp16 tails, and
 * positions only one side has quantized) as trailing blocks of the same launch (two launches); everything else as
 * described above.  kvmix_decode_attention_fused_plan tells which.
 *
 * Supported (kvmix_decode_attention_fused_supported returns 1, else the call returns
 * KVMIX_ERR_UNSUPPORTED): D = 128; keys 1/2/4-bit or dense 3-bit in groups of 32 or the reference's 3-bit words;
 * values 1/2/4-bit or dense 3-bit in groups of 32; 1, 2, 4 or 8 query heads per kv head.
 * workspace: at least kvmix_decode_attention_fused_workspace_bytes() bytes of device scratch.
 */
int kvmix_decode_attention_fused_supported(const kvmix_decode_attn_t *step);
size_t kvmix_decode_attention_fused_workspace_bytes(const kvmix_decode_attn_t *step);
int kvmix_decode_attention_fused(const kvmix_decode_attn_t *step, void *workspace, size_t workspace_bytes,
                                 kvmix_stream_t stream);

/*
 * How kvmix_decode_attention_fused would run a step of these sizes: which positions go through the matrix-core
 * kernel, how the rest is cut into slabs, and the launches' geometry.  No counterpart in the reference; it needs no
 * GPU and launches nothing (for the dispatch tests, for callers that choose between the two step forms, and for
 * reading profiles).  Only the sizes, strides, formats and the mask / device-length pointers' being NULL or not are
 * read from `step`; the operand pointers may be NULL.  Returns the code kvmix_decode_attention_fused would return
 * for the same sizes (KVMIX_ERR_NULL and KVMIX_ERR_WORKSPACE aside).
 */
typedef struct kvmix_attn_plan {
    int matrix;              /* 1: the positions [0, slab_begin) run on the matrix cores, one wave per tile */
    int recommended;         /* 1: at these sizes the single pass is the faster form (measured), 0: the four launches
                              * of kvmix_decode_attention are */
    int launches;            /* kernel launches of the step, the merge included */
    int64_t matrix_tiles;    /* tiles of 1024 positions (1408 with the reference's 3-bit keys) per query head; 0
                              * without the matrix-core kernel */
    int matrix_tile_waves;   /* waves that share a tile: 1, or 4 for steps with few (query head, tile) pairs (each wave
                              * then finishes a quarter of the tile as a slab of its own); 0 without the kernel */
    int64_t slab_positions;  /* positions per vector-ALU slab */
    int64_t slab_begin;      /* first position those slabs cover */
    int64_t slabs;           /* their number per query head */
    int64_t slab_blocks;     /* their blocks: trailing blocks of the matrix-core launch, or a launch of their own */
    unsigned matrix_grid[3], matrix_block[3];   /* the matrix-core launch, the slabs' blocks included */
} kvmix_attn_plan_t;
int kvmix_decode_attention_fused_plan(const kvmix_decode_attn_t *step, kvmix_attn_plan_t *plan);

/*
 * The tail append of a decode step fused with the rotary embedding before it: what
 * LlamaAttention_KVmix.forward does at models/modeling_llama_KVmix.py:102-112 for one new token
 * (apply_rotary_pos_emb on q and k, then torch.cat of k and v onto the fp16 tails), in one launch
 * and without re-allocating the tails.
 *
 *   qkv     [batch, heads + 2 * kv_heads, D] fp16: the query heads, then the key heads, then the
 *           value heads of the new token (the output of a fused q/k/v projection)
 *   cos, sin [D] fp16 for the token's position (rotate-half convention: both halves of D hold the
 *           same angles)
 *   q_out   [batch, heads, D] fp16: the rotated queries
 *   k_tail, v_tail [batch, kv_heads, slots, D] fp16 windows of the cache tails; the rotated key
 *           heads / the value heads are written to slot k_slot / v_slot, read from *_slot_dev when
 *           that is not NULL (a step replayed from a captured graph).  A device-side slot outside
 *           the window writes nothing.
 * The rotation is evaluated as the fp16 tensor expression x * cos + rotate_half(x) * sin evaluates
 * it (products and sum each rounded to fp16), so it is bit-identical to that composition.
 * D must be a multiple of 16.
 */
typedef struct kvmix_rope_append {
    const void *qkv;
    int64_t qkv_batch_stride;
    const void *cos, *sin;
    void *q_out;
    int64_t q_batch_stride;
    void *k_tail;
    int64_t k_tail_batch_stride, k_tail_head_stride, k_tail_token_stride, k_tail_slots, k_slot;
    const int64_t *k_slot_dev;
    void *v_tail;
    int64_t v_tail_batch_stride, v_tail_head_stride, v_tail_token_stride, v_tail_slots, v_slot;
    const int64_t *v_slot_dev;
    int64_t batch;
    int heads, kv_heads;
    int64_t D;
} kvmix_rope_append_t;

int kvmix_rope_append(const kvmix_rope_append_t *step, kvmix_stream_t stream);

/*
 * Measurement support, no counterpart in the reference and not called by any operator: a kernel
 * that only reads, in the access patterns of the GEMV kernels, to establish what streaming rate
 * the GPU reaches without arithmetic (the ceiling the GEMV figures are compared with), and how
 * that rate falls when arithmetic is added to the same loop.
 *   pattern 0 ("slab", the p.V pattern): `count` blocks of `waves` waves (1..16), block i reads the
 *       a0 contiguous bytes at buf + i * a0 in chunks of 64 * bytes_per_lane * in_flight bytes
 *       handed round-robin to its waves; a0 must be a multiple of the chunk.  Reads count * a0 bytes.
 *   pattern 1 ("rows", the q.K^T pattern): buf is [count slices][a0 rows][a1 row bytes]; a wave
 *       owns a column piece of 64 * bytes_per_lane bytes and walks it down the a0 rows of its
 *       slice, in_flight rows at a time; `waves` (1..4) neighbouring pieces per block.
 *       Reads count * a0 * a1 bytes.
 *   pattern 2 ("rows and side arrays", what a 4-bit q.K^T launch reads): pattern 1 with 8 bytes per
 *       lane and 16 rows in flight (bytes_per_lane and in_flight are ignored), plus per 16 rows one
 *       16-byte load per lane from each of two side arrays [count][a0][a1 / 8] that follow the code
 *       array in buf (64-byte pieces per row and wave, as the scales and zeros are read).
 *       Reads count * a0 * a1 * 1.25 bytes.
 * count >= 1, a0 >= 1 (pattern 2: >= 16), waves >= 1, else KVMIX_ERR_SHAPE.
 * bytes_per_lane in {4, 8, 16}, in_flight in {4, 8, 16}; sink: 4 writable bytes (never written
 * for a buffer that does not xor to one particular pattern).
 * flags: KVMIX_PROBE_NT non-temporal loads (pattern 2: of the code array); pattern 2 only:
 * KVMIX_PROBE_NT_SIDE the side arrays too (in the burst order only: the rotating order always reads them
 * with plain loads, as the GEMV kernels do), KVMIX_PROBE_XCD_ORDER consecutive logical blocks on one XCD,
 * KVMIX_PROBE_ROTATING the kernels' order of issue (four rows consumed, four refilled) instead of
 * 18 loads in a burst, KVMIX_PROBE_ALU(n) n = 0..15 rounds of synthetic arithmetic per four rows (a
 * round: 16 integer vector operations, four of them 32-bit multiplies, and one 4x4x4 matrix-core
 * operation), KVMIX_PROBE_LDS_KIB(k) k KiB of unused LDS per block to hold the resident waves down.
 */
#define KVMIX_PROBE_NT 1
#define KVMIX_PROBE_NT_SIDE 2
#define KVMIX_PROBE_XCD_ORDER 4
#define KVMIX_PROBE_ROTATING 8
#define KVMIX_PROBE_ALU(n) (((n) & 15) << 4)
#define KVMIX_PROBE_LDS_KIB(k) (((k) & 255) << 8)
int kvmix_probe_stream_read(const void *buf, int pattern, int64_t a0, int64_t a1, int count, int waves,
                            int bytes_per_lane, int in_flight, int flags, void *sink, kvmix_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* KVMIX_HIP_H */
