/*
 * tllm_hip.h -- C ABI of libtllm_hip.so: the gpt-oss layer kernels for MI355X (gfx950).
 *
 * Every entry point takes raw device pointers and sizes, launches on the HIP
 * stream it is given (a hipStream_t passed as void*; NULL = the null stream),
 * never allocates, never synchronises and never throws. It returns 0 on
 * success or a negative TLLM_E_* code; tllm_last_error() then holds a
 * thread-local message. All tensors are dense row-major unless a stride is
 * part of the signature. bf16 is the IEEE bfloat16 bit pattern (uint16_t).
 *
 * The "replaces" notes name the reference call each entry point stands in for
 * (paths relative to the reference checkout, tritonllm/gpt_oss/triton/).
 */
#ifndef TLLM_HIP_H
#define TLLM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TLLM_ABI_VERSION 1

enum {
  TLLM_OK = 0,
  TLLM_E_ARG = -1,      /* null pointer, negative size, bad flag            */
  TLLM_E_SHAPE = -2,    /* shape the kernels do not support                  */
  TLLM_E_ALIGN = -3,    /* pointer / stride not aligned as required          */
  TLLM_E_LAUNCH = -4    /* hipLaunchKernel reported an error                 */
};

#define TLLM_MAX_ROPE_FREQS 128

/* YaRN rotary parameters, built on the host from the restated formula of
 * model.py:267-305 (RotaryEmbedding._compute_concentration_and_inv_freq):
 * inv_freq[i], i < n_freq = head_dim/2, and the concentration that scales
 * both cos and sin. */
typedef struct TllmYarn {
  float inv_freq[TLLM_MAX_ROPE_FREQS];
  float concentration;
  int32_t n_freq;
} TllmYarn;

/* Where a rotary kernel takes its angles from.
 *   position of row r:  positions ? positions[r]
 *                                 : (r % tokens_per_batch) + (offset ? offset[0] : 0)
 *   then wrapped modulo max_ctx (triton_kernels.py:57-59, 1066-1070).
 *   cos/sin:  yarn != NULL  -> computed in registers:
 *                              angle = float(pos) * inv_freq[i] (one fp32 product),
 *                              cos(angle) * concentration, sin(angle) * concentration
 *             else          -> read from the fp32 tables cos_table/sin_table
 *                              [max_ctx, head_dim/2] (row stride table_row_stride floats)
 * positions / offset are DEVICE pointers (int64), so a captured graph can
 * replay with new positions. */
typedef struct TllmRope {
  const TllmYarn* yarn;          /* host pointer, copied into the launch          */
  const float* cos_table;        /* device, used when yarn == NULL                */
  const float* sin_table;        /* device, used when yarn == NULL                */
  int64_t table_row_stride;      /* floats between table rows                     */
  const int64_t* positions;      /* device [rows] or NULL                         */
  const int64_t* offset;         /* device (1,) or NULL                           */
  int64_t tokens_per_batch;      /* T of a [B,T,...] input; >= 1                  */
  int64_t max_ctx;               /* positions wrap modulo this; >= 1              */
} TllmRope;

int tllm_abi_version(void);
const char* tllm_last_error(void);

/* y[r,:] = x[r,:] * rsqrt(mean(x[r,:]^2) + eps) * scale[:], fp32 inside, one
 * round-to-nearest-even to bf16 on store. out may alias x.
 * replaces rmsnorm_forward(x, scale, eps, out) triton_kernels.py:28-35
 * (module RMSNorm.forward, model.py:55-68). scale is fp32 or bf16 [hidden]. */
int tllm_rmsnorm_bf16(const void* x, const void* scale, int scale_is_bf16, void* out,
                      int64_t rows, int64_t hidden, float eps, void* stream);

/* Token gather and RMSNorm of the gathered rows in one launch: x_out[t, :] = table[ids[t], :] (bit-exact; the hidden
 * state, torch.nn.Embedding at model.py:906-908, 920) and out[t, :] = RMSNorm(x_out[t, :]) (the first block's norm,
 * model.py:476; same arithmetic as tllm_rmsnorm_bf16, so the results are identical to the two calls). ids int32 or
 * int64; an id outside [0, vocab) gives a zero row in both outputs and sets *oob_flag (device int, may be NULL) to 1.
 * hidden must be a multiple of 8 up to 8192, x_out and out different buffers. No counterpart in the reference (two
 * launches there). */
int tllm_embed_rmsnorm_bf16(const void* table, const void* ids, int ids_is_i64, void* x_out, const void* scale,
                            int scale_is_bf16, void* out, int64_t n_tokens, int64_t hidden, int64_t vocab, float eps,
                            int* oob_flag, void* stream);

/* out[t,:] = table[ids[t],:], bit-exact row gather.
 * replaces torch.nn.Embedding forward, model.py:906-908, 920.
 * ids are int32 (the reference's token tensors, model.py:1170) or int64.
 * An id outside [0, vocab) writes a zero row and, if oob_flag != NULL, stores
 * 1 into *oob_flag (device int32) -- no fault, no host sync. */
int tllm_embedding_bf16(const void* table, const void* ids, int ids_is_i64, void* out,
                        int64_t n_tokens, int64_t hidden, int64_t vocab, int32_t* oob_flag,
                        void* stream);

/* Clamped SwiGLU: gate g and linear l are the even/odd columns of x
 * (interleaved != 0) or its first/second half (interleaved == 0);
 * if has_limit: g = min(g, limit), l = clamp(l, -limit, limit);
 * out = g * sigmoid(alpha * g) * (l + 1), fp32 inside, one RNE to bf16.
 * x is [rows, 2*n_out] with row stride x_row_stride elements (last stride 1),
 * out is [rows, n_out] dense.
 * replaces swiglu(x, alpha, limit, interleaved) moe.py:25-33 and
 * triton_kernels/swiglu.py:85-100 (swiglu / swiglu_torch). */
int tllm_swiglu_bf16(const void* x, void* out, int64_t rows, int64_t n_out, int64_t x_row_stride,
                     float alpha, float limit, int has_limit, int interleaved, void* stream);

/* cos[p - start, i] = cos(float(p) * inv_freq[i]) * concentration (and sin),
 * p in [start, start + n_pos): the tables RotaryEmbedding._compute_cos_sin
 * builds (model.py:307-313), computed with the same device routine the fused
 * kernels use in registers. cos/sin are fp32 [n_pos, n_freq] dense. */
int tllm_yarn_table_f32(float* cos, float* sin, int64_t start, int64_t n_pos,
                        const TllmYarn* yarn, void* stream);

/* In-place half-split rotary on q [rows, n_q_heads, head_dim] and
 * k [rows, n_kv_heads, head_dim] (bf16, dense): for d < head_dim/2
 *   o[d]      = x[d] * cos - x[d + hd/2] * sin
 *   o[d+hd/2] = x[d + hd/2] * cos + x[d] * sin      (fp32, one RNE per output).
 * replaces rope_forward(query, key, sin, cos, max_context_length, offset)
 * triton_kernels.py:90-108 (RotaryEmbedding.forward, model.py:329-337).
 * k may be NULL (n_kv_heads ignored). */
int tllm_rope_bf16(void* q, void* k, int64_t rows, int n_q_heads, int n_kv_heads, int head_dim,
                   const TllmRope* rope, void* stream);

/* Fused QKV projection + bias (+ rotary on q and k when rope != NULL).
 *   qkv[r, :] = x[r, :] . W^T + b       (bf16 in, fp32 accumulate)
 *   columns [0, n_q*hd) -> q, next n_kv*hd -> k, last n_kv*hd -> v;
 *   rotary is applied to the fp32 accumulator of q and k, then one RNE to bf16.
 * x [rows, hidden] dense; W [(n_q + 2 n_kv) * hd, hidden] dense; b bf16 or NULL.
 * Row r of q/k/v is written at q + r*q_row_stride, k + r*k_row_stride
 * + slot*kv_slot_stride, v likewise, strides in elements, where
 * slot = (kv_slot_stride != 0 && rope && rope->offset) ? rope->offset[0] : 0
 * is read on the device: with k/v pointing at a [B, n_ctx, n_kv, hd] cache,
 * k_row_stride = n_ctx*n_kv*hd and kv_slot_stride = n_kv*hd this is the
 * reference's write of the new token into the KV cache.
 *
 * _decode: weight-streaming kernels for few rows (any rows accepted). At the
 *   gpt-oss shape (hidden 2880, head_dim 64) the weight is read once whatever
 *   the row count; other shapes (hidden % 32 == 0, head_dim % 16 == 0: an MFMA
 *   kernel, once per 16 rows; anything else: a scalar kernel) are generic as
 *   the reference's kernel is. Needs no workspace: unlike the
 *   reference's split-K pair of launches (partials at triton_kernels.py:1200)
 *   the K reduction stays inside a workgroup.
 *   replaces qkv_rope_cache_decode_forward triton_kernels.py:1109-1255 and,
 *   with rope == NULL, qkv_decode_forward triton_kernels.py:615-659.
 * _prefill: LDS-staged bf16 MFMA GEMM with the bias + rotary epilogue.
 *   replaces F.linear + split + 3x contiguous + rope_forward,
 *   model.py:506-522. */
int tllm_qkv_rope_decode_bf16(const void* x, const void* W, const void* b,
                              void* q, void* k, void* v,
                              int64_t q_row_stride, int64_t k_row_stride, int64_t v_row_stride,
                              int64_t kv_slot_stride,
                              int64_t rows, int64_t hidden, int n_q_heads, int n_kv_heads, int head_dim,
                              const TllmRope* rope, void* stream);

/* tllm_rmsnorm_bf16 followed by tllm_qkv_rope_decode_bf16 in one launch: x is the raw
 * hidden state, the kernel normalises it (fp32, one RNE to bf16 -- the operand the two
 * separate calls would pass between them) while the weight streams in.
 * replaces the pair AttentionBlock.forward issues per decode step, model.py:476 + 489-503.
 * Exists for hidden == 2880, head_dim == 64 (TLLM_E_SHAPE otherwise). Up to 16 rows per
 * workgroup the norm runs inside the weight-streaming kernels; with more rows the call is
 * the two launches it replaces (RMSNorm into a caller-invisible buffer is not possible
 * without allocating, so more than 16 rows return TLLM_E_SHAPE: issue the two calls). */
int tllm_norm_qkv_rope_decode_bf16(const void* x, const void* norm_scale, int scale_is_bf16, float eps,
                                   const void* W, const void* b, void* q, void* k, void* v,
                                   int64_t q_row_stride, int64_t k_row_stride, int64_t v_row_stride,
                                   int64_t kv_slot_stride,
                                   int64_t rows, int64_t hidden, int n_q_heads, int n_kv_heads, int head_dim,
                                   const TllmRope* rope, void* stream);

/* Diagnostic of the fused-norm decode kernels: inside them the wavefronts of a workgroup wait for one another's
 * partial sums with a bounded poll. *expired becomes 1 if any such wait ever ran out on the current device since the
 * library was loaded (the launch then finished with wrong sums instead of hanging), else 0. Synchronises the device.
 * No counterpart in the reference. */
int tllm_qkv_decode_wait_expired(int32_t* expired);

/* The first layer of a decode step in one launch: token-embedding gather (torch.nn.Embedding, model.py:906-908, 920)
 * feeding the first block's RMSNorm + QKV + bias + rotary (model.py:476, 489-503). x_out[r, :] = table[ids[r], :]
 * (bit-exact, [rows, hidden] dense: the residual stream the following layers read), and q / k / v as
 * tllm_norm_qkv_rope_decode_bf16 computes them from x_out. ids: int32 or int64 [rows]; an id outside [0, vocab)
 * gives a zero row in x_out (and q / k / v computed from it) and sets *oob_flag (may be NULL), as tllm_embedding_bf16 does.
 * w_scale: NULL for a bf16 W, else W holds fp8 bytes as in tllm_qkv_rope_decode_w8_bf16. norm_scale must not be
 * NULL; hidden 2880, head_dim 64, rows <= 16 (larger batches: gather, then the QKV entry point), table smaller than
 * 4 GiB (the kernel addresses its rows with 32-bit byte offsets; TLLM_E_SHAPE otherwise). */
int tllm_embed_norm_qkv_rope_decode_bf16(const void* ids, int ids_is_i64, const void* table, int64_t vocab, void* x_out,
                                         int32_t* oob_flag, const void* norm_scale, int scale_is_bf16, float eps,
                                         const void* W, const float* w_scale, const void* b, void* q, void* k, void* v,
                                         int64_t q_row_stride, int64_t k_row_stride, int64_t v_row_stride,
                                         int64_t kv_slot_stride, int64_t rows, int64_t hidden, int n_q_heads, int n_kv_heads,
                                         int head_dim, const TllmRope* rope, void* stream);

/* The decode projection with an fp8 weight: W8 is [n_heads*64, hidden] OCP e4m3 bytes, w_scale one fp32
 * per output row, W[n][k] = fp8(W8[n][k]) * w_scale[n] (the reference's per-row quantisation,
 * triton_kernels.py:261-268; its use in the fused decode kernel, :927-940 and :963-965, argument
 * weight_scale of qkv_rope_cache_decode_forward :1109). Half the bytes of the bf16 kernel; activations stay
 * bf16, accumulation fp32. norm_scale may be NULL (no fused RMSNorm) or as in tllm_norm_qkv_rope_decode_bf16.
 * hidden == 2880 with head_dim == 64: the weight-streaming kernels; any other hidden % 32 == 0 with
 * head_dim % 16 == 0: the general MFMA decode kernel, norm_scale must be NULL there and q / k / v 4-byte aligned
 * with even strides (TLLM_E_SHAPE / TLLM_E_ALIGN otherwise). */
int tllm_qkv_rope_decode_w8_bf16(const void* x, const void* norm_scale, int scale_is_bf16, float eps,
                                 const void* W8, const float* w_scale, const void* b, void* q, void* k, void* v,
                                 int64_t q_row_stride, int64_t k_row_stride, int64_t v_row_stride,
                                 int64_t kv_slot_stride,
                                 int64_t rows, int64_t hidden, int n_q_heads, int n_kv_heads, int head_dim,
                                 const TllmRope* rope, void* stream);

int tllm_qkv_rope_prefill_bf16(const void* x, const void* W, const void* b,
                               void* q, void* k, void* v,
                               int64_t q_row_stride, int64_t k_row_stride, int64_t v_row_stride,
                               int64_t kv_slot_stride,
                               int64_t rows, int64_t hidden, int n_q_heads, int n_kv_heads, int head_dim,
                               const TllmRope* rope, void* stream);

/* Decode-size attention out-projection with bias and residual,
 *   out[r, n] = sum_k x[r, k] * W[n, k] + bias[n] + residual[r, n]        (fp32 accumulate, one RNE to bf16),
 * replaces out_residual_decode_forward(hidden, weight, bias, residual, weight_scale=None),
 * triton_kernels.py:1470-1517 (its split-K kernel :1340-1416 and reduce kernel :1419-1467, in one launch
 * and without the partial-sum buffer). x [rows, in_dim] bf16 dense; W [out_dim, in_dim] bf16 dense, or fp8
 * e4m3 bytes when w_scale (one fp32 per output row) is not NULL; bias [out_dim] or NULL; residual
 * [rows, out_dim] with res_row_stride elements between rows, or NULL; out likewise and MAY BE the residual
 * buffer (the reference writes its result into it). The weight-streaming kernel serves in_dim == 4096
 * with out_dim a multiple of 12 (gpt-oss: 2880 x 4096); other shapes take a plain kernel. */
int tllm_out_residual_decode_bf16(const void* x, const void* W, const float* w_scale, const void* bias,
                                  const void* residual, void* out, int64_t res_row_stride, int64_t out_row_stride,
                                  int64_t rows, int64_t in_dim, int64_t out_dim, void* stream);

/* Decode-size unembedding over the whole vocabulary, logits[r, v] = sum_k x[r, k] * W[v, k] (fp32 accumulate, one
 * RNE to bf16); replaces unembedding_decode_forward(hidden, weight), triton_kernels.py:163-197 (kernel :111-160),
 * and with w_scale != NULL unembedding_decode_fp8_forward :271-302 (W = fp8 e4m3 bytes, one fp32 scale per
 * vocabulary row, as quantised by :261-268). x [rows, hidden] bf16 dense, W [vocab, hidden] dense, logits
 * [rows, vocab] with logits_row_stride elements between rows. hidden must be a multiple of 64. One pass over the
 * weight serves up to 32 rows; more rows take one pass per 32. */
int tllm_unembedding_decode_bf16(const void* x, const void* W, const float* w_scale, void* logits,
                                 int64_t logits_row_stride, int64_t rows, int64_t hidden, int64_t vocab, void* stream);

/* Greedy sampling fused into the same stream: token_ids[r] = argmax_v of the fp32 sums above (lowest index on a
 * tie), no logits written; replaces unembedding_decode_argmax_forward, triton_kernels.py:363-401 (kernel
 * :305-360 + the torch argmax over tiles), and its fp8 twin :470-512. The per-wavefront candidates pass through
 * `workspace` (device memory, 4-byte aligned, at least tllm_unembedding_argmax_workspace_bytes(rows) bytes; the
 * reference takes its partial_max / partial_idx from its scratch pool the same way). token_ids: int32 [rows]. */
int64_t tllm_unembedding_argmax_workspace_bytes(int64_t rows);
int tllm_unembedding_argmax_bf16(const void* x, const void* W, const float* w_scale, void* workspace,
                                 int64_t workspace_bytes, int32_t* token_ids, int64_t rows, int64_t hidden,
                                 int64_t vocab, void* stream);

/* The same greedy sampling for callers that cannot allocate device memory or hand over a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc). No counterpart in the reference, which takes
 * its partial_max / partial_idx buffers from its scratch pool. The per-wavefront candidates pass through a
 * 512 KiB device array owned by the library (one copy per GPU, held until the process ends), so rows is limited to
 * tllm_unembedding_argmax_noalloc_max_rows() = 16; more rows return TLLM_E_SHAPE. The call allocates nothing and
 * gives the same token_ids as tllm_unembedding_argmax_bf16. All calls on one GPU share the array: calls that may run
 * concurrently on one GPU (different streams without ordering between them) race on it and must be serialised by the
 * caller. Nothing in the array needs clearing between calls.
 * The array's device address is looked up once per GPU, by a runtime query that is not allowed while a stream is
 * capturing: tllm_unembedding_argmax_noalloc_init() does it for the current device and is to be called (once per
 * device, outside any capture) by callers that capture. Without it the first eager call on a device does the look-up,
 * and a first call on a capturing stream returns TLLM_E_ARG instead of disturbing the capture. */
int64_t tllm_unembedding_argmax_noalloc_max_rows(void);
int tllm_unembedding_argmax_noalloc_init(void);
int tllm_unembedding_argmax_noalloc_bf16(const void* x, const void* W, const float* w_scale, int32_t* token_ids,
                                         int64_t rows, int64_t hidden, int64_t vocab, void* stream);

/* Decode attention with learned sinks and an optional sliding window: one new token per batch row against the KV
 * cache; replaces attention_decode(q, k, v, sinks, sm_scale, bandwidth, start_q), attention_tt_decode.py:290-408
 * (kernels :9-287), whose definition is attention_ref.py:4-42:
 *   keys lo..hi-1, hi = min(start_q + 1, n_kv_ctx), lo = window ? max(0, start_q - window + 1) : 0;
 *   out[h] = softmax over {sm_scale <q[h], k[n]>} U {sink[h]} applied to v (the sink has no value row).
 * q, out: [batch, n_kv_heads * group * 64] bf16 (head h = kv_head * group + g), row strides in elements;
 * k, v: [batch, n_kv_ctx, n_kv_heads, 64] bf16 with the given batch and token strides (the heads of a token
 * dense); sinks: [n_kv_heads * group] bf16 or NULL (then every head has a sink of logit 0, as in the reference);
 * start_q: DEVICE scalar, int32 or int64 (start_q_is_i64), read by the kernel; window 0 = none.
 * Long contexts are split over workgroups: tllm_attention_decode_workspace_bytes(...) says how much device
 * scratch (4-byte aligned) that needs for the same arguments -- 0 for short contexts; the reference allocates its
 * acc/m/l partials per call (:343-345). head_dim must be 64, group <= 16.
 * The launch (workgroup shape, number of splits) is planned on the host from n_kv_ctx, the size of the cache, like the
 * reference's SPLIT_K (:311-315); the kernels then use only as many of the planned splits as the context they read
 * from start_q needs. kv_len_hint (0: none) lets a caller that knows roughly how many keys are visible -- a decode
 * loop knows its position on the host -- have the launch planned for that instead of for the whole cache: results do
 * not depend on it, a hint that is too small only costs speed. Pass min(hint, n_kv_ctx) as n_kv_ctx to the three
 * planning helpers below when a hint is used. */
int tllm_attention_decode_splits(int64_t batch, int n_kv_heads, int64_t n_kv_ctx, int window);
/* Diagnostic: KV heads served by one workgroup for these arguments (8 or 4: one wavefront per head, contiguous
 * cache rows; 0: one KV head per workgroup). No counterpart in the reference. */
int tllm_attention_decode_heads_per_workgroup(int64_t batch, int n_kv_heads, int64_t n_kv_ctx, int window);
int64_t tllm_attention_decode_workspace_bytes(int64_t batch, int n_q_heads, int n_kv_heads, int64_t n_kv_ctx, int window);
int tllm_attention_decode_bf16(const void* q, const void* k, const void* v, const void* sinks, void* out,
                               int64_t q_row_stride, int64_t out_row_stride, int64_t kv_batch_stride,
                               int64_t kv_token_stride, int64_t batch, int64_t n_kv_ctx, int n_kv_heads, int group,
                               int head_dim, float sm_scale, int window, const void* start_q, int start_q_is_i64,
                               int64_t kv_len_hint, void* workspace, int64_t workspace_bytes, void* stream);

/* Prefill attention with sinks and an optional sliding window: n_q query positions per batch row against the keys
 * written so far. Replaces attention (attention_tt.py:167-242, kernel :17-164; definition attention_ref.py:4-42).
 * q [batch, n_q, n_kv_heads * group, 64] with batch / token strides in elements (heads adjacent: the layout the QKV
 * projection writes), k / v [batch, n_kv_ctx, n_kv_heads, 64] with batch / token strides (a view of the KV cache
 * will do), sinks [n_kv_heads * group] bf16 or NULL (logit 0, :103-106), out [batch, n_q, n_kv_heads * group * 64].
 * Query i sits at position start_q + i (start_q: one int32 / int64 element in device memory, read on the device) and
 * sees keys n <= position, n < n_kv_ctx and, when window > 0, n > position - window. Unlike the reference, no
 * transposed or padded copies of q, k, v are made. head_dim must be 64, sm_scale positive. */
int tllm_attention_prefill_bf16(const void* q, const void* k, const void* v, const void* sinks, void* out,
                                int64_t q_batch_stride, int64_t q_token_stride, int64_t out_batch_stride,
                                int64_t out_token_stride, int64_t kv_batch_stride, int64_t kv_token_stride,
                                int64_t batch, int64_t n_q, int64_t n_kv_ctx, int n_kv_heads, int group, int head_dim,
                                float sm_scale, int window, const void* start_q, int start_q_is_i64, void* stream);

/* MXFP4 -> bf16 expansion of checkpoint tensors (Checkpoint._get_mxfp4_tensor, weights.py:68-117): blocks
 * [n_blocks][16] bytes, 32 e2m1 values per block with the low nibble first (table weights.py:11-14); scales [n_blocks]
 * e8m0 bytes (bias 127); out [n_blocks][32] bf16 = FP4[nibble] * 2^(scale - 127), formed in fp32 and rounded once, as
 * torch.ldexp does on the reference's bf16 tensor. Bit-exact. */
int tllm_mxfp4_dequant_bf16(const void* blocks, const void* scales, void* out, int64_t n_blocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TLLM_HIP_H */
