// Pieces shared by the decode and prefill QKV kernels: argument block, host-side
// validation, the output-row addressing, and the shape-generic fallback kernel.
#pragma once

#include "common.h"

namespace tllm {

struct QkvArgs {
  const bf16* x;
  const bf16* W;
  const bf16* bias;   // may be null
  bf16* q;
  bf16* k;
  bf16* v;
  int64_t q_rs, k_rs, v_rs;   // elements between consecutive rows of q / k / v
  int64_t kv_slot_stride;     // elements per KV-cache slot (0: no slot offset)
  int64_t rows;
  int hidden;
  int n_q_heads, n_kv_heads, head_dim;
  int has_rope;
  const void* norm_scale;     // fused RMSNorm prologue (decode fast path only): scale [hidden], fp32 or bf16
  float norm_eps;
  const float* w_scale;        // fp8 weight (decode fast path only): one fp32 scale per output row
  // fused token-embedding gather (decode fast path with the fused norm only): x[r] = emb_table[emb_ids[r]], also
  // written to emb_out (the residual stream the following layers read)
  const void* emb_ids;         // int32 or int64 [rows]
  int emb_ids_i64;
  const bf16* emb_table;       // [emb_vocab, hidden]
  int64_t emb_vocab;
  bf16* emb_out;               // [rows, hidden] dense
  int32_t* emb_oob;            // may be null
};

// KV-cache slot the new token goes to (0 when the outputs are plain tensors). A global load: call it early.
__device__ __forceinline__ int64_t qkv_slot(const QkvArgs& a, const RopeArgs& ra) {
  return (a.kv_slot_stride != 0 && ra.offset != nullptr) ? ra.offset[0] : 0;
}

// Start of head `head` (0 .. n_q + 2 n_kv) of output row `row`.
__device__ __forceinline__ bf16* qkv_out_ptr(const QkvArgs& a, int64_t slot, int64_t row, int head) {
  if (head < a.n_q_heads) return a.q + row * a.q_rs + static_cast<int64_t>(head) * a.head_dim;
  head -= a.n_q_heads;
  if (head < a.n_kv_heads) return a.k + row * a.k_rs + slot * a.kv_slot_stride + static_cast<int64_t>(head) * a.head_dim;
  head -= a.n_kv_heads;
  return a.v + row * a.v_rs + slot * a.kv_slot_stride + static_cast<int64_t>(head) * a.head_dim;
}

int qkv_validate(const char* who, const void* x, const void* W, const void* q, const void* k, const void* v, int64_t q_rs,
                 int64_t k_rs, int64_t v_rs, int64_t kv_slot_stride, int64_t rows, int64_t hidden, int n_q_heads, int n_kv_heads,
                 int head_dim, const TllmRope* rope, QkvArgs* a, RopeArgs* ra, YarnFreqs* fr);

// The hidden-2880 decode kernel for up to xr = 8 rows per workgroup, or xr = 16 with the fused RMSNorm: bf16 or fp8 weight,
// optional fused RMSNorm and token gather (qkv_decode_r8.hip).
void launch_qkv_decode_r8(int xr, int norm, bool emb, bool w8, dim3 grid, hipStream_t st, const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr);
// ... and for 9..32 rows per workgroup, bf16 or fp8 weight, activations already normalised (qkv_decode_r32.hip).
void launch_qkv_decode_r32(bool w8, dim3 grid, hipStream_t st, const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr);
// ... and for any number of rows in one pass over the weight, activations already normalised (qkv_decode_rows.hip).
void launch_qkv_decode_rows(bool w8, dim3 grid, hipStream_t st, const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr);

// Any hidden size, any even head_dim: one workgroup per (head, row); each wavefront takes
// rotation pairs (d, d + hd/2) in turn and reduces the two dot products by shuffle.
void launch_qkv_generic(const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr, hipStream_t st);

}  // namespace tllm
