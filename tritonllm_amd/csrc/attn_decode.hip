// Decode attention with learned sinks and an optional sliding window, one new token per batch row against the KV
// cache (attention_decode, attention_tt_decode.py:290-408; kernels :9-287; definition attention_ref.py:4-42):
//
//   keys lo .. hi-1 with hi = min(start_q + 1, n_kv_ctx), lo = window ? max(0, start_q - window + 1) : 0
//   s[h, n]  = sm_scale * <q[h], k[n]>                       h = kv_head * G + g   (G query heads share a KV head)
//   out[h]   = sum_n exp(s[h, n] - m) v[n] / (sum_n exp(s[h, n] - m) + exp(sink[h] - m)),   m = max(sink[h], max_n s[h, n])
//
// The reference runs one program per query head, so the G heads of a group each read the same K and V; here a
// workgroup takes a (batch row, KV head, context split) and serves all G heads from one pass over K and V:
//   * four wavefronts take 32-key blocks of the split in turn, each with its own running (max, sum, accumulator);
//   * S^T = K . Q^T on v_mfma_f32_16x16x32_bf16 with the keys on M: K rows are K-contiguous in memory, so a lane
//     loads its 16 bytes of a key row straight into operand layout; Q sits in registers as the B operand;
//   * the accumulator layout of S^T (lane = head, registers = keys) IS the A-operand layout of P for O = P . V when
//     the MFMA's k slots are read as a permutation of the block's keys, so P never leaves the registers; V, whose
//     rows are d-contiguous, goes through a wavefront-private LDS tile and is gathered in that same key order;
//   * the per-head rescale factor exp(m_old - m_new) lives in the S^T layout and is fetched into the O layout
//     (registers = heads) by ds_bpermute;
//   * wavefronts meet once at the end through LDS; with more than one context split the workgroups leave
//     (max, sum, accumulator) in a workspace and a second small kernel folds them and the sink.
// start_q is read from device memory (int32 or int64), so a captured graph follows the growing context.
#include "common.h"

namespace tllm {

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

struct AttnArgs {
  const bf16* q;          // [B, n_q_heads * 64], row stride q_rs
  const bf16* k;          // [B, n_kv_ctx, n_kv_heads, 64]: batch stride kv_bs, token stride kv_ts (elements)
  const bf16* v;
  const bf16* sinks;      // [n_q_heads] or null (a null sink still counts, with logit 0, as in the reference)
  bf16* out;              // [B, n_q_heads * 64], row stride out_rs
  float* part;            // [splits][B][n_q_heads][66]: acc[64], max, sum (when splits > 1)
  const void* start_q;    // device scalar
  int start_is_i64;
  int64_t q_rs, out_rs, kv_bs, kv_ts;
  int n_kv_ctx, n_kv_heads, group, window, splits;
  float sm_scale;
};

namespace {
constexpr int AW = 4;                 // wavefronts per workgroup
constexpr int VROW = 128 + 16;        // V tile row in LDS: 64 bf16 + padding, bytes
constexpr int VTILE = 32 * VROW;
constexpr float kNegBig = -1.0e30f;
constexpr int PART = 66;              // floats per (split, row, head) in the workspace
}  // namespace

__device__ __forceinline__ int attn_start_q(const AttnArgs& a) {
  return a.start_is_i64 ? static_cast<int>(*reinterpret_cast<const int64_t*>(a.start_q)) : *reinterpret_cast<const int*>(a.start_q);
}

__global__ __launch_bounds__(AW * 64) void attn_decode_kernel(AttnArgs a) {
  __shared__ __align__(16) unsigned char vt[AW * VTILE];
  __shared__ float s_m[AW][16], s_l[AW][16];
  __shared__ float s_acc[AW][16][64 + 1];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int kvh = blockIdx.x / a.splits, split = blockIdx.x - kvh * a.splits;
  const int64_t b = blockIdx.y;
  const int G = a.group;
  const int n_q_heads = a.n_kv_heads * G;

  // ---- key range of this split
  const int start_q = attn_start_q(a);
  int hi = start_q + 1 < a.n_kv_ctx ? start_q + 1 : a.n_kv_ctx;
  hi = hi > 0 ? hi : 0;
  int lo = a.window > 0 ? (start_q - a.window + 1 > 0 ? start_q - a.window + 1 : 0) : 0;
  lo = lo < hi ? lo : hi;
  const int len = hi - lo;
  int chunk = (len + a.splits - 1) / a.splits;
  chunk = (chunk + 31) & ~31;                                 // whole 32-key blocks per split
  const int s_lo = lo + split * chunk < hi ? lo + split * chunk : hi;
  const int s_hi = s_lo + chunk < hi ? s_lo + chunk : hi;
  const int nblk = (s_hi - s_lo + 31) >> 5;

  // ---- Q as the B operand of S^T = K . Q^T: lane (n = head r16, k = 8 g + j) for each 32-wide half of d
  const int hq = r16 < G ? r16 : G - 1;                       // columns >= G repeat the last head; never stored
  const bf16* qrow = a.q + b * a.q_rs + (static_cast<int64_t>(kvh) * G + hq) * 64;
  const bf16x8 qb0 = *reinterpret_cast<const bf16x8*>(qrow + 8 * g);
  const bf16x8 qb1 = *reinterpret_cast<const bf16x8*>(qrow + 32 + 8 * g);

  const bf16* kbase = a.k + b * a.kv_bs + static_cast<int64_t>(kvh) * 64;
  const bf16* vbase = a.v + b * a.kv_bs + static_cast<int64_t>(kvh) * 64;
  unsigned char* vtile = vt + wave * VTILE;

  float m_run = kNegBig, l_run = 0.f;                          // of head r16 (replicated over the four lane groups)
  f32x4_t acc[4];                                              // O: lane (d = 16 nb + r16, heads 4 g + i)
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) acc[nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // A operands of a block: K[key = k0 + 16 kb + r16][32 t + 8 g ..]; V tile chunks: key (i*64+lane)/8, chunk (i*64+lane)%8.
  // Rows past the end of the split are clamped to its last key (finite values; their probabilities are zeroed).
  // Addressing is a block base (uniform) plus a 32-bit lane offset: row * token stride + a lane constant.
  const unsigned ts_b = static_cast<unsigned>(a.kv_ts) * 2u;   // token stride, bytes (a 32-key block spans < 4 GB)
  bf16x8 ka[2][2], vr[4];
  auto load_block = [&](int k0) {
    const int last = s_hi - k0 - 1;                            // last valid row of the block (>= 31 except in the final one)
    const unsigned char* kb0 = reinterpret_cast<const unsigned char*>(kbase + static_cast<int64_t>(k0) * a.kv_ts);
    const unsigned char* vb0 = reinterpret_cast<const unsigned char*>(vbase + static_cast<int64_t>(k0) * a.kv_ts);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int r = 16 * kb + r16;
      const unsigned off = static_cast<unsigned>(r < last ? r : last) * ts_b + 16u * g;
      ka[kb][0] = *reinterpret_cast<const bf16x8*>(kb0 + off);
      ka[kb][1] = *reinterpret_cast<const bf16x8*>(kb0 + off + 64);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = i * 64 + lane;
      const int r = c >> 3;
      vr[i] = *reinterpret_cast<const bf16x8*>(vb0 + static_cast<unsigned>(r < last ? r : last) * ts_b + 16u * (c & 7));
    }
  };

  if (nblk > 0 && wave < nblk) load_block(s_lo + 32 * wave);
  for (int blk = wave; blk < nblk; blk += AW) {
    const int k0 = s_lo + 32 * blk;
    // ---- S^T for the block's two 16-key halves
    f32x4_t st[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      st[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kb][0], qb0, f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      st[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kb][1], qb1, st[kb], 0, 0, 0);
    }
    // V tile into LDS (row-major, as loaded)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = i * 64 + lane;
      *reinterpret_cast<bf16x8*>(vtile + (c >> 3) * VROW + (c & 7) * 16) = vr[i];
    }
    // The next block's loads go out before this one's arithmetic. Unconditional (a load under a branch makes the
    // compiler wait for it where the paths join): the last round simply requests its own block again.
    load_block(s_lo + 32 * (blk + AW < nblk ? blk + AW : blk));

    // ---- online softmax for head r16: this lane holds keys k0 + 16 kb + 4 g + i
    float sc[8];
    float bmax = kNegBig;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = k0 + 16 * kb + 4 * g + i;
        const float s = key < s_hi ? st[kb][i] * a.sm_scale : kNegBig;
        sc[4 * kb + i] = s;
        bmax = fmaxf(bmax, s);
      }
    bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
    const float m_new = fmaxf(m_run, bmax);
    const float alpha = __expf(m_run - m_new);
    float psum = 0.f;
    bf16x8 pa;                                                 // A operand of P . V: k slot j <-> key 4 g + j (j < 4), 16 + 4 g + j - 4
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float p = sc[j] > 0.5f * kNegBig ? __expf(sc[j] - m_new) : 0.f;
      psum += p;
      pa[j] = static_cast<bf16>(p);
    }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;

    // ---- rescale O (registers = heads 4 g + i) by the alpha of those heads (held by lanes with r16 == head).
    // Once the running maxima have settled -- after the first blocks, for most inputs -- every alpha is exactly 1
    // and the whole step (four bpermutes, sixteen multiplies, the accumulators' trip out of the MFMA registers) is
    // skipped, wavefront-uniformly.
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float al = __shfl(alpha, 4 * g + i, 64);
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) acc[nb][i] *= al;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      // B operand: V[key(j)][d = 16 nb + r16] for the eight k slots of this lane group
      bf16x8 vb;
      const unsigned char* col = vtile + (16 * nb + r16) * 2;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = j < 4 ? 4 * g + j : 16 + 4 * g + (j - 4);
        vb[j] = *reinterpret_cast<const bf16*>(col + key * VROW);
      }
      acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, vb, acc[nb], 0, 0, 0);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }

  // ---- the four wavefronts meet: (max, sum) per head, accumulator per (head, d)
  if (g == 0) {
    s_m[wave][r16] = m_run;
    s_l[wave][r16] = l_run;
  }
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int i = 0; i < 4; ++i) s_acc[wave][4 * g + i][16 * nb + r16] = acc[nb][i];
  __syncthreads();

  // thread -> (head = tid / 16 (< 16), four d: tid % 16 + 16 j)
  const int eh = tid >> 4, ed = tid & 15;
  if (eh >= G) return;
  float m_all = kNegBig;
#pragma unroll
  for (int w = 0; w < AW; ++w) m_all = fmaxf(m_all, s_m[w][eh]);
  float l_all = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int w = 0; w < AW; ++w) {
    const float f = __expf(s_m[w][eh] - m_all);              // a wavefront without keys has sum 0 and accumulator 0
    l_all += s_l[w][eh] * f;
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] += s_acc[w][eh][ed + 16 * j] * f;
  }
  const int head = kvh * G + eh;
  if (a.splits > 1) {
    float* p = a.part + ((static_cast<int64_t>(split) * gridDim.y + b) * n_q_heads + head) * PART;
#pragma unroll
    for (int j = 0; j < 4; ++j) p[ed + 16 * j] = o[j];
    if (ed == 0) {
      p[64] = m_all;
      p[65] = l_all;
    }
    return;
  }
  const float sink = a.sinks ? static_cast<float>(a.sinks[head]) : 0.f;
  const float m_f = fmaxf(m_all, sink);
  const float f = __expf(m_all - m_f);
  const float z = l_all * f + __expf(sink - m_f);
  bf16* orow = a.out + b * a.out_rs + static_cast<int64_t>(head) * 64;
#pragma unroll
  for (int j = 0; j < 4; ++j) orow[ed + 16 * j] = static_cast<bf16>(o[j] * f / z);
}

// One wavefront per (batch row, head): fold the context splits and the sink. Lane s first fetches (max, sum) of
// split s, so the weights of all splits are known after one round trip; the accumulators are then summed with
// eight independent loads in flight (a loop of dependent loads would cost one memory latency per split).
__global__ __launch_bounds__(64) void attn_decode_reduce_kernel(AttnArgs a, int batch) {
  const int head = blockIdx.x, lane = threadIdx.x;
  const int64_t b = blockIdx.y;
  const int n_q_heads = a.n_kv_heads * a.group;
  const int64_t split_stride = static_cast<int64_t>(batch) * n_q_heads * PART;
  const float* p0 = a.part + (b * n_q_heads + head) * PART;
  const bool has = lane < a.splits;
  const float m_s = has ? p0[lane * split_stride + 64] : kNegBig;
  const float l_s = has ? p0[lane * split_stride + 65] : 0.f;
  float m_all = m_s;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m_all = fmaxf(m_all, __shfl_xor(m_all, o, 64));
  const float f_s = __expf(m_s - m_all);                     // 0 for the lanes without a split
  const float l_all = wave_sum(l_s * f_s);
  float o = 0.f;
  for (int s0 = 0; s0 < a.splits; s0 += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int s = s0 + u < a.splits ? s0 + u : a.splits - 1;
      v[u] = p0[s * split_stride + lane];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float f = __shfl(f_s, s0 + u < a.splits ? s0 + u : 0, 64);
      o += (s0 + u < a.splits) ? v[u] * f : 0.f;
    }
  }
  const float sink = a.sinks ? static_cast<float>(a.sinks[head]) : 0.f;
  const float m_f = fmaxf(m_all, sink);
  const float f = __expf(m_all - m_f);
  const float z = l_all * f + __expf(sink - m_f);
  a.out[b * a.out_rs + static_cast<int64_t>(head) * 64 + lane] = static_cast<bf16>(o * f / z);
}

}  // namespace tllm

using namespace tllm;

// Context splits, from measurements at B = 1 and 8, contexts 1K - 32K: first enough workgroups to give every CU one
// (with one batch row and eight KV heads that alone asks for 32 splits), beyond that about 1024 keys per workgroup
// (eight 32-key blocks per wavefront: fewer and the per-workgroup start-up dominates, more and too few wavefronts
// are resident to cover the load latency); never less than 128 keys per split. A sliding window bounds the context.
extern "C" int tllm_attention_decode_splits(int64_t batch, int n_kv_heads, int64_t n_kv_ctx, int window) {
  const int64_t ctx = (window > 0 && window < n_kv_ctx) ? window : n_kv_ctx;
  const int64_t units = batch * n_kv_heads > 0 ? batch * n_kv_heads : 1;
  const int64_t fill = (256 + units - 1) / units;
  const int64_t by_work = (ctx + 1023) / 1024;
  int64_t s = fill > by_work ? fill : by_work;
  const int64_t cap = (ctx + 127) / 128;
  if (s > cap) s = cap;
  if (s < 1) s = 1;
  if (s > 64) s = 64;
  return (int)s;
}

extern "C" int64_t tllm_attention_decode_workspace_bytes(int64_t batch, int n_q_heads, int n_kv_heads, int64_t n_kv_ctx, int window) {
  const int s = tllm_attention_decode_splits(batch, n_kv_heads, n_kv_ctx, window);
  return s > 1 ? static_cast<int64_t>(s) * batch * n_q_heads * PART * 4 : 0;
}

extern "C" int tllm_attention_decode_bf16(const void* q, const void* k, const void* v, const void* sinks, void* out, int64_t q_row_stride,
                                          int64_t out_row_stride, int64_t kv_batch_stride, int64_t kv_token_stride, int64_t batch,
                                          int64_t n_kv_ctx, int n_kv_heads, int group, int head_dim, float sm_scale, int window,
                                          const void* start_q, int start_q_is_i64, void* workspace, int64_t workspace_bytes, void* stream) {
  TLLM_REQUIRE(batch >= 0 && n_kv_ctx >= 1 && n_kv_ctx < (1ll << 31) && n_kv_heads >= 1, TLLM_E_SHAPE,
               "attention_decode: batch %lld, n_kv_ctx %lld, n_kv_heads %d", (long long)batch, (long long)n_kv_ctx, n_kv_heads);
  TLLM_REQUIRE(head_dim == 64, TLLM_E_SHAPE, "attention_decode: head_dim %d (only 64 is built)", head_dim);
  TLLM_REQUIRE(group >= 1 && group <= 16, TLLM_E_SHAPE, "attention_decode: %d query heads per KV head (1..16)", group);
  TLLM_REQUIRE(window >= 0, TLLM_E_ARG, "attention_decode: window %d", window);
  if (batch == 0) return TLLM_OK;
  TLLM_REQUIRE(batch <= 65535, TLLM_E_SHAPE, "attention_decode: batch %lld too large", (long long)batch);
  TLLM_REQUIRE(q && k && v && out && start_q, TLLM_E_ARG, "attention_decode: q, k, v, out and start_q must not be NULL");
  TLLM_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && q_row_stride % 8 == 0 && kv_batch_stride % 8 == 0 && kv_token_stride % 8 == 0,
               TLLM_E_ALIGN, "attention_decode: q, k, v must be 16-byte aligned with strides that are multiples of 8 elements");
  TLLM_REQUIRE(kv_token_stride >= static_cast<int64_t>(n_kv_heads) * 64, TLLM_E_ARG, "attention_decode: kv_token_stride < n_kv_heads * 64");
  AttnArgs a{};
  a.q = (const bf16*)q;
  a.k = (const bf16*)k;
  a.v = (const bf16*)v;
  a.sinks = (const bf16*)sinks;
  a.out = (bf16*)out;
  a.start_q = start_q;
  a.start_is_i64 = start_q_is_i64;
  a.q_rs = q_row_stride;
  a.out_rs = out_row_stride;
  a.kv_bs = kv_batch_stride;
  a.kv_ts = kv_token_stride;
  a.n_kv_ctx = (int)n_kv_ctx;
  a.n_kv_heads = n_kv_heads;
  a.group = group;
  a.window = window;
  a.sm_scale = sm_scale;
  a.splits = tllm_attention_decode_splits(batch, n_kv_heads, n_kv_ctx, window);
  const int64_t need = tllm_attention_decode_workspace_bytes(batch, n_kv_heads * group, n_kv_heads, n_kv_ctx, window);
  TLLM_REQUIRE(need == 0 || (workspace != nullptr && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 4 == 0), TLLM_E_ARG,
               "attention_decode: workspace of %lld bytes needed (tllm_attention_decode_workspace_bytes), got %lld", (long long)need,
               (long long)workspace_bytes);
  a.part = static_cast<float*>(workspace);
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(attn_decode_kernel, dim3((unsigned)(n_kv_heads * a.splits), (unsigned)batch), dim3(AW * 64), 0, st, a);
  int rc = check_launch("attention_decode");
  if (rc != TLLM_OK || a.splits == 1) return rc;
  hipLaunchKernelGGL(attn_decode_reduce_kernel, dim3((unsigned)(n_kv_heads * group), (unsigned)batch), dim3(64), 0, st, a, (int)batch);
  return check_launch("attention_decode(reduce)");
}
