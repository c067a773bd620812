// Prefill attention with learned sinks and an optional sliding window: many query positions per batch row against
// the keys written so far (attention, attention_tt.py:166-236; kernel :17-164; definition attention_ref.py:4-42):
//
//   query i of a batch row sits at position p = start_q + i and sees the keys n with
//       n <= p,   n < n_kv_ctx,   n > p - window (when a window is set)
//   s[i, h, n] = sm_scale * <q[i, h], k[n, kv(h)]>                      kv(h) = h / G   (G query heads share a KV head)
//   out[i, h]  = sum_n exp(s - m) v[n, kv(h)] / (sum_n exp(s - m) + exp(sink[h] - m)),    m = max(sink[h], max_n s)
//
// The reference transposes q, k and v into head-major copies, pads them to the block size and runs one program per
// (64 queries, query head). Here the kernel reads q as the QKV projection wrote it ([token, head, 64]) and k / v in
// the cache layout ([token, kv head, 64]), and writes [token, head * 64]: no copies on either side.
//
//   * a workgroup takes 128 consecutive queries of NH query heads that share a KV head, four wavefronts of 32 queries;
//     K / V blocks of 64 keys pass through two LDS stages (registers -> LDS while the previous block is computed,
//     one barrier per block) and serve all NH heads;
//   * S^T = K . Q^T on v_mfma_f32_32x32x16_bf16 with the keys on M: a lane then owns ONE query (column) and 16 keys
//     per 32-key block, so the running maximum, the running sum and the rescale factor of the online softmax are
//     lane-local apart from one exchange between the two half-wavefronts;
//   * those accumulator registers are, pairwise, the B operand (P^T) of O^T = V^T . P^T when the MFMA's k slots are read
//     as a permutation of the block's keys, so P never leaves the registers; V is written into LDS transposed
//     ([d][key], keys in that permuted order, two keys per 32-bit write) so that the A operand is one 16-byte read;
//   * both tiles are XOR-swizzled in 16-byte chunks: fragment reads are conflict-free;
//   * the KV head is the fastest-varying part of the workgroup index, so with eight KV heads each XCD's L2 holds the
//     K and V of one head; the query tiles with the most keys to visit are launched first.
// start_q is read from device memory (int32 or int64).
#include "common.h"

namespace tllm {

struct AttnPrefillArgs {
  const bf16* q;          // [B, n_q, n_heads, 64]: batch stride q_bs, token stride q_ts (elements), heads adjacent
  const bf16* k;          // [B, n_kv_ctx, n_kv_heads, 64]: batch stride kv_bs, token stride kv_ts
  const bf16* v;
  const bf16* sinks;      // [n_heads] or null (logit 0, attention_tt.py:103-106)
  bf16* out;              // [B, n_q, n_heads * 64]: batch stride out_bs, token stride out_ts
  const void* start_q;    // device scalar
  int start_is_i64;
  int64_t q_bs, q_ts, out_bs, out_ts, kv_bs, kv_ts;
  int batch, n_q, n_kv_ctx, n_kv_heads, group, window;
  float sm_scale;
};

namespace {
constexpr int PBM = 128;              // queries per workgroup
constexpr int PBN = 64;               // keys per block
constexpr int KT_BYTES = PBN * 128;   // K tile [key][64 d]
constexpr int VT_BYTES = 64 * 128;    // V^T tile [d][64 keys]
constexpr int PSTAGE = KT_BYTES + VT_BYTES;
constexpr float kLog2e = 1.4426950408889634f;
}  // namespace

// 16-byte chunk swizzle of a V^T row: consecutive rows (fragment reads) and rows eight apart (the transposing writes)
// both land on distinct chunks.
__device__ __forceinline__ int vt_swizzle(int d) { return ((d >> 1) ^ (d >> 3)) & 7; }

template <int NH>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(AttnPrefillArgs a) {
  __shared__ __align__(16) unsigned char smem[2 * PSTAGE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, h = lane >> 5;

  // workgroup -> (kv head, head sub-group, batch row, query tile); kv head fastest, long tiles first
  const int nsub = a.group / NH;
  const int ntiles = (a.n_q + PBM - 1) / PBM;
  unsigned id = blockIdx.x;
  const int kvh = id % a.n_kv_heads;
  id /= a.n_kv_heads;
  const int sub = id % nsub;
  id /= nsub;
  const int b = id % a.batch;
  id /= a.batch;
  const int tile = ntiles - 1 - static_cast<int>(id);
  const int head0 = kvh * a.group + sub * NH;

  const int start = a.start_is_i64 ? static_cast<int>(*reinterpret_cast<const int64_t*>(a.start_q)) : *reinterpret_cast<const int*>(a.start_q);
  const int q0 = tile * PBM;
  const int qw0 = q0 + wave * 32;          // the wavefront's first query
  const int p0 = start + qw0;              // and its position
  const int q_end = q0 + PBM < a.n_q ? q0 + PBM : a.n_q;
  int kv_hi = start + q_end < a.n_kv_ctx ? start + q_end : a.n_kv_ctx;       // keys the tile's last query sees (exclusive)
  kv_hi = kv_hi > 0 ? kv_hi : 0;
  int kv_lo = a.window > 0 ? start + q0 - a.window + 1 : 0;
  kv_lo = kv_lo > 0 ? kv_lo : 0;
  kv_lo = kv_lo < kv_hi ? kv_lo : kv_hi;
  const int blk_lo = kv_lo / PBN, blk_hi = (kv_hi + PBN - 1) / PBN;
  const int key_max = kv_hi - 1;           // rows beyond it are never visible and may hold anything: not loaded

  const bf16* kp = a.k + b * a.kv_bs + kvh * 64;
  const bf16* vp = a.v + b * a.kv_bs + kvh * 64;

  // ---- Q fragments (B operand: lane = query, 8 d per half-wavefront and k16 step)
  bf16x8 qf[NH][4];
  {
    int qrow = qw0 + l31;
    qrow = qrow < a.n_q ? qrow : a.n_q - 1;
    const bf16* qp = a.q + b * a.q_bs + static_cast<int64_t>(qrow) * a.q_ts + head0 * 64 + h * 8;
#pragma unroll
    for (int hd = 0; hd < NH; ++hd)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) qf[hd][kk] = *reinterpret_cast<const bf16x8*>(qp + hd * 64 + kk * 16);
  }

  // ---- K / V block movers. K: thread -> two 16-byte chunks. V: thread -> 8 d of two keys that are neighbours in the
  // permuted key order (keys 2p, 2p + 1), written as eight 32-bit (key pair) words into V^T.
  bf16x8 kr[2], vr[2];
  auto load_block = [&](int blk) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int ci = tid + 256 * j;
      int key = blk * PBN + (ci >> 3);
      key = key < key_max ? key : key_max;
      kr[j] = *reinterpret_cast<const bf16x8*>(kp + static_cast<int64_t>(key) * a.kv_ts + (ci & 7) * 8);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      int key = blk * PBN + 2 * (tid >> 3) + j;
      key = key < key_max ? key : key_max;
      vr[j] = *reinterpret_cast<const bf16x8*>(vp + static_cast<int64_t>(key) * a.kv_ts + (tid & 7) * 8);
    }
  };
  auto store_block = [&](int stage) {
    unsigned char* ks = smem + stage * PSTAGE;
    unsigned char* vs = ks + KT_BYTES;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int ci = tid + 256 * j;
      const int key = ci >> 3, ch = ci & 7;
      *reinterpret_cast<bf16x8*>(ks + key * 128 + ((ch ^ ((key >> 1) & 7)) << 4)) = kr[j];
    }
    // key r of the block = kb*32 + c*16 + u*8 + hh*4 + i sits at column kb*32 + c*16 + hh*8 + u*4 + i of V^T
    const int r0 = 2 * (tid >> 3);
    const int chunk = (r0 >> 5) * 4 + ((r0 >> 4) & 1) * 2 + ((r0 >> 2) & 1);
    const int within = ((r0 >> 3) & 1) * 4 + (r0 & 3);
    const int dc = tid & 7;
    typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;
    const u32x4 w0 = __builtin_bit_cast(u32x4, vr[0]), w1 = __builtin_bit_cast(u32x4, vr[1]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = dc * 8 + e;
      const unsigned word = (e & 1) ? ((w0[e >> 1] >> 16) | (w1[e >> 1] & 0xffff0000u)) : ((w0[e >> 1] & 0xffffu) | (w1[e >> 1] << 16));
      *reinterpret_cast<unsigned*>(vs + d * 128 + ((chunk ^ vt_swizzle(d)) << 4) + within * 2) = word;
    }
  };

  // ---- running state: lane = query; m in log2 units of the scaled logits
  const float c = a.sm_scale * kLog2e;
  float m_run[NH], l_run[NH];
  f32x16 o[NH][2];
#pragma unroll
  for (int hd = 0; hd < NH; ++hd) {
    m_run[hd] = -INFINITY;
    l_run[hd] = 0.f;
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[hd][db][r] = 0.f;
  }

  if (blk_lo < blk_hi) {
    load_block(blk_lo);
    store_block(0);
  }
  __syncthreads();

  for (int blk = blk_lo; blk < blk_hi; ++blk) {
    const int stage = (blk - blk_lo) & 1;
    const bool more = blk + 1 < blk_hi;
    if (more) load_block(blk + 1);

    const int key0 = blk * PBN;
    // does any of the wavefront's 32 queries see a key of this block?
    const bool active = key0 <= p0 + 31 && (a.window <= 0 || key0 + PBN - 1 >= p0 - a.window + 1);
    if (active) {
      const unsigned char* ks = smem + stage * PSTAGE;
      const unsigned char* vs = ks + KT_BYTES;
      // S^T[key, query]
      f32x16 s[NH][2];
#pragma unroll
      for (int hd = 0; hd < NH; ++hd)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) s[hd][kb][r] = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(ks + (kb * 32 + l31) * 128 + (((kk * 2 + h) ^ ((l31 >> 1) & 7)) << 4));
#pragma unroll
          for (int hd = 0; hd < NH; ++hd) s[hd][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[hd][kk], s[hd][kb], 0, 0, 0);
        }
      // mask where the block crosses the causal diagonal, the window's trailing edge or the end of the keys
      const bool full = key0 + PBN - 1 <= p0 && key0 + PBN - 1 < a.n_kv_ctx && (a.window <= 0 || key0 >= p0 + 31 - a.window + 1);
      if (!full) {
        const int qp = p0 + l31;
        const int upper = qp < a.n_kv_ctx - 1 ? qp : a.n_kv_ctx - 1;
        const int lower = a.window > 0 ? qp - a.window + 1 : -2147483647;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = key0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            const bool vis = key <= upper && key >= lower;
#pragma unroll
            for (int hd = 0; hd < NH; ++hd) s[hd][kb][r] = vis ? s[hd][kb][r] : -INFINITY;
          }
      }
      // online softmax, P^T in bf16 straight into operand registers
      bf16x8 pf[NH][2][2];
#pragma unroll
      for (int hd = 0; hd < NH; ++hd) {
        float mx = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[hd][kb][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run[hd], mx * c);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run[hd] - m_use);
        m_run[hd] = m_new;
        float lsum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s[hd][kb][r], c, -m_use));
            lsum += p;
            pf[hd][kb][r >> 3][r & 7] = static_cast<bf16>(p);
          }
        l_run[hd] = fmaf(l_run[hd], alpha, lsum);
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[hd][db][r] *= alpha;
      }
      // O^T[d, query] += V^T[d, keys] . P^T[keys, query]
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int cc = 0; cc < 2; ++cc) {
            const int d = db * 32 + l31;
            const bf16x8 vf = *reinterpret_cast<const bf16x8*>(vs + d * 128 + (((kb * 4 + cc * 2 + h) ^ vt_swizzle(d)) << 4));
#pragma unroll
            for (int hd = 0; hd < NH; ++hd) o[hd][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[hd][kb][cc], o[hd][db], 0, 0, 0);
          }
    }
    if (more) store_block(stage ^ 1);
    __syncthreads();
  }

  // ---- the sink joins the denominator; normalise; store (lane = query: 8-byte runs of four d)
  const int qrow = qw0 + l31;
#pragma unroll
  for (int hd = 0; hd < NH; ++hd) {
    const float l_tot = l_run[hd] + __shfl_xor(l_run[hd], 32, 64);
    const float sk = a.sinks ? static_cast<float>(a.sinks[head0 + hd]) * kLog2e : 0.f;
    const float m_f = fmaxf(m_run[hd], sk);
    const float so = __builtin_amdgcn_exp2f(m_run[hd] - m_f);
    const float inv = so / fmaf(l_tot, so, __builtin_amdgcn_exp2f(sk - m_f));
    if (qrow < a.n_q) {
      bf16* op = a.out + b * a.out_bs + static_cast<int64_t>(qrow) * a.out_ts + (head0 + hd) * 64 + 4 * h;
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          bf16x4 w;
#pragma unroll
          for (int i = 0; i < 4; ++i) w[i] = static_cast<bf16>(o[hd][db][4 * j + i] * inv);
          *reinterpret_cast<bf16x4*>(op + db * 32 + 8 * j) = w;
        }
    }
  }
}

}  // namespace tllm

using namespace tllm;

extern "C" int tllm_attention_prefill_bf16(const void* q, const void* k, const void* v, const void* sinks, void* out, int64_t q_batch_stride,
                                           int64_t q_token_stride, int64_t out_batch_stride, int64_t out_token_stride,
                                           int64_t kv_batch_stride, int64_t kv_token_stride, int64_t batch, int64_t n_q, int64_t n_kv_ctx,
                                           int n_kv_heads, int group, int head_dim, float sm_scale, int window, const void* start_q,
                                           int start_q_is_i64, void* stream) {
  TLLM_REQUIRE(batch >= 0 && n_q >= 0 && n_kv_ctx >= 1 && n_kv_heads >= 1, TLLM_E_SHAPE,
               "attention_prefill: batch %lld, n_q %lld, n_kv_ctx %lld, n_kv_heads %d", (long long)batch, (long long)n_q, (long long)n_kv_ctx,
               n_kv_heads);
  TLLM_REQUIRE(n_kv_ctx < (1ll << 30) && n_q < (1ll << 30), TLLM_E_SHAPE, "attention_prefill: n_q %lld / n_kv_ctx %lld too large",
               (long long)n_q, (long long)n_kv_ctx);
  TLLM_REQUIRE(head_dim == 64, TLLM_E_SHAPE, "attention_prefill: head_dim %d (only 64 is built)", head_dim);
  TLLM_REQUIRE(group >= 1 && group <= 64, TLLM_E_SHAPE, "attention_prefill: %d query heads per KV head (1..64)", group);
  TLLM_REQUIRE(window >= 0, TLLM_E_ARG, "attention_prefill: window %d", window);
  TLLM_REQUIRE(sm_scale > 0.f, TLLM_E_ARG, "attention_prefill: sm_scale %g must be positive", (double)sm_scale);
  if (batch == 0 || n_q == 0) return TLLM_OK;
  TLLM_REQUIRE(q && k && v && out && start_q, TLLM_E_ARG, "attention_prefill: q, k, v, out and start_q must not be NULL");
  const int64_t n_heads = static_cast<int64_t>(n_kv_heads) * group;
  TLLM_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out) && q_batch_stride % 8 == 0 && q_token_stride % 8 == 0 &&
                   out_batch_stride % 8 == 0 && out_token_stride % 8 == 0 && kv_batch_stride % 8 == 0 && kv_token_stride % 8 == 0,
               TLLM_E_ALIGN, "attention_prefill: q, k, v, out must be 16-byte aligned with strides that are multiples of 8 elements");
  TLLM_REQUIRE(q_token_stride >= n_heads * 64 && out_token_stride >= n_heads * 64, TLLM_E_ARG,
               "attention_prefill: q / out token stride < n_heads * 64");
  TLLM_REQUIRE(kv_token_stride >= static_cast<int64_t>(n_kv_heads) * 64, TLLM_E_ARG, "attention_prefill: kv_token_stride < n_kv_heads * 64");
  AttnPrefillArgs a{};
  a.q = (const bf16*)q;
  a.k = (const bf16*)k;
  a.v = (const bf16*)v;
  a.sinks = (const bf16*)sinks;
  a.out = (bf16*)out;
  a.start_q = start_q;
  a.start_is_i64 = start_q_is_i64;
  a.q_bs = q_batch_stride;
  a.q_ts = q_token_stride;
  a.out_bs = out_batch_stride;
  a.out_ts = out_token_stride;
  a.kv_bs = kv_batch_stride;
  a.kv_ts = kv_token_stride;
  a.batch = (int)batch;
  a.n_q = (int)n_q;
  a.n_kv_ctx = (int)n_kv_ctx;
  a.n_kv_heads = n_kv_heads;
  a.group = group;
  a.window = window;
  a.sm_scale = sm_scale;
  const int nh = group % 2 == 0 ? 2 : 1;
  const int64_t ntiles = (n_q + PBM - 1) / PBM;
  const int64_t wgs = ntiles * batch * n_kv_heads * (group / nh);
  TLLM_REQUIRE(batch < (1ll << 24) && wgs < (1ll << 31), TLLM_E_SHAPE, "attention_prefill: %lld workgroups are too many for one launch", (long long)wgs);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (nh == 2)
    hipLaunchKernelGGL(attn_prefill_kernel<2>, dim3((unsigned)wgs), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL(attn_prefill_kernel<1>, dim3((unsigned)wgs), dim3(256), 0, st, a);
  return check_launch("attention_prefill");
}
