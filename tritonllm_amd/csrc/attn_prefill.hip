// Prefill attention with learned sinks and an optional sliding window: many query positions per batch row against
// the keys written so far (attention, attention_tt.py:167-242; kernel :17-164; definition attention_ref.py:4-42):
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
//     K / V blocks of 64 keys pass through four LDS stages filled by global_load_lds_dwordx4 (no staging registers, no
//     LDS writes; three blocks in flight behind the one being computed, one hand-spelled wait + barrier per block)
//     and serve all NH heads;
//   * S^T = K . Q^T on v_mfma_f32_32x32x16_bf16 with the keys on M: a lane then owns ONE query (column) and 16 keys
//     per 32-key block, so the running maximum, the running sum and the rescale factor of the online softmax are
//     lane-local apart from one exchange between the two half-wavefronts;
//   * those accumulator registers are, pairwise, the B operand (P^T) of O^T = V^T . P^T when the MFMA's k slots are read
//     as a permutation of the block's keys, so P never leaves the registers; V stays row-major in LDS and the A operand
//     (V^T: lane = d, 8 keys) comes out of two transposing reads (ds_read_b64_tr_b16: within 16 lanes, lane i receives
//     element i % 4 of the 8 bytes addressed by lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4);
//   * the running maximum is only raised when a block exceeds it by more than 2^8 (exponents stay far from overflow, the
//     result is the same quotient), so the accumulator is almost never rescaled; the weights are summed, as the bf16
//     values the MFMA multiplies with, two per v_dot2c_f32_bf16;
//   * both tiles are XOR-swizzled in 16-byte chunks: fragment reads are conflict-free (K) or at the two-pass minimum (V);
//   * the KV head is the fastest-varying part of the workgroup index, so with eight KV heads each XCD's L2 holds the
//     K and V of one head; the query tiles with the most keys to visit are launched first.
// start_q is read from device memory (int32 or int64).
#include "common.h"

namespace tllm {

struct AttnPrefillArgs {
  const bf16* q;          // [B, n_q, n_heads, 64]: batch stride q_bs, token stride q_ts (elements), heads adjacent
  const bf16* k;          // [B, n_kv_ctx, n_kv_heads, 64]: batch stride kv_bs, token stride kv_ts
  const bf16* v;
  const bf16* sinks;      // [n_heads] or null (logit 0, attention_tt.py:100-104)
  bf16* out;              // [B, n_q, n_heads * 64]: batch stride out_bs, token stride out_ts
  const void* start_q;    // device scalar
  int start_is_i64;
  int64_t q_bs, q_ts, out_bs, out_ts, kv_bs, kv_ts;
  int batch, n_q, n_kv_ctx, n_kv_heads, group, window;
  float sm_scale;
};

namespace {
constexpr int PBN = 64;               // keys per block
constexpr int KT_BYTES = PBN * 128;   // K tile [key][64 d]
constexpr int VT_BYTES = PBN * 128;   // V tile [key][64 d]
constexpr int PSTAGE = KT_BYTES + VT_BYTES;
constexpr int NSTG = 4;               // LDS stages: three blocks in flight behind the one being computed
constexpr float kLog2e = 1.4426950408889634f;
}  // namespace

constexpr float kRaise = 8.f;         // log2 units by which a block must exceed the running maximum to move it

// 16-byte chunk swizzle of a V row: a transposing read touches eight consecutive keys x 64 bytes; this spreads them
// over the banks evenly.
__device__ __forceinline__ int v_swizzle(int key) { return (((key >> 1) & 1) << 2) | ((key >> 2) & 3); }

// The value lane l ^ 32 holds: lanes l and l ^ 32 carry the two halves of one query's keys.
__device__ __forceinline__ float other_half(float x, int high) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);   // r[0]: the low half's x in every lane, r[1]: the high half's
  return __builtin_bit_cast(float, high ? r[0] : r[1]);
}

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short i16x4;

// NH: query heads (of one KV head) per wavefront. QG: groups of 32 queries per workgroup; the four wavefronts are QG
// query groups x 4 / QG head sets, so a workgroup covers 32 * QG queries of NH * 4 / QG heads.
template <int NH, int QG>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(AttnPrefillArgs a) {
  constexpr int PBM = 32 * QG;                    // queries per workgroup
  constexpr int HS = 4 / QG;                      // head sets
  constexpr int DPT = 4;                          // global->LDS load instructions per wavefront and block (1 KB each)
  __shared__ __align__(16) unsigned char smem[NSTG * PSTAGE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, h = lane >> 5;

  // workgroup -> (kv head, head sub-group, batch row, query tile); kv head fastest. Long tiles go first; when the whole
  // launch is resident at once (two workgroups per CU), the second workgroup of each CU is taken in the opposite
  // order, so a CU that got a long tile gets a short one next to it.
  const int nsub = a.group / (NH * HS);
  const int ntiles = (a.n_q + PBM - 1) / PBM;
  unsigned id = blockIdx.x;
  const int kvh = id % a.n_kv_heads;
  id /= a.n_kv_heads;
  {
    const unsigned per_round = 256 / (a.n_kv_heads < 256 ? a.n_kv_heads : 256);      // first workgroups of the CUs, per KV head
    const unsigned n = gridDim.x / a.n_kv_heads;
    if (per_round > 0 && n <= 2 * per_round && id >= per_round) id = n + per_round - 1 - id;
  }
  const int sub = id % nsub;
  id /= nsub;
  const int b = id % a.batch;
  id /= a.batch;
  const int tile = ntiles - 1 - static_cast<int>(id);
  const int head0 = kvh * a.group + (sub * HS + wave / QG) * NH;

  // ---- Q fragments (B operand: lane = query, 8 d per half-wavefront and k16 step), requested before the start
  // position is read: their addresses do not depend on it, so they travel while that (dependent) load is on its way
  const int q0 = tile * PBM;
  const int qw0 = q0 + (wave % QG) * 32;   // the wavefront's first query
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

  const int start = a.start_is_i64 ? static_cast<int>(*reinterpret_cast<const int64_t*>(a.start_q)) : *reinterpret_cast<const int*>(a.start_q);
  const int p0 = start + qw0;              // the position of the wavefront's first query
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

  // ---- K / V block movers: global_load_lds_dwordx4 (no staging registers, no LDS writes). One instruction fills
  // 1 KB = 8 tile rows, the lanes' 16 bytes landing at M0 + 16 * lane; the swizzle is applied by choosing which chunk of
  // the row a lane fetches. A stage is the K tile followed by the V tile, so a wavefront's DPT instructions all belong
  // to one of the two.
  const bool dma_v = wave * DPT >= 8;
  const bf16* dma_src = dma_v ? vp : kp;
  int dma_row[DPT], dma_col[DPT];
  const bf16* dma_ptr[DPT];                       // the lane's chunk of its row of key block 0
#pragma unroll
  for (int j = 0; j < DPT; ++j) {
    const int row = ((wave * DPT + j) & 7) * 8 + (lane >> 3);
    dma_row[j] = row;
    dma_col[j] = ((lane & 7) ^ (dma_v ? v_swizzle(row) : ((row >> 1) & 7))) * 8;
    dma_ptr[j] = dma_src + static_cast<int64_t>(row) * a.kv_ts + dma_col[j];
  }
  const unsigned lds0 = static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem)) + wave * DPT * 1024;
  const int64_t blk_stride = static_cast<int64_t>(PBN) * a.kv_ts;
  auto issue_block = [&](int blk, int stage) {
    const bool whole = blk * PBN + PBN - 1 <= key_max;       // no row of the block lies beyond the last visible key
#pragma unroll
    for (int j = 0; j < DPT; ++j) {
      const bf16* g;
      if (whole) {
        g = dma_ptr[j] + blk * blk_stride;
      } else {
        int key = blk * PBN + dma_row[j];
        key = key < key_max ? key : key_max;
        g = dma_src + static_cast<int64_t>(key) * a.kv_ts + dma_col[j];
      }
      const unsigned m0v = lds0 + stage * PSTAGE + j * 1024;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0v), "v"(g) : "memory", "m0");
    }
  };
  // wait until all but the `behind` youngest blocks' loads of this wavefront have landed, then meet the others
  auto wait_and_meet = [&](int behind) {
    if (behind >= 2)
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * DPT) : "memory");
    else if (behind == 1)
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(DPT) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  };

  // K fragment (A operand of S^T): lane = key l31 of a 32-key half, 16 bytes at d = kk*16 + h*8
  const int k_row = l31 * 128, k_sw = (l31 >> 1) & 7;
  // V^T fragment (A operand of O^T): lane = d; the transposing read wants from lane j of each 16 the address of
  // four d (quad j % 4 of the lane group's 16) of key j / 4 of the four keys this half-wavefront takes
  const int v_key = 4 * h + ((lane & 15) >> 2);                       // + 16*cc + 8*u + 32*kb
  const int v_d = (l31 & 16) + 4 * (lane & 3);                        // + 32*db

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

  const int nblk = blk_hi - blk_lo;
#pragma unroll
  for (int i = 0; i < 2; ++i)
    if (i < nblk) issue_block(blk_lo + i, i);

  {
    // The compiler does not see the direct-to-LDS loads in its count of outstanding loads; were the fragments first
    // used inside the loop, its wait for them there would be "nothing outstanding" and drain the blocks in flight on
    // every step. Pin the wait here, where the first blocks have to land anyway.
#pragma unroll
    for (int hd = 0; hd < NH; ++hd)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) asm volatile("" : "+v"(qf[hd][kk]));
  }

  wait_and_meet(0);                              // blocks 0 and 1 have landed

  auto process = [&](int blk, int stage) __attribute__((always_inline)) {
    const int key0 = blk * PBN;
    // does any of the wavefront's 32 queries see a key of this block?
    const bool active = key0 <= p0 + 31 && (a.window <= 0 || key0 + PBN - 1 >= p0 - a.window + 1);
    if (active) {
      const unsigned char* ks = smem + stage * PSTAGE;
      const unsigned char* vs = ks + KT_BYTES;
      // S^T[key, query]
      f32x16 s[NH][2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(ks + kb * 32 * 128 + k_row + (((kk * 2 + h) ^ k_sw) << 4));
#pragma unroll
          for (int hd = 0; hd < NH; ++hd) {
            if (kk == 0) {
              const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
              s[hd][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[hd][kk], zero, 0, 0, 0);
            } else {
              s[hd][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[hd][kk], s[hd][kb], 0, 0, 0);
            }
          }
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
      // online softmax. First the block maxima of all heads and ONE (rare) branch that raises running maxima; what
      // follows is then a single straight-line region in which the exponentials of one (head, 32-key half) and the
      // P.V MFMAs of the one before it can be issued in turn.
      bool raise[NH];
      float mx[NH];
      bool any = false;
#pragma unroll
      for (int hd = 0; hd < NH; ++hd) {
        float t = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) t = fmaxf(t, s[hd][kb][r]);
        mx[hd] = fmaxf(t, other_half(t, h)) * c;
        // the maximum moves only when this block tops it by more than kRaise: p stays below 2^kRaise otherwise
        raise[hd] = mx[hd] > m_run[hd] + kRaise;                  // false while mx is -inf (nothing visible yet)
        any = any || raise[hd];
      }
      if (__builtin_amdgcn_ballot_w64(any) != 0) {
#pragma unroll
        for (int hd = 0; hd < NH; ++hd) {
          const float m_new = raise[hd] ? mx[hd] : m_run[hd];
          const float alpha = raise[hd] ? __builtin_amdgcn_exp2f(m_run[hd] - m_new) : 1.f;     // -inf - finite: 0
          m_run[hd] = m_new;
          l_run[hd] *= alpha;
#pragma unroll
          for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[hd][db][r] *= alpha;
        }
      }
      const bf16x2 one2 = {static_cast<bf16>(1.0f), static_cast<bf16>(1.0f)};
#pragma unroll
      for (int hd = 0; hd < NH; ++hd) {
        const float m_use = m_run[hd] == -INFINITY ? 0.f : m_run[hd];
        float lsum = l_run[hd];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          // P^T in bf16 straight into operand registers
          bf16x8 pf[2];
#pragma unroll
          for (int r = 0; r < 16; ++r) pf[r >> 3][r & 7] = static_cast<bf16>(__builtin_amdgcn_exp2f(fmaf(s[hd][kb][r], c, -m_use)));
          // the denominator sums the rounded weights the numerator's MFMA multiplies with, two per instruction
#pragma unroll
          for (int cc = 0; cc < 2; ++cc) {
            lsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(pf[cc], pf[cc], 0, 1), one2, lsum, false);
            lsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(pf[cc], pf[cc], 2, 3), one2, lsum, false);
            lsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(pf[cc], pf[cc], 4, 5), one2, lsum, false);
            lsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(pf[cc], pf[cc], 6, 7), one2, lsum, false);
          }
          // O^T[d, query] += V^T[d, keys] . P^T[keys, query]
#pragma unroll
          for (int cc = 0; cc < 2; ++cc)
#pragma unroll
            for (int db = 0; db < 2; ++db) {
              i16x4 part[2];
#pragma unroll
              for (int u = 0; u < 2; ++u) {
                const int key = kb * 32 + cc * 16 + u * 8 + v_key;
                const int d = db * 32 + v_d;
                part[u] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) i16x4*)(vs + key * 128 + (((d >> 3) ^ v_swizzle(key)) << 4) + (d & 7) * 2));
              }
              typedef __attribute__((__vector_size__(8 * sizeof(short)))) short i16x8;
              const i16x8 both = __builtin_shufflevector(part[0], part[1], 0, 1, 2, 3, 4, 5, 6, 7);
              o[hd][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pf[cc], o[hd][db], 0, 0, 0);
            }
        }
        l_run[hd] = lsum;
      }
    }
  };

  // Two blocks per step: the step's loads refill the two stages the previous step read (every wavefront has left it),
  // have two blocks of arithmetic to land behind, and are met with one wait + barrier.
  for (int i = 0; i < nblk; i += 2) {
#pragma unroll
    for (int j = 2; j < 4; ++j)
      if (i + j < nblk) issue_block(blk_lo + i + j, (i + j) & (NSTG - 1));
    process(blk_lo + i, i & (NSTG - 1));
    if (i + 1 < nblk) process(blk_lo + i + 1, (i + 1) & (NSTG - 1));
    wait_and_meet(0);
  }

  // ---- the sink joins the denominator; normalise. A lane holds 8-byte runs of ONE query's row, so storing from here
  // would be 64 scattered 8-byte writes per instruction (measured: ~3 us of a workgroup's life). The wavefront's
  // 32 x (NH x 64) tile goes through its own patch of the now idle stages instead and leaves as whole 128-byte rows.
  constexpr int OROW = NH * 128 + 16;            // patch row: the NH heads of a query + padding (2-way conflicts at most)
  unsigned char* patch = smem + wave * (32 * OROW);
#pragma unroll
  for (int hd = 0; hd < NH; ++hd) {
    const float l_tot = l_run[hd] + other_half(l_run[hd], h);
    const float sk = a.sinks ? static_cast<float>(a.sinks[head0 + hd]) * kLog2e : 0.f;
    const float m_f = fmaxf(m_run[hd], sk);
    const float so = __builtin_amdgcn_exp2f(m_run[hd] - m_f);
    const float inv = so / fmaf(l_tot, so, __builtin_amdgcn_exp2f(sk - m_f));
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        bf16x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = static_cast<bf16>(o[hd][db][4 * j + i] * inv);
        *reinterpret_cast<bf16x4*>(patch + l31 * OROW + hd * 128 + (db * 32 + 8 * j + 4 * h) * 2) = w;
      }
  }
  // 16-byte chunks in row-major order: eight lanes per 128-byte head row, NH x 8 per query
  bf16* ob = a.out + b * a.out_bs + head0 * 64;
#pragma unroll
  for (int it = 0; it < NH * 4; ++it) {
    const int idx = it * 64 + lane;
    const int row = idx / (NH * 8), ch = idx % (NH * 8);
    const bf16x8 w = *reinterpret_cast<const bf16x8*>(patch + row * OROW + ch * 16);
    if (qw0 + row < a.n_q) *reinterpret_cast<bf16x8*>(ob + static_cast<int64_t>(qw0 + row) * a.out_ts + ch * 8) = w;
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
  // Workgroup shape: 128 queries x 2 heads (two heads per wavefront) as soon as that gives every CU two workgroups;
  // below that 64 queries x 2 heads with one head per wavefront: twice the workgroups, and the longest of them -- it
  // sets the time of so small a launch -- takes about half as long per key block (one prompt of 1024 tokens: 28.8 ->
  // 21.4 us; at 2048 tokens, 512 workgroups of the large shape, the two are level). Odd group sizes: 128 x 1.
  const int nh = group % 2 == 0 ? 2 : 1;
  const int64_t wgs128 = (n_q + 127) / 128 * batch * n_kv_heads * (group / nh);
  const bool small = nh == 2 && wgs128 < 512;
  const int64_t wgs = small ? (n_q + 63) / 64 * batch * n_kv_heads * (group / 2) : wgs128;
  TLLM_REQUIRE(batch < (1ll << 24) && wgs < (1ll << 31), TLLM_E_SHAPE, "attention_prefill: %lld workgroups are too many for one launch", (long long)wgs);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (small)
    hipLaunchKernelGGL((attn_prefill_kernel<1, 2>), dim3((unsigned)wgs), dim3(256), 0, st, a);
  else if (nh == 2)
    hipLaunchKernelGGL((attn_prefill_kernel<2, 4>), dim3((unsigned)wgs), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((attn_prefill_kernel<1, 4>), dim3((unsigned)wgs), dim3(256), 0, st, a);
  return check_launch("attention_prefill");
}
