// Decode attention with learned sinks and an optional sliding window, one new token per batch row against the KV
// cache (attention_decode, attention_tt_decode.py:290-408; kernels :9-287; definition attention_ref.py:4-42):
//
//   keys lo .. hi-1 with hi = min(start_q + 1, n_kv_ctx), lo = window ? max(0, start_q - window + 1) : 0
//   s[h, n]  = sm_scale * <q[h], k[n]>                       h = kv_head * G + g   (G query heads share a KV head)
//   out[h]   = sum_n exp(s[h, n] - m) v[n] / (sum_n exp(s[h, n] - m) + exp(sink[h] - m)),   m = max(sink[h], max_n s[h, n])
//
// The reference runs one program per query head, so the G heads of a group each read the same K and V; here a
// wavefront serves all G heads of a KV head from one pass over K and V, in one of two workgroup shapes:
//   * ROWS (large batch x context): a workgroup takes a (batch row, context split, group of eight or four adjacent
//     KV heads) and has one wavefront per KV head, each walking the split's 32-key blocks in order. Together the
//     wavefronts read whole (or half) cache rows -- all KV heads of a token are adjacent in memory -- so the workgroup
//     streams long contiguous runs of K and of V; with nontemporal loads the whole-row pattern measures 6.8 TB/s on
//     its own, where one-KV-head-per-workgroup streams stop at 5.2 TB/s (128-byte pieces at a 1 KB stride, the
//     sibling heads arriving from other workgroups at other times);
//   * HEAD (few batch rows): a workgroup takes a (batch row, KV head, context split); four wavefronts take the
//     split's blocks in turn, each with its own running (max, sum, accumulator), and meet once at the end through
//     LDS. This shape yields n_kv_heads times more workgroups, which is what fills the machine at batch 1;
//   * S^T = K . Q^T on v_mfma_f32_16x16x32_bf16 with the keys on M: K rows are K-contiguous in memory, so a lane
//     loads its 16 bytes of a key row straight into operand layout; Q sits in registers as the B operand;
//   * the accumulator layout of S^T (lane = head, registers = keys) IS the A-operand layout of P for O = P . V when
//     the MFMA's k slots are read as a permutation of the block's keys, so P never leaves the registers; V, whose
//     rows are d-contiguous, goes through a wavefront-private LDS tile and is gathered in that same key order;
//   * the per-head rescale factor exp(m_old - m_new) lives in the S^T layout and is fetched into the O layout
//     (registers = heads) by ds_bpermute;
//   * with more than one context split the workgroups leave (max, sum, accumulator) in a workspace and a second
//     small kernel folds them and the sink.
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
  int n_kv_ctx, n_kv_heads, group, window;
  int splits;             // planned on the host (grid size, workspace stride); the kernels use no more than the context needs
  int fill, keys_shift;   // the planning inputs that do not depend on the context: splits that fill the CUs, log2 of the target keys per workgroup
  float sm_scale;
};

// Context splits for `units` independent (batch row, head group) streams over `ctx` visible keys: first enough
// workgroups to fill the 256 CUs, beyond that about keys_per_wg keys each, never less than 128 keys per split, at most
// 64. The host plans the launch with it from the size of the cache (or the caller's hint of the current length); the
// kernels evaluate it again with the length they read from start_q and leave the splits beyond that idle, so a cache
// allocated for 131072 tokens costs a context of 4096 no more splits than it needs.
__host__ __device__ inline int attn_fill(int64_t units) { return static_cast<int>((256 + (units > 0 ? units : 1) - 1) / (units > 0 ? units : 1)); }

__host__ __device__ inline int attn_splits_for(int fill, int ctx, int keys_shift) {   // a few 32-bit shifts and compares: the kernels run this
  const int cap = ((ctx - 1) >> 7) + 1;                        // ctx >= 1
  const int by_work = ((ctx - 1) >> keys_shift) + 1;
  int s = fill > by_work ? fill : by_work;
  s = s < cap ? s : cap;
  s = s > 1 ? s : 1;
  return s < 64 ? s : 64;
}

namespace {
constexpr int AW = 4;                 // wavefronts per workgroup, HEAD shape
constexpr int RW = 8;                 // most wavefronts (= KV heads) per workgroup, ROWS shape
constexpr int VROW = 128 + 16;        // V tile row in LDS: 64 bf16 + padding, bytes
constexpr int VTILE = 32 * VROW;
constexpr float kNegBig = -1.0e30f;
constexpr int PART = 66;              // floats per (split, row, head) in the workspace
}  // namespace

__device__ __forceinline__ int attn_start_q(const AttnArgs& a) {
  return a.start_is_i64 ? static_cast<int>(*reinterpret_cast<const int64_t*>(a.start_q)) : *reinterpret_cast<const int*>(a.start_q);
}

// Visible keys lo .. hi-1 and the number of splits that take part (<= the planned a.splits).
__device__ __forceinline__ int attn_live_splits(const AttnArgs& a, int* lo_out, int* hi_out) {
  const int start_q = attn_start_q(a);
  int hi = start_q + 1 < a.n_kv_ctx ? start_q + 1 : a.n_kv_ctx;
  hi = hi > 0 ? hi : 0;
  int lo = a.window > 0 ? (start_q - a.window + 1 > 0 ? start_q - a.window + 1 : 0) : 0;
  lo = lo < hi ? lo : hi;
  *lo_out = lo;
  *hi_out = hi;
  const int s = attn_splits_for(a.fill, hi - lo > 0 ? hi - lo : 1, a.keys_shift);
  return s < a.splits ? s : a.splits;
}

template <bool ROWS>
__global__ __launch_bounds__((ROWS ? RW : AW) * 64) void attn_decode_kernel(AttnArgs a) {
  __shared__ __align__(16) unsigned char vt[(ROWS ? RW : AW) * VTILE];
  __shared__ __align__(16) unsigned char kt[(ROWS ? RW : AW) * VTILE];   // K tile, the same shape
  __shared__ float s_m[ROWS ? 1 : AW][16], s_l[ROWS ? 1 : AW][16];
  __shared__ float s_acc[ROWS ? 1 : AW][ROWS ? 1 : 16][64 + 1];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int G = a.group;
  const int n_q_heads = a.n_kv_heads * G;

  // ---- key range of this split; the splits the context does not need leave at once (the whole workgroup)
  // The grid is (head groups x planned splits, batch rows), x fastest. When the context needs fewer splits than were
  // planned, the workgroups are renumbered so that the live ones are the first live x groups x batch in launch order
  // -- they then spread over the CUs exactly as a launch planned for this context would, and the rest exit at once
  // (left where they were launched, live and idle workgroups pile up unevenly: 140 against 89 us at B = 8 with
  // 32768 of a 131072-token cache in use).
  int lo, hi;
  const int live = attn_live_splits(a, &lo, &hi);
  int grp, split;
  int64_t b;
  if (live == a.splits) {
    grp = blockIdx.x / a.splits;
    split = blockIdx.x - grp * a.splits;
    b = blockIdx.y;
  } else {
    const unsigned ngrp = gridDim.x / a.splits;
    const unsigned idx = blockIdx.y * gridDim.x + blockIdx.x, per_row = live * ngrp;
    if (idx >= per_row * gridDim.y) return;
    const unsigned bb = idx / per_row, r = idx - bb * per_row;
    b = bb;
    grp = r / live;
    split = r - grp * live;
  }
  // ROWS: the group's KV heads sit on the workgroup's wavefronts
  const int kvh = ROWS ? grp * static_cast<int>(blockDim.x >> 6) + wave : grp;
  const int len = hi - lo;
  int chunk = (len + live - 1) / live;
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
  unsigned char* ktile = kt + wave * VTILE;

  float m_run = kNegBig, l_run = 0.f;                          // of head r16 (replicated over the four lane groups)
  f32x4_t acc[4];                                              // O: lane (d = 16 nb + r16, heads 4 g + i)
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) acc[nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // A operands of a block: K[key = k0 + 16 kb + r16][32 t + 8 g ..]; V tile chunks: key (i*64+lane)/8, chunk (i*64+lane)%8.
  // Rows past the end of the split are clamped to its last key (finite values; their probabilities are zeroed).
  // Addressing is a block base (uniform) plus a 32-bit lane offset: row * token stride + a lane constant.
  const unsigned ts_b = static_cast<unsigned>(a.kv_ts) * 2u;   // token stride, bytes (a 32-key block spans < 4 GB)
  // The ROWS stream is read once and is far larger than the caches: nontemporal. The HEAD shape serves short
  // contexts, where the cache lines of a token are shared with sibling workgroups and may still be cache-resident.
  auto ld = [](const unsigned char* p) {
    return ROWS ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p)) : *reinterpret_cast<const bf16x8*>(p);
  };
  // K and V both arrive row-major, eight neighbouring lanes covering one 128-byte row piece; K's A-operand fragments
  // (lane = (key, k group)) are then read out of LDS. Loaded straight into operand layout, neighbouring lanes ask for
  // different rows -- 64 requests of 16 bytes per instruction, which the memory side serves at three quarters of the rate.
  bf16x8 kr[4], vr[4];
  auto load_block = [&](int k0) {
    const int last = s_hi - k0 - 1;                            // last valid row of the block (>= 31 except in the final one)
    const unsigned char* kb0 = reinterpret_cast<const unsigned char*>(kbase + static_cast<int64_t>(k0) * a.kv_ts);
    const unsigned char* vb0 = reinterpret_cast<const unsigned char*>(vbase + static_cast<int64_t>(k0) * a.kv_ts);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = i * 64 + lane;
      const int r = c >> 3;
      const unsigned off = static_cast<unsigned>(r < last ? r : last) * ts_b + 16u * (c & 7);
      kr[i] = ld(kb0 + off);
      vr[i] = ld(vb0 + off);
    }
  };

  constexpr int STEP = ROWS ? 1 : AW;                          // ROWS: every wavefront walks all blocks (of its own KV head)
  const int first = ROWS ? 0 : wave;
  if (first < nblk) load_block(s_lo + 32 * first);
  for (int blk = first; blk < nblk; blk += STEP) {
    const int k0 = s_lo + 32 * blk;
    // ---- S^T for the block's two 16-key halves
    // K and V tiles into LDS (row-major, as loaded)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = i * 64 + lane;
      *reinterpret_cast<bf16x8*>(ktile + (c >> 3) * VROW + (c & 7) * 16) = kr[i];
      *reinterpret_cast<bf16x8*>(vtile + (c >> 3) * VROW + (c & 7) * 16) = vr[i];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f32x4_t st[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const unsigned char* krow = ktile + (16 * kb + r16) * VROW + 16 * g;
      const bf16x8 ka0 = *reinterpret_cast<const bf16x8*>(krow), ka1 = *reinterpret_cast<const bf16x8*>(krow + 64);
      st[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka0, qb0, f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      st[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka1, qb1, st[kb], 0, 0, 0);
    }
    // The next block's loads go out before this one's arithmetic. Unconditional (a load under a branch makes the
    // compiler wait for it where the paths join): the last round simply requests its own block again.
    load_block(s_lo + 32 * (blk + STEP < nblk ? blk + STEP : blk));

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
    bmax = max_over_lane_bits_16_32(bmax);
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
    psum = sum_over_lane_bits_16_32(psum);
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

  if constexpr (ROWS) {
    // ---- each wavefront owns its heads outright: O sits in lane (d = 16 nb + r16), registers = heads 4 g + i; the
    // (max, sum) of head h sit in the lanes with r16 == h
    float* p = a.part + ((static_cast<int64_t>(split) * gridDim.y + b) * n_q_heads + static_cast<int64_t>(kvh) * G) * PART;
    if (a.splits > 1 && g == 0 && r16 < G) {
      p[r16 * PART + 64] = m_run;
      p[r16 * PART + 65] = l_run;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int hh = 4 * g + i;
      const float m_h = __shfl(m_run, hh, 64), l_h = __shfl(l_run, hh, 64);
      if (hh >= G) continue;
      if (a.splits > 1) {
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) p[hh * PART + 16 * nb + r16] = acc[nb][i];
      } else {
        const int head = kvh * G + hh;
        const float sink = a.sinks ? static_cast<float>(a.sinks[head]) : 0.f;
        const float m_f = fmaxf(m_h, sink);
        const float f = __expf(m_h - m_f);
        const float z = l_h * f + __expf(sink - m_f);
        bf16* orow = a.out + b * a.out_rs + static_cast<int64_t>(head) * 64;
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) orow[16 * nb + r16] = static_cast<bf16>(acc[nb][i] * f / z);
      }
    }
    return;
  }

  // ---- HEAD: the four wavefronts meet: (max, sum) per head, accumulator per (head, d)
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
  // (max, sum) of every planned split and the accumulators of the first eight are requested before start_q is known
  // (one memory round trip for up to eight splits, not three); the records of splits that did not take part are
  // whatever the workspace held and are masked out once the number of live splits is known.
  const float m_raw = lane < a.splits ? p0[lane * split_stride + 64] : kNegBig;
  const float l_raw = lane < a.splits ? p0[lane * split_stride + 65] : 0.f;
  float v[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) v[u] = p0[(u < a.splits ? u : a.splits - 1) * split_stride + lane];
  int lo, hi;
  const int live = attn_live_splits(a, &lo, &hi);            // the splits that wrote a record
  const bool has = lane < live;
  const float m_s = has ? m_raw : kNegBig;
  const float l_s = has ? l_raw : 0.f;
  const float m_all = wave_max(m_s);
  const float f_s = __expf(m_s - m_all);                     // 0 for the lanes without a split
  const float l_all = wave_sum(l_s * f_s);
  float o = 0.f;
  for (int s0 = 0; s0 < live; s0 += 8) {
    if (s0 > 0) {
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = p0[(s0 + u < live ? s0 + u : live - 1) * split_stride + lane];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      // the split index is the same in every lane: a scalar lane read, not a trip through the LDS crossbar
      const float f = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f_s),
                                                                          __builtin_amdgcn_readfirstlane(s0 + u < live ? s0 + u : 0)));
      o += (s0 + u < live) ? v[u] * f : 0.f;
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

// Workgroup shape and context splits, from measurements at B = 1 .. 32, contexts 1K - 128K.
// ROWS (a workgroup per (batch row, split, group of 8 or 4 KV heads), one wavefront per KV head) streams faster but
// yields fewer workgroups, each wavefront walking its blocks one after the other: it is taken when it still gives
// every CU a workgroup with at least 512 keys per split, in the head grouping that makes the splits longest
// (us, HEAD -> ROWS: B = 8 at 32K 106 -> 86, at 8K 33 -> 27; B = 32 at 4K 56 -> 47;
// B = 16 at 4K 32 -> 27; B = 4 at 32K 61 -> 47, at 16K 34 -> 28; B = 2 at 32K 34 -> 30, at 16K 18 -> 20 (HEAD kept);
// B = 1: HEAD throughout) -- and with splits of 256 keys and more when those are at most 28 (32 from 320 keys on)
// and the HEAD shape would split the context as well (a HEAD launch that needs no second kernel stays ahead):
// B = 8 at 4K 16.7 -> 16.1, at 5K 21.0 -> 18.4, at 6K 24.7 -> 20.9, at 7K 27.4 -> 23.1; B = 16 at 2K 17.4 -> 15.8, at
// 3K 24.4 -> 20.6; B = 24 at 2K 29.3 -> 25.2, at 1.5K 22.2 -> 20.6; B = 12 at 4K 29.1 -> 26.0; B = 5 at 8K 26.9 -> 23.6,
// at 10K 30.9 -> 27.3; B = 6 at 8K 29.2 -> 26.4; B = 4 at 12K 24.8 -> 21.9 (with 32 splits of 256 keys, B = 4 at 8K:
// 16.7 -> 17.2, and with 64, B = 2 at 16K: 17.0 -> 19.2 -- HEAD kept; B = 32 at 1K, where HEAD needs one launch:
// 14.2 -> 16.4, HEAD kept; splits of 128-255 keys: 0-6 % slower than HEAD; two KV heads per workgroup: 20-30 % slower
// than either shape wherever it would be chosen). Splits: first enough workgroups to fill the 256 CUs, beyond that about 4096 (ROWS) /
// 2048 (HEAD) keys per workgroup, never less than 128 keys per split -- and one split fewer per stream where that
// spreads the workgroups more evenly over the CUs (attn_pick_splits). Against 1024 keys per ROWS workgroup and no
// such balancing: B = 8 at 32K 85.2 -> 79.8, at 64K 174.6 -> 160.3, at 128K 333 -> 321; B = 32 at 8K 84.5 -> 79.5;
// B = 12 at 4K 25.9 -> 20.9, at 8K 44.7 -> 35.5, at 12K 61.3 -> 49.4, at 20K 81.9 -> 76.4; B = 5 / 6 / 7 at 8K
// 23.6 / 26.2 / 29.2 -> 19.6 / 21.4 / 23.9, at 4K 14.7 / 16.5 / 18.3 -> 13.2 / 14.7 / 14.8; B = 10 at 4K 22.8 -> 18.6;
// B = 20 at 3K 29.9 -> 24.1; B = 24 at 2K 25.0 -> 20.6; B = 28 at 1280 keys 21.4 -> 17.6; B = 3 at 100K 106 -> 97;
// unchanged (within 0.3 %) at the other 30 of 48 batch x context points tried.
// A sliding window bounds the context.
struct AttnPlan { int heads_per_wg; int splits; int fill; int keys_shift; };   // heads_per_wg 0: the HEAD shape

constexpr int kRowsKeysShift = 12, kHeadKeysShift = 11;   // log2 of the keys per workgroup beyond which a context is split further
// Splits for `units` streams: attn_splits_for's answer, unless one split fewer per unit-row of workgroups spreads the
// work more evenly -- 24 units x 11 splits are 264 workgroups, eight CUs with two of them while the rest have one,
// where 24 x 10 leave sixteen CUs idle and everybody done 1.8 times sooner. Compared by the keys the busiest CU walks.
static int attn_pick_splits(int64_t units, int ctx, int shift) {
  const int s0 = attn_splits_for(attn_fill(units), ctx, shift);
  const int by_work = ((ctx - 1) >> shift) + 1;
  int s1 = static_cast<int>(256 / (units > 0 ? units : 1));
  s1 = s1 > by_work ? s1 : by_work;
  s1 = s1 > 1 ? s1 : 1;
  if (s1 >= s0) return s0;
  auto busiest = [&](int s) {
    const int64_t rounds = (units * s + 255) / 256;
    const int64_t keys = (((ctx + s - 1) / s) + 31) & ~31;
    return rounds * keys;
  };
  return busiest(s1) < busiest(s0) ? s1 : s0;
}

static AttnPlan attn_plan(int64_t batch, int n_kv_heads, int64_t n_kv_ctx, int window) {
  const int64_t ctx = (window > 0 && window < n_kv_ctx) ? window : n_kv_ctx;
  // eight or four KV heads per workgroup: whichever fills the machine with the longest splits (ties: the wider one)
  AttnPlan best{0, 0, 0, 0};
  int64_t best_keys = 0;
  for (int hpw = RW; hpw >= 4; hpw >>= 1) {
    if (n_kv_heads % hpw != 0) continue;
    const int64_t units = batch * (n_kv_heads / hpw);
    const int s = attn_pick_splits(units, static_cast<int>(ctx), kRowsKeysShift);
    const int64_t keys = ctx / s;
    // splits of 256-511 keys too, when there are not too many of them and the HEAD shape would need its second launch as well
    const bool head_splits_too = attn_splits_for(attn_fill(batch * n_kv_heads), static_cast<int>(ctx), kHeadKeysShift) > 1;
    const bool long_enough = keys >= 512 || (head_splits_too && ((keys >= 256 && s <= 28) || (keys >= 320 && s <= 32)));
    if (units * s >= 224 && long_enough && keys > best_keys) {
      best = {hpw, s, s, kRowsKeysShift};                 // (the kernels' own evaluation starts from the chosen count)
      best_keys = keys;
    }
  }
  if (best.heads_per_wg) return best;
  const int sh = attn_pick_splits(batch * n_kv_heads, static_cast<int>(ctx), kHeadKeysShift);
  return {0, sh, sh, kHeadKeysShift};
}

extern "C" int tllm_attention_decode_heads_per_workgroup(int64_t batch, int n_kv_heads, int64_t n_kv_ctx, int window) {
  return attn_plan(batch, n_kv_heads, n_kv_ctx, window).heads_per_wg;
}

extern "C" int tllm_attention_decode_splits(int64_t batch, int n_kv_heads, int64_t n_kv_ctx, int window) {
  return attn_plan(batch, n_kv_heads, n_kv_ctx, window).splits;
}

extern "C" int64_t tllm_attention_decode_workspace_bytes(int64_t batch, int n_q_heads, int n_kv_heads, int64_t n_kv_ctx, int window) {
  const int s = tllm_attention_decode_splits(batch, n_kv_heads, n_kv_ctx, window);
  return s > 1 ? static_cast<int64_t>(s) * batch * n_q_heads * PART * 4 : 0;
}

extern "C" int tllm_attention_decode_bf16(const void* q, const void* k, const void* v, const void* sinks, void* out, int64_t q_row_stride,
                                          int64_t out_row_stride, int64_t kv_batch_stride, int64_t kv_token_stride, int64_t batch,
                                          int64_t n_kv_ctx, int n_kv_heads, int group, int head_dim, float sm_scale, int window,
                                          const void* start_q, int start_q_is_i64, int64_t kv_len_hint, void* workspace,
                                          int64_t workspace_bytes, void* stream) {
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
  TLLM_REQUIRE(kv_len_hint >= 0, TLLM_E_ARG, "attention_decode: kv_len_hint %lld", (long long)kv_len_hint);
  const int64_t plan_ctx = (kv_len_hint > 0 && kv_len_hint < n_kv_ctx) ? kv_len_hint : n_kv_ctx;
  const AttnPlan plan = attn_plan(batch, n_kv_heads, plan_ctx, window);
  a.splits = plan.splits;
  a.fill = plan.fill;
  a.keys_shift = plan.keys_shift;
  const int64_t need = tllm_attention_decode_workspace_bytes(batch, n_kv_heads * group, n_kv_heads, plan_ctx, window);
  TLLM_REQUIRE(need == 0 || (workspace != nullptr && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 4 == 0), TLLM_E_ARG,
               "attention_decode: workspace of %lld bytes needed (tllm_attention_decode_workspace_bytes), got %lld", (long long)need,
               (long long)workspace_bytes);
  a.part = static_cast<float*>(workspace);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (plan.heads_per_wg)
    hipLaunchKernelGGL(attn_decode_kernel<true>, dim3((unsigned)(n_kv_heads / plan.heads_per_wg * a.splits), (unsigned)batch),
                       dim3(plan.heads_per_wg * 64), 0, st, a);
  else
    hipLaunchKernelGGL(attn_decode_kernel<false>, dim3((unsigned)(n_kv_heads * a.splits), (unsigned)batch), dim3(AW * 64), 0, st, a);
  int rc = check_launch("attention_decode");
  if (rc != TLLM_OK || a.splits == 1) return rc;
  hipLaunchKernelGGL(attn_decode_reduce_kernel, dim3((unsigned)(n_kv_heads * group), (unsigned)batch), dim3(64), 0, st, a, (int)batch);
  return check_launch("attention_decode(reduce)");
}
