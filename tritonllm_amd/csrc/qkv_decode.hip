// Decode-size fused QKV projection + bias + rotary: weight-streaming kernels.
//
// With a handful of activation rows the 29.5 MB weight is read once and nothing else matters: the
// kernels are HBM-bound. All of them use the matrix core with the weight rows on the M side and
// the activation rows on the N side -- the MFMA does the K reduction across lanes for free and
// leaves the VALU to the rotary epilogue -- and keep a rotation pair (row d and row d+32 of a
// head) inside one workgroup so the rotation needs no second pass. The kernels:
//   qkv_decode_r8_kernel   hidden == 2880 (gpt-oss), up to 8 rows, bf16 weight: qkv_decode_r8.hip, the fastest.
//   qkv_decode_r32_kernel  hidden == 2880, 9..32 rows per workgroup, bf16 weight, no fused norm: qkv_decode_r32.hip.
//   qkv_decode_cu_kernel   hidden == 2880, the other cases (fused norm beyond 8 rows, fp8 weight): one workgroup per CU, coalesced
//                          loads, LDS-transposed operands; see its comment.
//   qkv_decode_kernel      head_dim == 64, hidden % 32 == 0: operands loaded straight into MFMA
//                          layout (simple, ~1.8x slower: every lane is its own cache-line request).
//   qkv_generic_kernel     anything else: shuffle-reduced dot products.
#include "qkv_common.h"

namespace tllm {

// ------------------------------------------------------------------------------------------------
// validation shared with the prefill entry point
int qkv_validate(const char* who, const void* x, const void* W, const void* q, const void* k, const void* v, int64_t q_rs,
                 int64_t k_rs, int64_t v_rs, int64_t kv_slot_stride, int64_t rows, int64_t hidden, int n_q_heads, int n_kv_heads,
                 int head_dim, const TllmRope* rope, QkvArgs* a, RopeArgs* ra, YarnFreqs* fr) {
  TLLM_REQUIRE(rows >= 0 && hidden > 0 && hidden < (1 << 30), TLLM_E_ARG, "%s: rows %lld / hidden %lld invalid", who, (long long)rows,
               (long long)hidden);
  TLLM_REQUIRE(n_q_heads >= 0 && n_kv_heads >= 0 && n_q_heads + n_kv_heads > 0, TLLM_E_ARG, "%s: head counts %d/%d invalid", who,
               n_q_heads, n_kv_heads);
  TLLM_REQUIRE(head_dim > 0 && head_dim % 2 == 0, TLLM_E_SHAPE, "%s: head_dim %d must be even and positive", who, head_dim);
  TLLM_REQUIRE(x && W, TLLM_E_ARG, "%s: null x or W", who);
  TLLM_REQUIRE((q || n_q_heads == 0) && ((k && v) || n_kv_heads == 0), TLLM_E_ARG, "%s: null output pointer", who);
  TLLM_REQUIRE(q_rs >= (int64_t)n_q_heads * head_dim && k_rs >= (int64_t)n_kv_heads * head_dim &&
                   v_rs >= (int64_t)n_kv_heads * head_dim,
               TLLM_E_ARG, "%s: output row stride smaller than the row", who);
  TLLM_REQUIRE(kv_slot_stride >= 0, TLLM_E_ARG, "%s: kv_slot_stride negative", who);
  TLLM_REQUIRE(rows < (1ll << 31), TLLM_E_SHAPE, "%s: rows %lld too large", who, (long long)rows);
  *ra = RopeArgs{};
  *fr = YarnFreqs{};
  if (rope) {
    int rc = make_rope_args(rope, head_dim, ra, fr);
    if (rc != TLLM_OK) return rc;
  }
  a->x = (const bf16*)x;
  a->W = (const bf16*)W;
  a->q = (bf16*)q;
  a->k = (bf16*)k;
  a->v = (bf16*)v;
  a->q_rs = q_rs;
  a->k_rs = k_rs;
  a->v_rs = v_rs;
  a->kv_slot_stride = kv_slot_stride;
  a->rows = rows;
  a->hidden = (int)hidden;
  a->n_q_heads = n_q_heads;
  a->n_kv_heads = n_kv_heads;
  a->head_dim = head_dim;
  a->has_rope = rope != nullptr;
  a->norm_scale = nullptr;
  a->norm_eps = 0.f;
  a->w_scale = nullptr;
  a->emb_ids = nullptr;
  a->emb_ids_i64 = 0;
  a->emb_table = nullptr;
  a->emb_vocab = 0;
  a->emb_out = nullptr;
  a->emb_oob = nullptr;
  return TLLM_OK;
}

// ------------------------------------------------------------------------------------------------
// shape-generic fallback
__global__ __launch_bounds__(256) void qkv_generic_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr) {
  const int head = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = a.head_dim >> 1;
  for (int64_t row = blockIdx.y; row < a.rows; row += gridDim.y) {
  const bf16* xr = a.x + row * a.hidden;
  bf16* out = qkv_out_ptr(a, qkv_slot(a, ra), row, head);
  const bool rotate = a.has_rope && head < a.n_q_heads + a.n_kv_heads;
  const int64_t pos = rotate ? rope_position(ra, row) : 0;
  for (int d = wave; d < half; d += 4) {
    const int64_t c_lo = static_cast<int64_t>(head) * a.head_dim + d, c_hi = c_lo + half;
    const bf16* w_lo = a.W + c_lo * a.hidden;
    const bf16* w_hi = a.W + c_hi * a.hidden;
    float lo = 0.f, hi = 0.f;
    for (int kk = lane; kk < a.hidden; kk += 64) {
      const float xv = static_cast<float>(xr[kk]);
      lo = fmaf(static_cast<float>(w_lo[kk]), xv, lo);
      hi = fmaf(static_cast<float>(w_hi[kk]), xv, hi);
    }
    lo = wave_sum(lo);
    hi = wave_sum(hi);
    if (lane == 0) {
      if (a.bias) {
        lo += static_cast<float>(a.bias[c_lo]);
        hi += static_cast<float>(a.bias[c_hi]);
      }
      if (rotate) {
        float c, s;
        rope_cos_sin(ra, fr, pos, d, &c, &s);
        const float rl = lo * c - hi * s, rh = hi * c + lo * s;
        lo = rl;
        hi = rh;
      }
      out[d] = static_cast<bf16>(lo);
      out[d + half] = static_cast<bf16>(hi);
    }
  }
  }
}

void launch_qkv_generic(const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr, hipStream_t st) {
  const int heads = a.n_q_heads + 2 * a.n_kv_heads;
  const unsigned gy = static_cast<unsigned>(a.rows < 65535 ? a.rows : 65535);   // rows beyond grid.y are looped in-kernel
  hipLaunchKernelGGL(qkv_generic_kernel, dim3((unsigned)heads, gy), dim3(256), 0, st, a, ra, fr);
}

// ------------------------------------------------------------------------------------------------
// MFMA kernel for any hidden % 32 == 0 (head_dim 64). A workgroup owns 16 weight rows of one head --
// dims [8p, 8p+8) and their partners [32+8p, 32+8p+8) -- and up to 16 activation rows; its wavefronts
// split K in runs of SPW k32-steps whose loads are all issued before the first multiply.
// v_mfma_f32_16x16x32_bf16: tile row 4*qd + i is dim 8p + 2*qd + (i & 1), plus 32 when i >= 2, so
// each lane's four accumulators are two complete (lo, hi) pairs.
template <int NW, int SPW>
__global__ __launch_bounds__(NW * 64) void qkv_decode_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr) {
  __shared__ float red[NW][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int head = blockIdx.x >> 2, piece = blockIdx.x & 3;
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * 16;
  const int kvec = a.hidden >> 3;       // 16-byte vectors per row
  const int nsteps = a.hidden >> 5;     // MFMA k-steps of 32
  const int m = lane & 15, g = lane >> 4;

  const int dim_a = 8 * piece + 2 * (m >> 2) + (m & 1) + ((m & 2) ? 32 : 0);
  const bf16x8* wrow = reinterpret_cast<const bf16x8*>(a.W) + (static_cast<int64_t>(head) * 64 + dim_a) * kvec + g;
  // Lanes past the last activation row re-read a live lane's row (same addresses, no extra traffic);
  // their output column is dropped.
  const int64_t xrow_idx = row0 + m;
  const bool xvalid = xrow_idx < a.rows;
  const int nvalid = static_cast<int>(a.rows - row0 < 16 ? a.rows - row0 : 16);
  const bf16x8* xrow = reinterpret_cast<const bf16x8*>(a.x) + (row0 + (xvalid ? m : m % nvalid)) * kvec + g;
  const bool rotate = a.has_rope && head < a.n_q_heads + a.n_kv_heads;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = wave * SPW; s0 < nsteps; s0 += NW * SPW) {
    bf16x8 wa[SPW], xb[SPW];
#pragma unroll
    for (int i = 0; i < SPW; ++i) {       // clamped, never predicated: a tail step re-reads the last one and is masked below
      const int step = s0 + i < nsteps ? s0 + i : nsteps - 1;
      wa[i] = __builtin_nontemporal_load(wrow + step * 4);
      xb[i] = xrow[step * 4];
    }
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      if (s0 + i < nsteps) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[i], xb[i], acc, 0, 0, 0);
    }
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave][i][lane] = acc[i];
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int w = 1; w < NW; ++w) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] += red[w][i][lane];
  }
  if (!xvalid) return;

  // the lane holds activation row xrow_idx and dims d0, d0 + 1 (acc[0], acc[1]) with their partners (acc[2], acc[3])
  const int d0 = 8 * piece + 2 * g;
  const int col = head * 64 + d0;
  float lo0 = acc[0], lo1 = acc[1], hi0 = acc[2], hi1 = acc[3];
  if (a.bias) {
    lo0 += static_cast<float>(a.bias[col]);
    lo1 += static_cast<float>(a.bias[col + 1]);
    hi0 += static_cast<float>(a.bias[col + 32]);
    hi1 += static_cast<float>(a.bias[col + 33]);
  }
  if (rotate) {
    const int64_t pos = rope_position(ra, xrow_idx);
    float c0, s0, c1, s1;
    rope_cos_sin(ra, fr, pos, d0, &c0, &s0);
    rope_cos_sin(ra, fr, pos, d0 + 1, &c1, &s1);
    const float r0 = lo0 * c0 - hi0 * s0, r1 = lo1 * c1 - hi1 * s1;
    const float r2 = hi0 * c0 + lo0 * s0, r3 = hi1 * c1 + lo1 * s1;
    lo0 = r0;
    lo1 = r1;
    hi0 = r2;
    hi1 = r3;
  }
  bf16* out = qkv_out_ptr(a, qkv_slot(a, ra), xrow_idx, head);
  bf16x2 plo, phi;
  plo[0] = static_cast<bf16>(lo0);
  plo[1] = static_cast<bf16>(lo1);
  phi[0] = static_cast<bf16>(hi0);
  phi[1] = static_cast<bf16>(hi1);
  *reinterpret_cast<bf16x2*>(out + d0) = plo;
  *reinterpret_cast<bf16x2*>(out + d0 + 32) = phi;
}

// ------------------------------------------------------------------------------------------------
// One-workgroup-per-CU variant for hidden == 2880 (the default decode kernel).
//
// The 2560 rotation pairs are dealt out ten at a time: 256 workgroups, each needing most of a CU's
// LDS, so the dispatcher has to place exactly one per CU and every CU streams exactly 1/256 of the
// weight (20 rows x 5760 B). Fifteen wavefronts split K (six k32-steps each); all loads of the
// kernel -- the small ones the epilogue needs first, then activations, then weights -- are issued
// unconditionally (indices clamped, never predicated) before anything is consumed, so the compiler
// has no join to wait at and ~180 KB per CU is in flight from the first microsecond.
// Loads are coalesced along K; the MFMA operand layout is produced by a pass through a
// wavefront-private LDS patch. v_mfma_f32_32x32x16_bf16: M = 32 tile rows (pair slot p at row p, its
// partner at row p + 16), N = up to XR activation rows. After one barrier the fifteen partial tiles
// are summed by 16 x XR threads, one (pair, activation row) each, which also add the bias, rotate
// with cos/sin they computed while the loads were in flight, round once and store.
// NORM: 0 = x is used as it is; 1 / 2 = x is first RMS-normalised with an fp32 / bf16 scale (fused prologue).
// W8: the weight is fp8 (OCP e4m3) with one fp32 scale per output row, W[n][k] = fp8[n][k] * w_scale[n]
// (triton_kernels.py:261-268, 927-940, 963-965). Half the bytes to stream; the values are widened to bf16 (exact)
// on their way into the LDS patch, so the MFMAs and the fp32 accumulation are those of the bf16 kernel, and the
// row scale multiplies the finished sum.
// EMB: the activation rows are gathered from an embedding table by token id (the first layer of a decode step:
// model.py:906-920 feeds the gather straight into the first block's norm + QKV); the workgroup with blockIdx.x == 0
// also writes the gathered rows out, as the residual stream. An id outside the table gives a zero row (its loads are
// clamped to a real row and the values discarded) and raises the flag, as the stand-alone gather does.
template <int XR, int CH, int NORM, bool W8, bool EMB = false>
__global__ __launch_bounds__(960) void qkv_decode_cu_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr) {
  static_assert(!EMB || NORM != 0, "the fused gather exists with the fused norm only");
  constexpr int NW = 15, SPW = 6, NCH = SPW / CH, PAIRS = 10;
  constexpr int KV = 360;                 // 16-byte vectors per activation row (hidden 2880)
  constexpr int KVW = W8 ? 180 : 360;     // ... per weight row
  constexpr int WROW = CH * 64 + 16;      // padded patch row, bytes
  constexpr int CPR = CH * 4;             // 16-byte chunks per row per patch (bf16)
  constexpr int CPRW = W8 ? CPR / 2 : CPR;            // ... of the weight as it lies in memory
  constexpr int WL = (2 * PAIRS * CPRW + 63) / 64;    // weight load instructions per patch
  constexpr int XL = (XR * CPR + 63) / 64;          // activation load instructions per patch
  constexpr int PATCH = (32 + XR) * WROW;
  constexpr int RED = XR * 32;            // floats per wavefront in the reduction buffer
  static_assert(SPW % CH == 0, "patches must tile the K slice");
  static_assert(NW * RED * 4 <= NW * PATCH, "reduction buffer aliases the patches");
  static_assert(16 * XR <= 960, "one epilogue thread per (pair slot, activation row)");
  __shared__ __align__(16) unsigned char lds[NW * PATCH];
  __shared__ float s_pin[16];
  __shared__ float s_part[NORM ? NW * XR : 1], s_rinv[NORM ? XR : 1];
  static_assert((NCH * XR * CPR + SPW * 32) * 4 <= PATCH, "sum-of-squares and scale scratch alias the wavefront's patch");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int total_pairs = (a.n_q_heads + 2 * a.n_kv_heads) * 32;
  const int pair0 = blockIdx.x * PAIRS;
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * XR;
  const int nvalid = static_cast<int>(a.rows - row0 < XR ? a.rows - row0 : XR);

  // ---- epilogue role of this thread: pair slot es, activation row en (clamped to real ones for the loads)
  const int es = tid & 15, en = tid >> 4;
  const bool evalid = tid < 16 * XR && es < PAIRS && pair0 + es < total_pairs && en < nvalid;
  const int egp = evalid ? pair0 + es : 0;
  const int ehead = egp >> 5, ed = egp & 31;
  const int64_t erow = row0 + (evalid ? en : 0);
  const bool erot = a.has_rope && ehead < a.n_q_heads + a.n_kv_heads;

  // ---- every global load of the kernel, oldest first
  const int64_t* pos_ptr = ra.positions ? ra.positions + erow : reinterpret_cast<const int64_t*>(a.W);
  const int64_t* off_ptr = ra.offset ? ra.offset : reinterpret_cast<const int64_t*>(a.W);
  const unsigned short* bias_ptr = reinterpret_cast<const unsigned short*>(a.bias ? a.bias : a.W);
  const int64_t pos_ld = *pos_ptr;
  const int64_t off_ld = *off_ptr;
  // The 32-row variant with the fused norm has no register left to hold the two bias values through the kernel
  // (the compiler would spill them at the very top, behind a full wait for the first loads): it fetches them
  // after the MFMAs instead, where the two reduction barriers cover the latency.
  constexpr bool LATE_BIAS = NORM != 0 && XR == 32;
  unsigned short b_lo = 0, b_hi = 0;
  if constexpr (!LATE_BIAS) {
    b_lo = bias_ptr[ehead * 64 + ed];
    b_hi = bias_ptr[ehead * 64 + 32 + ed];
  }
  const float freq = fr.v[ed];
  float ws_lo = 1.f, ws_hi = 1.f;
  if constexpr (W8) {
    ws_lo = a.w_scale[ehead * 64 + ed];
    ws_hi = a.w_scale[ehead * 64 + 32 + ed];
  }
  __builtin_amdgcn_sched_barrier(0);

  const bf16x8* xg = reinterpret_cast<const bf16x8*>(a.x) + row0 * KV + wave * (SPW * 4);
  const bf16x8* wg = reinterpret_cast<const bf16x8*>(a.W) + wave * (W8 ? SPW * 2 : SPW * 4);   // 16-byte units either way
  bf16x8 xr[NCH * XL], wr[NCH * WL];
  // The norm scale of this wavefront's K slice (SPW * 32 values): one load per wavefront, parked in LDS later.
  f32x4 sc32 = {};
  bf16x8 sc16 = {};
  if constexpr (NORM == 1) sc32 = reinterpret_cast<const f32x4*>(a.norm_scale)[wave * (SPW * 8) + (lane < SPW * 8 ? lane : SPW * 8 - 1)];
  if constexpr (NORM == 2) sc16 = reinterpret_cast<const bf16x8*>(a.norm_scale)[wave * (SPW * 4) + (lane < SPW * 4 ? lane : SPW * 4 - 1)];
  // EMB: where each of this lane's activation rows starts in the table (one id per load slot, fetched first)
  const bf16x8* xsrc[XL];
  bool xok[XL];
  if constexpr (EMB) {
    int64_t id[XL];
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      int e = i * 64 + lane;
      e = e < XR * CPR ? e : XR * CPR - 1;
      int r = e / CPR;
      r = r < nvalid ? r : nvalid - 1;
      id[i] = a.emb_ids_i64 ? reinterpret_cast<const int64_t*>(a.emb_ids)[row0 + r]
                            : static_cast<int64_t>(reinterpret_cast<const int*>(a.emb_ids)[row0 + r]);
    }
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      const bool ok = id[i] >= 0 && id[i] < a.emb_vocab;
      xok[i] = ok;
      if (!ok && a.emb_oob) *a.emb_oob = 1;
      const int64_t idc = id[i] < 0 ? 0 : (id[i] < a.emb_vocab ? id[i] : a.emb_vocab - 1);
      xsrc[i] = reinterpret_cast<const bf16x8*>(a.emb_table) + idc * KV + wave * (SPW * 4);
    }
  }
  auto load_x = [&]() {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
#pragma unroll
      for (int i = 0; i < XL; ++i) {          // patch chunk e -> activation row e / CPR, chunk e % CPR
        int e = i * 64 + lane;
        e = e < XR * CPR ? e : XR * CPR - 1;
        int r = e / CPR;
        const int kc = e - r * CPR;
        r = r < nvalid ? r : nvalid - 1;
        if constexpr (EMB) xr[j * XL + i] = xsrc[i][j * CPR + kc];
        else xr[j * XL + i] = xg[r * KV + j * CPR + kc];
      }
    }
  };
  // Order of the requests. All 256 workgroups read the same few activation rows, which the L2s can only hand
  // out at their own pace (32 CUs per L2 asking for the same lines), while the weight stream has the whole
  // HBM latency ahead of it: without the norm the weight requests go first and the activations follow in
  // their shadow. With the fused norm the activations are needed first (see below).
  if constexpr (NORM != 0) load_x();
  auto load_w = [&](int idx) {               // weight load idx: patch j = idx / WL, chunk slot i = idx % WL
    const int j = idx / WL, i = idx % WL;
    int e = i * 64 + lane;                    // patch chunk e -> weight row e / CPRW: the ten low rows, then their partners
    e = e < 2 * PAIRS * CPRW ? e : 2 * PAIRS * CPRW - 1;
    const int r = e / CPRW, kc = e - r * CPRW;
    int gp = pair0 + (r < PAIRS ? r : r - PAIRS);
    gp = gp < total_pairs ? gp : total_pairs - 1;
    const unsigned wrow = static_cast<unsigned>(gp >> 5) * 64u + (gp & 31) + (r < PAIRS ? 0u : 32u);
    wr[idx] = __builtin_nontemporal_load(wg + wrow * static_cast<unsigned>(KVW) + j * CPRW + kc);
  };
  // A CU holds a bounded number of loads in flight and a wavefront stalls when it issues one beyond that. With
  // the fused norm every wavefront must see its activations, and meet the others at a barrier, before any MFMA
  // can start; a wavefront stuck issuing weight loads would get there only when the stream has almost drained.
  // So only the first NEARLY weight loads are requested up front (enough to keep the memory pipe busy during
  // the norm), behind a rendezvous that puts every wavefront's activation loads ahead of them in the queue;
  // the rest follow right after the norm's barriers.
  constexpr int NEARLY = NORM == 0 ? NCH * WL : (XR == 32 ? 0 : 2);   // XR == 32 has no registers to spare for any
  if constexpr (NORM != 0) __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int idx = 0; idx < NEARLY; ++idx) load_w(idx);
  if constexpr (NORM == 0) load_x();
  __builtin_amdgcn_sched_barrier(0);

  // ---- cos/sin of this thread's (pair, row) while the weights are in flight.
  // The store pins the frequency load above the weight stream: with its only use inside the
  // conditional below, the compiler would sink it there and then have to drain every load to read it.
  s_pin[es] = freq;
  float cs = 1.f, sn = 0.f;
  const int64_t slot = (a.kv_slot_stride != 0 && ra.offset != nullptr) ? off_ld : 0;
  // Only the first 16 * XR threads have an epilogue role; the test is uniform per wavefront, and the other
  // wavefronts must skip this: the 64-bit position arithmetic and the sincos are some six hundred vector
  // instructions, and fifteen wavefronts doing them on four SIMDs would take as long as the whole weight stream.
  if (a.has_rope && tid < 16 * XR) {
    int64_t pos = ra.positions ? pos_ld : (erow % ra.tokens_per_batch) + (ra.offset ? off_ld : 0);
    pos = rope_wrap(pos, ra.max_ctx);
    if (ra.use_yarn) yarn_cos_sin(pos, freq, ra.concentration, &cs, &sn);
    else rope_cos_sin(ra, fr, pos, ed, &cs, &sn);
  }

  __builtin_amdgcn_sched_barrier(0);

  // ---- fused RMSNorm prologue: turn the raw activation chunks held in registers into
  // bf16(x * rsqrt(mean(x^2) + eps) * scale), the exact operand the two-launch form passes between its kernels.
  // Sum of squares: per-chunk partials -> the wavefront's LDS patch (idle so far) -> one lane per row adds its
  // row's chunks -> the fifteen K slices meet in s_part -> s_rinv.
  if constexpr (NORM != 0) {
    float* tmp = reinterpret_cast<float*>(lds + wave * PATCH);
    float* wscale = tmp + NCH * XR * CPR;
    if constexpr (EMB) {                      // an id outside the table stands for a zero row (the load itself read a real one)
#pragma unroll
      for (int c = 0; c < NCH * XL; ++c) {
        if (!xok[c % XL]) {
#pragma unroll
          for (int q = 0; q < 8; ++q) xr[c][q] = static_cast<bf16>(0.f);
        }
      }
    }
    if constexpr (NORM == 1) {
      if (lane < SPW * 8) reinterpret_cast<f32x4*>(wscale)[lane] = sc32;
    } else {
      if (lane < SPW * 4) {
        f32x4 lo4, hi4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          lo4[q] = static_cast<float>(sc16[q]);
          hi4[q] = static_cast<float>(sc16[4 + q]);
        }
        reinterpret_cast<f32x4*>(wscale)[2 * lane] = lo4;
        reinterpret_cast<f32x4*>(wscale)[2 * lane + 1] = hi4;
      }
    }
#pragma unroll
    for (int c = 0; c < NCH * XL; ++c) {
      const int e = (c % XL) * 64 + lane;
      float ssq = 0.f;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float f = static_cast<float>(xr[c][q]);
        ssq = fmaf(f, f, ssq);
      }
      if (e < XR * CPR) tmp[(c / XL) * (XR * CPR) + e] = ssq;
    }
    if constexpr (EMB) {
      if (blockIdx.x == 0) {                  // one workgroup per row chunk leaves the gathered rows behind
        bf16x8* xo = reinterpret_cast<bf16x8*>(a.emb_out) + row0 * KV + wave * (SPW * 4);
#pragma unroll
        for (int c = 0; c < NCH * XL; ++c) {
          const int e = (c % XL) * 64 + lane;
          const int r = e / CPR, kc = e - r * CPR;
          if (e < XR * CPR && r < nvalid) xo[r * KV + (c / XL) * CPR + kc] = xr[c];
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (lane < XR) {
      float p = 0.f;
#pragma unroll
      for (int j = 0; j < NCH; ++j) {
#pragma unroll
        for (int c = 0; c < CPR / 4; ++c) {
          const f32x4 t4 = *reinterpret_cast<const f32x4*>(tmp + j * (XR * CPR) + lane * CPR + 4 * c);
          p += (t4[0] + t4[1]) + (t4[2] + t4[3]);
        }
      }
      s_part[wave * XR + lane] = p;
    }
    __syncthreads();
    if (tid < XR) {
      float ss = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) ss += s_part[w * XR + tid];
      s_rinv[tid] = rsqrtf(ss * (1.0f / 2880.0f) + a.norm_eps);
    }
    __syncthreads();
#pragma unroll
    for (int idx = NEARLY; idx < NCH * WL; ++idx) load_w(idx);
    __builtin_amdgcn_sched_barrier(0);
    // Chunk c's scale values and 1/rms are fetched from LDS while chunk c-1 is being scaled, and each chunk is
    // fenced off from the next: written plainly, the compiler either serialises every LDS latency or sinks the
    // arithmetic down to the patch writes and keeps every chunk's scale values alive until then, next to all the
    // weight loads' destination registers (it then spills those, with a full drain of the load queue each).
    typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;
    constexpr int NC = NCH * XL;
    f32x4 s_lo, s_hi, n_lo = {}, n_hi = {};
    float rinv, n_rinv = 0.f;
    auto fetch = [&](int c, f32x4& lo4, f32x4& hi4, float& ri) {
      int e = (c % XL) * 64 + lane;
      e = e < XR * CPR ? e : XR * CPR - 1;
      const f32x4* sp = reinterpret_cast<const f32x4*>(wscale) + 2 * ((c / XL) * CPR + e % CPR);
      lo4 = sp[0];
      hi4 = sp[1];
      ri = s_rinv[e / CPR];
    };
    fetch(0, s_lo, s_hi, rinv);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      if (c + 1 < NC) fetch(c + 1, n_lo, n_hi, n_rinv);
      __builtin_amdgcn_sched_barrier(0);
      u32x4 bits = __builtin_bit_cast(u32x4, xr[c]);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        asm volatile("" : "+v"(bits[q]));       // the fp32 copies of the sum-of-squares pass must not stay alive
        bf16x2 t;
        t[0] = static_cast<bf16>(__uint_as_float(bits[q] << 16) * rinv * (q < 2 ? s_lo[2 * q] : s_hi[2 * q - 4]));
        t[1] = static_cast<bf16>(__uint_as_float(bits[q] & 0xffff0000u) * rinv * (q < 2 ? s_lo[2 * q + 1] : s_hi[2 * q - 3]));
        bits[q] = __builtin_bit_cast(unsigned, t);
        asm volatile("" : "+v"(bits[q]));       // ... and the arithmetic must not sink to the patch write below
      }
      xr[c] = __builtin_bit_cast(bf16x8, bits);
      __builtin_amdgcn_sched_barrier(0);
      s_lo = n_lo;
      s_hi = n_hi;
      rinv = n_rinv;
    }
  }

  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  const int m = lane & 31, h = lane >> 5;
  unsigned char* wp = lds + wave * PATCH;            // 32 tile rows (only those of real pairs are written)
  unsigned char* xp = wp + 32 * WROW;                // XR activation rows
  const unsigned char* wfrag = wp + m * WROW + h * 16;
  const unsigned char* xfrag = xp + (m & (XR - 1)) * WROW + h * 16;   // stale LDS in unused rows/columns is never stored
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      const int e = i * 64 + lane;
      const int r = e / CPR, kc = e - r * CPR;
      if (e < XR * CPR && r < nvalid) *reinterpret_cast<bf16x8*>(xp + r * WROW + kc * 16) = xr[j * XL + i];
    }
#pragma unroll
    for (int i = 0; i < WL; ++i) {
      const int e = i * 64 + lane;
      const int r = e / CPRW, kc = e - r * CPRW;
      const int trow = r < PAIRS ? r : r - PAIRS + 16;
      if constexpr (W8) {
        // sixteen fp8 -> sixteen bf16 (exact: e4m3 fits), two chunks of the patch row
        typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4;
        typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
        const i32x4 raw = __builtin_bit_cast(i32x4, wr[j * WL + i]);
        bf16x8 w0, w1;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const f32x2 p0 = __builtin_amdgcn_cvt_pk_f32_fp8(raw[d], false), p1 = __builtin_amdgcn_cvt_pk_f32_fp8(raw[d], true);
          bf16x8& dst = d < 2 ? w0 : w1;
          dst[4 * (d & 1) + 0] = static_cast<bf16>(p0[0]);
          dst[4 * (d & 1) + 1] = static_cast<bf16>(p0[1]);
          dst[4 * (d & 1) + 2] = static_cast<bf16>(p1[0]);
          dst[4 * (d & 1) + 3] = static_cast<bf16>(p1[1]);
        }
        if (e < 2 * PAIRS * CPRW) {
          *reinterpret_cast<bf16x8*>(wp + trow * WROW + kc * 32) = w0;
          *reinterpret_cast<bf16x8*>(wp + trow * WROW + kc * 32 + 16) = w1;
        }
      } else {
        if (e < 2 * PAIRS * CPRW) *reinterpret_cast<bf16x8*>(wp + trow * WROW + kc * 16) = wr[j * WL + i];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < 2 * CH; ++t) {
      const bf16x8 fa = *reinterpret_cast<const bf16x8*>(wfrag + t * 32);
      const bf16x8 fb = *reinterpret_cast<const bf16x8*>(xfrag + t * 32);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  if constexpr (LATE_BIAS) {
    b_lo = bias_ptr[ehead * 64 + ed];
    b_hi = bias_ptr[ehead * 64 + 32 + ed];
  }
  // ---- fifteen partial tiles -> LDS as [wave][tile row][activation row] (lanes of one store hit distinct banks)
  __syncthreads();
  float* red = reinterpret_cast<float*>(lds);
  if (m < XR) {
#pragma unroll
    for (int v = 0; v < 16; ++v) red[wave * RED + (8 * (v >> 2) + 4 * h + (v & 3)) * XR + m] = acc[v];
  }
  __syncthreads();
  if (!evalid) return;
  float lo = 0.f, hi = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    lo += red[w * RED + es * XR + en];
    hi += red[w * RED + (16 + es) * XR + en];
  }
  if constexpr (W8) {
    lo *= ws_lo;
    hi *= ws_hi;
  }
  if (a.bias) {
    lo += __uint_as_float(static_cast<unsigned>(b_lo) << 16);
    hi += __uint_as_float(static_cast<unsigned>(b_hi) << 16);
  }
  if (erot) {
    const float rl = lo * cs - hi * sn, rh = hi * cs + lo * sn;
    lo = rl;
    hi = rh;
  }
  bf16* out = qkv_out_ptr(a, slot, erow, ehead);
  out[ed] = static_cast<bf16>(lo);
  out[ed + 32] = static_cast<bf16>(hi);
}

}  // namespace tllm

using namespace tllm;

// The kernel above serves what the two streaming kernels do not: the fused norm (and gather) at 9..16 rows.
static void launch_cu_embed(int norm, bool w8, dim3 grid, hipStream_t st, const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr) {
#define TLLM_CUE(NORM)                                                                                              \
  do {                                                                                                              \
    if (w8) hipLaunchKernelGGL((qkv_decode_cu_kernel<16, 3, NORM, true, true>), grid, dim3(960), 0, st, a, ra, fr);  \
    else hipLaunchKernelGGL((qkv_decode_cu_kernel<16, 3, NORM, false, true>), grid, dim3(960), 0, st, a, ra, fr);    \
  } while (0)
  if (norm == 1) TLLM_CUE(1);
  else TLLM_CUE(2);
#undef TLLM_CUE
}

static void launch_cu(int xr, int norm, bool w8, dim3 grid, hipStream_t st, const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr) {
#define TLLM_CU(XR, CH, NORM)                                                                                   \
  do {                                                                                                          \
    if (w8) hipLaunchKernelGGL((qkv_decode_cu_kernel<XR, CH, NORM, true>), grid, dim3(960), 0, st, a, ra, fr);  \
    else hipLaunchKernelGGL((qkv_decode_cu_kernel<XR, CH, NORM, false>), grid, dim3(960), 0, st, a, ra, fr);    \
  } while (0)
  (void)xr;                                                               // 16: the only height left
  if (norm == 1) TLLM_CU(16, 3, 1);
  else TLLM_CU(16, 3, 2);
#undef TLLM_CU
}

// Shared tail of the hidden-2880 decode entry points: row-count -> kernel variant and grid.
static int launch_decode_2880(const char* what, QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr, int norm, bool w8, int64_t rows,
                              int heads, hipStream_t st) {
  TLLM_REQUIRE(static_cast<int64_t>(heads) * 64 * 2880 < (1ll << 31), TLLM_E_SHAPE, "%s: weight too large", what);
  const bool emb = a.emb_ids != nullptr;
  // the fused gather addresses table rows with 32-bit byte offsets
  TLLM_REQUIRE(!emb || a.emb_vocab * 5760 < (1ll << 32), TLLM_E_SHAPE, "%s: embedding table of %lld rows too large for the fused gather", what,
               (long long)a.emb_vocab);
  const bool r32 = rows > 8 && norm == 0 && !emb;                          // 9..32 rows per workgroup, normalised activations
  const int xr = rows <= 8 ? 8 : ((rows <= 16 && !r32) ? 16 : 32);
  const int64_t chunks = (rows + xr - 1) / xr;
  TLLM_REQUIRE(chunks <= 65535, TLLM_E_SHAPE, "%s: rows %lld too many for the decode kernel", what, (long long)rows);
  const dim3 grid((unsigned)((heads * 32 + 9) / 10), (unsigned)chunks);
  if (r32) launch_qkv_decode_r32(w8, grid, st, a, ra, fr);
  else if (xr == 8) launch_qkv_decode_r8(norm, emb, w8, grid, st, a, ra, fr);
  else if (emb) launch_cu_embed(norm, w8, grid, st, a, ra, fr);
  else launch_cu(xr, norm, w8, grid, st, a, ra, fr);
  return check_launch(what);
}

struct EmbedSrc {
  const void* ids;
  int ids_i64;
  const void* table;
  int64_t vocab;
  int32_t* oob_flag;
};

// Common body of the entry points that exist for the gpt-oss shape only (fused gather, fused norm and/or fp8 weight).
static int decode_2880_entry(const char* what, const void* x, const void* norm_scale, int scale_is_bf16, float eps, const void* W,
                             const float* w_scale, bool w8, const void* b, void* q, void* k, void* v, int64_t q_row_stride,
                             int64_t k_row_stride, int64_t v_row_stride, int64_t kv_slot_stride, int64_t rows, int64_t hidden,
                             int n_q_heads, int n_kv_heads, int head_dim, const TllmRope* rope, void* stream,
                             const EmbedSrc* emb = nullptr) {
  QkvArgs a;
  RopeArgs ra;
  YarnFreqs fr;
  int rc = qkv_validate(what, x, W, q, k, v, q_row_stride, k_row_stride, v_row_stride, kv_slot_stride, rows, hidden, n_q_heads,
                        n_kv_heads, head_dim, rope, &a, &ra, &fr);
  if (rc != TLLM_OK) return rc;
  if (emb) {
    TLLM_REQUIRE(emb->ids && emb->table && emb->vocab > 0, TLLM_E_ARG, "%s: ids, table must not be NULL and vocab positive", what);
    TLLM_REQUIRE(norm_scale != nullptr, TLLM_E_ARG, "%s: the fused gather needs the fused norm (norm_scale is NULL)", what);
    TLLM_REQUIRE(rows <= 16, TLLM_E_SHAPE, "%s: at most 16 rows (got %lld): gather, then call the QKV entry point", what, (long long)rows);
    TLLM_REQUIRE(aligned16(emb->table) && reinterpret_cast<uintptr_t>(emb->ids) % (emb->ids_i64 ? 8 : 4) == 0, TLLM_E_ALIGN,
                 "%s: table must be 16-byte aligned and ids aligned to their size", what);
    a.emb_ids = emb->ids;
    a.emb_ids_i64 = emb->ids_i64;
    a.emb_table = static_cast<const bf16*>(emb->table);
    a.emb_vocab = emb->vocab;
    a.emb_out = const_cast<bf16*>(a.x);
    a.emb_oob = emb->oob_flag;
  }
  TLLM_REQUIRE(hidden == 2880 && head_dim == 64, TLLM_E_SHAPE,
               "%s: this kernel exists for hidden 2880 / head_dim 64 only (got %lld / %d)", what, (long long)hidden, head_dim);
  TLLM_REQUIRE(aligned16(x) && aligned16(W) && aligned16(norm_scale), TLLM_E_ALIGN, "%s: x, W and norm_scale must be 16-byte aligned", what);
  TLLM_REQUIRE(!w8 || (w_scale != nullptr && reinterpret_cast<uintptr_t>(w_scale) % 4 == 0), TLLM_E_ARG,
               "%s: w_scale must be a 4-byte aligned device pointer", what);
  // 32 rows of raw activations do not fit next to the weight ring, and a row's factor is needed before its first
  // product: above 16 rows the norm is a launch of its own, which this library cannot insert (it owns no buffer).
  TLLM_REQUIRE(norm_scale == nullptr || rows <= 16, TLLM_E_SHAPE,
               "%s: the fused RMSNorm exists for up to 16 rows (got %lld): call tllm_rmsnorm_bf16, then the projection without norm_scale",
               what, (long long)rows);
  a.bias = (const bf16*)b;
  a.norm_scale = norm_scale;
  a.norm_eps = eps;
  a.w_scale = w_scale;
  if (rows == 0) return TLLM_OK;
  return launch_decode_2880(what, a, ra, fr, norm_scale ? (scale_is_bf16 ? 2 : 1) : 0, w8, rows, n_q_heads + 2 * n_kv_heads,
                            static_cast<hipStream_t>(stream));
}

extern "C" int tllm_norm_qkv_rope_decode_bf16(const void* x, const void* norm_scale, int scale_is_bf16, float eps, const void* W,
                                              const void* b, void* q, void* k, void* v, int64_t q_row_stride, int64_t k_row_stride,
                                              int64_t v_row_stride, int64_t kv_slot_stride, int64_t rows, int64_t hidden, int n_q_heads,
                                              int n_kv_heads, int head_dim, const TllmRope* rope, void* stream) {
  if (norm_scale == nullptr) {
    set_error("norm_qkv_rope_decode: norm_scale is NULL");
    return TLLM_E_ARG;
  }
  return decode_2880_entry("norm_qkv_rope_decode", x, norm_scale, scale_is_bf16, eps, W, nullptr, false, b, q, k, v, q_row_stride,
                           k_row_stride, v_row_stride, kv_slot_stride, rows, hidden, n_q_heads, n_kv_heads, head_dim, rope, stream);
}

extern "C" int tllm_embed_norm_qkv_rope_decode_bf16(const void* ids, int ids_is_i64, const void* table, int64_t vocab, void* x_out,
                                                    int32_t* oob_flag, const void* norm_scale, int scale_is_bf16, float eps, const void* W,
                                                    const float* w_scale, const void* b, void* q, void* k, void* v, int64_t q_row_stride,
                                                    int64_t k_row_stride, int64_t v_row_stride, int64_t kv_slot_stride, int64_t rows,
                                                    int64_t hidden, int n_q_heads, int n_kv_heads, int head_dim, const TllmRope* rope,
                                                    void* stream) {
  const EmbedSrc emb{ids, ids_is_i64, table, vocab, oob_flag};
  return decode_2880_entry("embed_norm_qkv_rope_decode", x_out, norm_scale, scale_is_bf16, eps, W, w_scale, w_scale != nullptr, b, q, k, v,
                           q_row_stride, k_row_stride, v_row_stride, kv_slot_stride, rows, hidden, n_q_heads, n_kv_heads, head_dim, rope,
                           stream, &emb);
}

extern "C" int tllm_qkv_rope_decode_w8_bf16(const void* x, const void* norm_scale, int scale_is_bf16, float eps, const void* W8,
                                            const float* w_scale, const void* b, void* q, void* k, void* v, int64_t q_row_stride,
                                            int64_t k_row_stride, int64_t v_row_stride, int64_t kv_slot_stride, int64_t rows,
                                            int64_t hidden, int n_q_heads, int n_kv_heads, int head_dim, const TllmRope* rope,
                                            void* stream) {
  return decode_2880_entry("qkv_rope_decode_w8", x, norm_scale, scale_is_bf16, eps, W8, w_scale, true, b, q, k, v, q_row_stride,
                           k_row_stride, v_row_stride, kv_slot_stride, rows, hidden, n_q_heads, n_kv_heads, head_dim, rope, stream);
}

extern "C" int tllm_qkv_rope_decode_bf16(const void* x, const void* W, const void* b, void* q, void* k, void* v, int64_t q_row_stride,
                                         int64_t k_row_stride, int64_t v_row_stride, int64_t kv_slot_stride, int64_t rows,
                                         int64_t hidden, int n_q_heads, int n_kv_heads, int head_dim, const TllmRope* rope,
                                         void* stream) {
  QkvArgs a;
  RopeArgs ra;
  YarnFreqs fr;
  int rc = qkv_validate("qkv_rope_decode", x, W, q, k, v, q_row_stride, k_row_stride, v_row_stride, kv_slot_stride, rows, hidden,
                        n_q_heads, n_kv_heads, head_dim, rope, &a, &ra, &fr);
  if (rc != TLLM_OK) return rc;
  a.bias = (const bf16*)b;
  if (rows == 0) return TLLM_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int heads = n_q_heads + 2 * n_kv_heads;
  const bool mfma_ok = head_dim == 64 && hidden % 32 == 0 && aligned16(x) && aligned16(W);
  if (mfma_ok && hidden == 2880 && aligned16(b) && static_cast<int64_t>(heads) * 64 * hidden < (1ll << 31)) {
    // 32-bit element offsets inside W and x are enough here; outputs are written element-wise, any alignment
    return launch_decode_2880("qkv_rope_decode", a, ra, fr, 0, false, rows, heads, st);
  }
  const bool out4 = (reinterpret_cast<uintptr_t>(q) % 4 == 0) && (reinterpret_cast<uintptr_t>(k) % 4 == 0) &&
                    (reinterpret_cast<uintptr_t>(v) % 4 == 0) && q_row_stride % 2 == 0 && k_row_stride % 2 == 0 &&
                    v_row_stride % 2 == 0 && kv_slot_stride % 2 == 0;
  if (mfma_ok && out4) {
    const int64_t chunks = (rows + 15) / 16;
    TLLM_REQUIRE(chunks <= 65535, TLLM_E_SHAPE, "qkv_rope_decode: rows %lld too many for the decode kernel", (long long)rows);
    hipLaunchKernelGGL((qkv_decode_kernel<4, 16>), dim3((unsigned)(heads * 4), (unsigned)chunks), dim3(4 * 64), 0, st, a, ra, fr);
    return check_launch("qkv_rope_decode");
  }
  launch_qkv_generic(a, ra, fr, st);
  return check_launch("qkv_rope_decode(generic)");
}
