// Decode-size fused QKV projection + bias + rotary: weight-streaming kernels.
//
// With a handful of activation rows the 29.5 MB weight is read once and nothing else matters: the
// kernels are HBM-bound. All of them use the matrix core with the weight rows on the M side and
// the activation rows on the N side -- the MFMA does the K reduction across lanes for free and
// leaves the VALU to the rotary epilogue -- and keep a rotation pair (row d and row d+32 of a
// head) inside one workgroup so the rotation needs no second pass. The kernels:
//   qkv_decode_r8_kernel   hidden == 2880 (gpt-oss), up to 8 rows per workgroup, or up to 16 with the fused RMSNorm; bf16 or
//                          fp8 weight, optional fused norm and token gather: qkv_decode_r8.hip, the fastest.
//   qkv_decode_r32_kernel  hidden == 2880, 9..32 rows per workgroup, bf16 or fp8 weight, no fused norm: qkv_decode_r32.hip.
//   qkv_decode_rows_kernel hidden == 2880, more than 32 rows: the weight read once and held, the rows streamed past it:
//                          qkv_decode_rows.hip.
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
// MFMA kernel for any hidden % 32 == 0 and head_dim % 16 == 0 (the reference's decode kernel is generic over both,
// triton_kernels.py:1127-1158). A workgroup owns 16 weight rows of one head -- dims [8p, 8p+8) and their partners
// [half+8p, half+8p+8), half = head_dim / 2 -- and up to 16 activation rows; its wavefronts
// split K in runs of SPW k32-steps whose loads are all issued before the first multiply.
// v_mfma_f32_16x16x32_bf16: tile row 4*qd + i is dim 8p + 2*qd + (i & 1), plus half when i >= 2, so
// each lane's four accumulators are two complete (lo, hi) pairs.
// W8: the weight is fp8 (OCP e4m3) with one fp32 scale per output row (the reference's fp8 branch is as generic as its
// bf16 one, triton_kernels.py:927-940): eight bytes per lane and step, widened to bf16 in registers (exact), the row
// scale applied to the finished sum.
// A run's 16 weight rows x SPW steps arrive row by row -- one load instruction = one row's contiguous run, 64 lanes x 16
// bytes (fp8: x 8) -- and pass a wavefront-private LDS patch on their way into A-operand layout (loaded straight into
// that layout every lane's bytes are a request of their own, and the memory side serves such a stream at three
// quarters of the rate).
template <int NW, int SPW, bool W8 = false>
__global__ __launch_bounds__(NW * 64) void qkv_decode_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr) {
  __shared__ float red[NW][4][64];
  constexpr int WROW = SPW * (W8 ? 32 : 64) + 16;           // patch row: a run's bytes of one weight row + padding (conflict-free fragment reads)
  extern __shared__ __align__(16) unsigned char wpatch_all[];   // [NW][16][WROW]
  static_assert(SPW == 16, "a load instruction covers one row's run of 16 steps");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = a.head_dim >> 1, pieces = half >> 3;
  const int head = blockIdx.x / pieces, piece = blockIdx.x - head * pieces;
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * 16;
  const int kvec = a.hidden >> 3;       // 16-byte vectors per row
  const int nsteps = a.hidden >> 5;     // MFMA k-steps of 32
  const int m = lane & 15, g = lane >> 4;

  typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2;
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
    u32x2 wa8[SPW];
#pragma unroll
    for (int i = 0; i < SPW; ++i) {       // clamped, never predicated: a tail step re-reads the last one and is masked below
      const int step = s0 + i < nsteps ? s0 + i : nsteps - 1;
      // load i = tile row i: lane l fetches chunk s0 * 4 + l of that row -- 16 bytes of a bf16 row, 8 of an fp8 row, either
      // way the lane's share of the run's 16 steps -- clamped at the row's end (a tail run re-reads the last chunk; those
      // steps are masked below)
      const int chunk = s0 * 4 + lane < kvec ? s0 * 4 + lane : kvec - 1;
      const int dim_i = 8 * piece + 2 * (i >> 2) + (i & 1) + ((i & 2) ? half : 0);
      const int64_t wrow_i = static_cast<int64_t>(head) * a.head_dim + dim_i;
      if constexpr (W8) {
        wa8[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(reinterpret_cast<const unsigned char*>(a.W) + wrow_i * a.hidden) + chunk);
      } else {
        wa[i] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(a.W) + wrow_i * kvec + chunk);
      }
      xb[i] = xrow[step * 4];
    }
    unsigned char* wp = wpatch_all + wave * (16 * WROW);
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      if constexpr (W8) *reinterpret_cast<u32x2*>(wp + i * WROW + lane * 8) = wa8[i];
      else *reinterpret_cast<bf16x8*>(wp + i * WROW + lane * 16) = wa[i];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      if constexpr (W8) wa8[i] = *reinterpret_cast<const u32x2*>(wp + m * WROW + (4 * i + g) * 8);
      else wa[i] = *reinterpret_cast<const bf16x8*>(wp + m * WROW + (4 * i + g) * 16);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the next run's writes come after these reads
    __builtin_amdgcn_wave_barrier();
    if constexpr (W8) {
#pragma unroll
      for (int i = 0; i < SPW; ++i) wa[i] = fp8x8_to_bf16x8(wa8[i][0], wa8[i][1]);
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
  const int col = head * a.head_dim + d0;
  float lo0 = acc[0], lo1 = acc[1], hi0 = acc[2], hi1 = acc[3];
  if constexpr (W8) {
    lo0 *= a.w_scale[col];
    lo1 *= a.w_scale[col + 1];
    hi0 *= a.w_scale[col + half];
    hi1 *= a.w_scale[col + half + 1];
  }
  if (a.bias) {
    lo0 += static_cast<float>(a.bias[col]);
    lo1 += static_cast<float>(a.bias[col + 1]);
    hi0 += static_cast<float>(a.bias[col + half]);
    hi1 += static_cast<float>(a.bias[col + half + 1]);
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
  *reinterpret_cast<bf16x2*>(out + d0 + half) = phi;
}

}  // namespace tllm

using namespace tllm;

// Shared tail of the hidden-2880 decode entry points: row-count -> kernel variant and grid.
static int launch_decode_2880(const char* what, QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr, int norm, bool w8, int64_t rows,
                              int heads, hipStream_t st) {
  TLLM_REQUIRE(static_cast<int64_t>(heads) * 64 * 2880 < (1ll << 31), TLLM_E_SHAPE, "%s: weight too large", what);
  const bool emb = a.emb_ids != nullptr;
  // the fused gather addresses table rows with 32-bit byte offsets
  TLLM_REQUIRE(!emb || a.emb_vocab * 5760 < (1ll << 32), TLLM_E_SHAPE, "%s: embedding table of %lld rows too large for the fused gather", what,
               (long long)a.emb_vocab);
  // up to 8 rows: the 8-row streaming kernel; 9..16 rows with the fused norm (and gather): its 16-row form; without the
  // norm (the callers refuse a fused norm above 16 rows) up to 32 rows the 32-row kernel, and beyond that the kernel
  // that keeps the weight and streams the rows past it, so that the weight is read once whatever the row count
  const unsigned col_groups = (unsigned)((heads * 32 + 9) / 10);
  const bool use_rows = rows > 32;                        // (at 17..32 rows the 32-row kernel is 0.7-1.6 us faster: it overlaps the two streams)
  if (rows <= 8) launch_qkv_decode_r8(8, norm, emb, w8, dim3(col_groups, 1), st, a, ra, fr);
  else if (rows <= 16 && (norm != 0 || emb)) launch_qkv_decode_r8(16, norm, emb, w8, dim3(col_groups, 1), st, a, ra, fr);
  else if (use_rows) launch_qkv_decode_rows(w8, dim3(col_groups, 1), st, a, ra, fr);
  else {
    const int64_t chunks = (rows + 31) / 32;
    TLLM_REQUIRE(chunks <= 65535, TLLM_E_SHAPE, "%s: rows %lld too many for the decode kernel", what, (long long)rows);
    launch_qkv_decode_r32(w8, dim3(col_groups, (unsigned)chunks), st, a, ra, fr);
  }
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
  if (hidden == 2880 && head_dim == 64)
    return decode_2880_entry("qkv_rope_decode_w8", x, norm_scale, scale_is_bf16, eps, W8, w_scale, true, b, q, k, v, q_row_stride,
                             k_row_stride, v_row_stride, kv_slot_stride, rows, hidden, n_q_heads, n_kv_heads, head_dim, rope, stream);
  // other shapes: the general MFMA decode kernel with the fp8 weight (no fused norm there)
  QkvArgs a;
  RopeArgs ra;
  YarnFreqs fr;
  int rc = qkv_validate("qkv_rope_decode_w8", x, W8, q, k, v, q_row_stride, k_row_stride, v_row_stride, kv_slot_stride, rows, hidden,
                        n_q_heads, n_kv_heads, head_dim, rope, &a, &ra, &fr);
  if (rc != TLLM_OK) return rc;
  TLLM_REQUIRE(norm_scale == nullptr, TLLM_E_SHAPE,
               "qkv_rope_decode_w8: the fused RMSNorm exists for hidden 2880 / head_dim 64 only: call tllm_rmsnorm_bf16 first");
  TLLM_REQUIRE(head_dim % 16 == 0 && hidden % 32 == 0, TLLM_E_SHAPE,
               "qkv_rope_decode_w8: head_dim %d must be a multiple of 16 and hidden %lld of 32", head_dim, (long long)hidden);
  TLLM_REQUIRE(aligned16(x) && aligned16(W8), TLLM_E_ALIGN, "qkv_rope_decode_w8: x and W must be 16-byte aligned");
  TLLM_REQUIRE(w_scale != nullptr && reinterpret_cast<uintptr_t>(w_scale) % 4 == 0, TLLM_E_ARG,
               "qkv_rope_decode_w8: w_scale must be a 4-byte aligned device pointer");
  const bool out4 = (reinterpret_cast<uintptr_t>(q) % 4 == 0) && (reinterpret_cast<uintptr_t>(k) % 4 == 0) &&
                    (reinterpret_cast<uintptr_t>(v) % 4 == 0) && q_row_stride % 2 == 0 && k_row_stride % 2 == 0 &&
                    v_row_stride % 2 == 0 && kv_slot_stride % 2 == 0;
  TLLM_REQUIRE(out4, TLLM_E_ALIGN, "qkv_rope_decode_w8: q, k, v must be 4-byte aligned with even strides at this shape");
  a.bias = (const bf16*)b;
  a.w_scale = w_scale;
  if (rows == 0) return TLLM_OK;
  const int heads = n_q_heads + 2 * n_kv_heads;
  const int64_t chunks = (rows + 15) / 16;
  TLLM_REQUIRE(chunks <= 65535, TLLM_E_SHAPE, "qkv_rope_decode_w8: rows %lld too many for the decode kernel", (long long)rows);
  // wavefronts per workgroup 1 / 2 / 4 / 8: 16.2 / 13.0 / 13.6 / 14.0 us at hidden 4096, 8 or 16 rows (a run is half the bytes of
  // a bf16 run, so two wavefronts keep as much in flight as one does there); loaded straight into operand layout, four
  // wavefronts: 19.6 us
  constexpr int GNW = 2;
  hipLaunchKernelGGL((qkv_decode_kernel<GNW, 16, true>), dim3((unsigned)(heads * (head_dim / 16)), (unsigned)chunks), dim3(GNW * 64),
                     GNW * 16 * (16 * 32 + 16), static_cast<hipStream_t>(stream), a, ra, fr);
  return check_launch("qkv_rope_decode_w8");
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
  const bool mfma_ok = head_dim % 16 == 0 && hidden % 32 == 0 && aligned16(x) && aligned16(W);
  if (mfma_ok && head_dim == 64 && hidden == 2880 && aligned16(b) && static_cast<int64_t>(heads) * 64 * hidden < (1ll << 31)) {
    // 32-bit element offsets inside W and x are enough here; outputs are written element-wise, any alignment
    return launch_decode_2880("qkv_rope_decode", a, ra, fr, 0, false, rows, heads, st);
  }
  const bool out4 = (reinterpret_cast<uintptr_t>(q) % 4 == 0) && (reinterpret_cast<uintptr_t>(k) % 4 == 0) &&
                    (reinterpret_cast<uintptr_t>(v) % 4 == 0) && q_row_stride % 2 == 0 && k_row_stride % 2 == 0 &&
                    v_row_stride % 2 == 0 && kv_slot_stride % 2 == 0;
  if (mfma_ok && out4) {
    const int64_t chunks = (rows + 15) / 16;
    TLLM_REQUIRE(chunks <= 65535, TLLM_E_SHAPE, "qkv_rope_decode: rows %lld too many for the decode kernel", (long long)rows);
    // wavefronts per workgroup 1 / 2 / 4 / 8: 14.0 / 14.7 / 15.5 / 17.2 us at hidden 4096, 8 rows (one wavefront then walks K in
    // runs of 512, one after the other; two register sets taken in turn, so that the next run's loads are out while a run is
    // multiplied, changed nothing: 14.1 us, at 292 registers one wavefront per SIMD)
    constexpr int GNW = 1;
    constexpr size_t kPatchBytes = GNW * 16 * (16 * 64 + 16);   // the wavefronts' weight patches
    static bool attr_set = false;   // raising the dynamic-LDS limit is idempotent; a benign race at worst repeats it
    if (!attr_set) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_decode_kernel<GNW, 16>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)kPatchBytes);
      TLLM_REQUIRE(e == hipSuccess, TLLM_E_LAUNCH, "qkv_rope_decode: cannot raise LDS limit: %s", hipGetErrorString(e));
      attr_set = true;
    }
    hipLaunchKernelGGL((qkv_decode_kernel<GNW, 16>), dim3((unsigned)(heads * (head_dim / 16)), (unsigned)chunks), dim3(GNW * 64), kPatchBytes, st, a, ra,
                       fr);
    return check_launch("qkv_rope_decode");
  }
  launch_qkv_generic(a, ra, fr, st);
  return check_launch("qkv_rope_decode(generic)");
}
