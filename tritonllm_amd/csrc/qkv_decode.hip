// Decode-size fused QKV projection + bias + rotary: a weight-streaming kernel.
//
// The 29.5 MB weight is read exactly once per call, so the kernel is HBM-bound and is
// organised around keeping the whole weight in flight:
//   * a workgroup owns 16 weight rows of one head -- dims [8p, 8p+8) and their rotation
//     partners [32+8p, 32+8p+8) -- so a rotation pair never leaves the workgroup;
//     80 heads x 4 pieces = 320 workgroups, all resident at once on 256 CUs;
//   * the K dimension is split over the workgroup's wavefronts; every wavefront issues
//     all of its 128-bit weight loads (and the matching activation loads, which hit L2)
//     before the first multiply, so ~all of W is requested up front;
//   * the arithmetic is v_mfma_f32_16x16x32_bf16 with the weight rows as the M side and
//     up to 16 activation rows as the N side -- the matrix core does the K reduction
//     across lanes for free and leaves the VALU idle for the rotary epilogue;
//   * partial tiles of the wavefronts meet in LDS; wavefront 0 adds the bias, rotates the
//     fp32 accumulator with cos/sin it computed while the loads were in flight, rounds
//     once to bf16 and writes q / k / v (k and v optionally into a KV-cache slot).
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
  bf16* out = qkv_out_ptr(a, ra, row, head);
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
// the weight-streaming MFMA kernel (head_dim == 64, hidden % 32 == 0)
template <int NW, int SPW, bool kExact>   // kExact: hidden == 32 * NW * SPW, no tail guards anywhere in the loop
__global__ __launch_bounds__(NW * 64) void qkv_decode_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr) {
  __shared__ float red[NW][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int head = blockIdx.x >> 2, piece = blockIdx.x & 3;
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * 16;
  const int kvec = a.hidden >> 3;       // 16-byte vectors per row
  const int nsteps = a.hidden >> 5;     // MFMA k-steps of 32
  const int m = lane & 15, g = lane >> 4;

  // A side: weight row held by this lane. Tile row m = 4*qd + i maps to dim
  // 8*piece + 2*qd + (i & 1), plus 32 when i >= 2, so that after the MFMA each lane's
  // four accumulators are two (lo, hi) rotation pairs.
  const int dim_a = 8 * piece + 2 * (m >> 2) + (m & 1) + ((m & 2) ? 32 : 0);
  const bf16x8* wrow = reinterpret_cast<const bf16x8*>(a.W) + (static_cast<int64_t>(head) * 64 + dim_a) * kvec + g;
  // B side: activation row n = lane % 16 of this 16-row chunk. Lanes past the last row re-read
  // a valid row (same addresses as a live lane, so no extra traffic); their output column is dropped.
  const int64_t xrow_idx = row0 + m;
  const bool xvalid = xrow_idx < a.rows;
  const int nvalid = static_cast<int>(a.rows - row0 < 16 ? a.rows - row0 : 16);
  const bf16x8* xrow = reinterpret_cast<const bf16x8*>(a.x) + (row0 + (xvalid ? m : m % nvalid)) * kvec + g;

  const bool rotate = a.has_rope && head < a.n_q_heads + a.n_kv_heads;
  // position first: its load is then the oldest outstanding one and can be waited for alone
  // and the two YaRN frequencies of this lane's pairs come out of the kernel-argument block now,
  // so nothing issued after the weight loads has to be waited for before the cos/sin math.
  int64_t pos = 0;
  const float f0 = fr.v[8 * piece + 2 * g], f1 = fr.v[8 * piece + 2 * g + 1];   // zeros when no YaRN block was given
  if (rotate && wave == 0) pos = rope_position_raw(ra, xvalid ? xrow_idx : row0);
  __builtin_amdgcn_sched_barrier(0);

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float cs[2] = {1.f, 1.f}, sn[2] = {0.f, 0.f};

  for (int s0 = wave * SPW; s0 < nsteps; s0 += NW * SPW) {
    bf16x8 wa[SPW], xb[SPW];
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      const int step = s0 + i;
      if (kExact || step < nsteps) {
        wa[i] = __builtin_nontemporal_load(wrow + step * 4);
        xb[i] = xrow[step * 4];
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          wa[i][j] = static_cast<bf16>(0.f);
          xb[i][j] = static_cast<bf16>(0.f);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (wave == 0 && s0 == 0 && rotate) {
      // cos/sin for this lane's two pairs, computed while the weight loads are in flight
      const int d0 = 8 * piece + 2 * g;
      pos = rope_wrap(pos, ra.max_ctx);
      if (ra.use_yarn) {
        yarn_cos_sin(pos, f0, ra.concentration, &cs[0], &sn[0]);
        yarn_cos_sin(pos, f1, ra.concentration, &cs[1], &sn[1]);
      } else {
        rope_cos_sin(ra, fr, pos, d0, &cs[0], &sn[0]);
        rope_cos_sin(ra, fr, pos, d0 + 1, &cs[1], &sn[1]);
      }
    }
#pragma unroll
    for (int i = 0; i < SPW; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[i], xb[i], acc, 0, 0, 0);
    if (kExact) break;
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

  // Output side: lane holds activation row n = lane % 16 and, with qd = lane / 16,
  // dims d0 = 8*piece + 2*qd and d0 + 1 (acc[0], acc[1]) and their partners (acc[2], acc[3]).
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
    const float r0 = lo0 * cs[0] - hi0 * sn[0], r1 = lo1 * cs[1] - hi1 * sn[1];
    const float r2 = hi0 * cs[0] + lo0 * sn[0], r3 = hi1 * cs[1] + lo1 * sn[1];
    lo0 = r0;
    lo1 = r1;
    hi0 = r2;
    hi1 = r3;
  }
  bf16* out = qkv_out_ptr(a, ra, xrow_idx, head);
  bf16x2 plo, phi;
  plo[0] = static_cast<bf16>(lo0);
  plo[1] = static_cast<bf16>(lo1);
  phi[0] = static_cast<bf16>(hi0);
  phi[1] = static_cast<bf16>(hi1);
  *reinterpret_cast<bf16x2*>(out + d0) = plo;
  *reinterpret_cast<bf16x2*>(out + d0 + 32) = phi;
}

}  // namespace tllm

using namespace tllm;

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
  const bool fast = head_dim == 64 && hidden % 32 == 0 && aligned16(x) && aligned16(W) &&
                    (reinterpret_cast<uintptr_t>(q) % 4 == 0) && (reinterpret_cast<uintptr_t>(k) % 4 == 0) &&
                    (reinterpret_cast<uintptr_t>(v) % 4 == 0) && q_row_stride % 2 == 0 && k_row_stride % 2 == 0 &&
                    v_row_stride % 2 == 0 && kv_slot_stride % 2 == 0;
  if (!fast) {
    launch_qkv_generic(a, ra, fr, st);
    return check_launch("qkv_rope_decode(generic)");
  }
  const int heads = n_q_heads + 2 * n_kv_heads;
  const int64_t chunks = (rows + 15) / 16;
  TLLM_REQUIRE(chunks <= 65535, TLLM_E_SHAPE, "qkv_rope_decode: rows %lld too many for the decode kernel", (long long)rows);
  dim3 grid((unsigned)(heads * 4), (unsigned)chunks);
  if (hidden == 32 * 5 * 18)   // 2880: five wavefronts x 18 k-steps, the whole weight in flight at once
    hipLaunchKernelGGL((qkv_decode_kernel<5, 18, true>), grid, dim3(5 * 64), 0, st, a, ra, fr);
  else
    hipLaunchKernelGGL((qkv_decode_kernel<4, 16, false>), grid, dim3(4 * 64), 0, st, a, ra, fr);
  return check_launch("qkv_rope_decode");
}
