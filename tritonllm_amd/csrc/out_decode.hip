// Decode-size attention out-projection with bias and residual:  out[r, n] = sum_k x[r, k] * W[n, k] + b[n] + res[r, n]
// (out_residual_decode_forward, triton_kernels.py:1470-1517; split-K kernel :1340-1416 + reduce :1419-1467).
// One launch, no partial-sum workspace; `out` may be the residual buffer itself, as in the reference.
//
//   out_decode_r8_kernel    (out_decode_r8.hip) in_dim == 4096, out_dim % 12 == 0, up to 8 rows, bf16 or fp8 weight
//   out_decode_r32_kernel   (out_decode_r32.hip) the same shape, more rows in chunks of 32, bf16 weight
//   out_decode_cu_kernel    in_dim == 4096, out_dim % 12 == 0 (gpt-oss: [2880, 4096]), more rows, fp8 weight: the weight-streaming layout
//                           of the decode QKV kernel -- one workgroup per CU-sized share of the output features,
//                           sixteen wavefronts splitting K, every load unconditional and issued up front, operands
//                           through wavefront-private LDS patches into v_mfma_f32_32x32x16_bf16, one reduction.
//   out_generic_kernel      any other shape: one wavefront per (row, feature) dot product.
//
// W8: fp8 (OCP e4m3) weight with one fp32 scale per output row, as the reference's ATTN_FP8 option
// (triton_kernels.py:1385-1408); the values are widened to bf16 (exact) on their way into LDS and the row scale
// multiplies the finished sum.
#include "out_common.h"

namespace tllm {

template <int XR, int CH, bool W8>
__global__ __launch_bounds__(1024) void out_decode_cu_kernel(OutArgs a) {
  constexpr int NW = 16, SPW = 8, NCH = SPW / CH, RW = 12;   // 16 wavefronts x 8 slices of 32 = K 4096; 12 features per workgroup
  constexpr int KV = 512;                     // 16-byte vectors per activation row
  constexpr int KVW = W8 ? 256 : 512;         // ... per weight row
  constexpr int WROW = CH * 64 + 16;          // padded patch row, bytes
  constexpr int CPR = CH * 4;                 // 16-byte chunks per row per patch (bf16)
  constexpr int CPRW = W8 ? CPR / 2 : CPR;    // ... of the weight as it lies in memory
  constexpr int WL = (RW * CPRW + 63) / 64;   // weight load instructions per patch
  constexpr int XL = (XR * CPR + 63) / 64;    // activation load instructions per patch
  constexpr int PATCH = (16 + XR) * WROW;     // 16 tile rows for the weight (12 used) + XR activation rows
  constexpr int RED = XR * 16;                // floats per wavefront in the reduction buffer
  static_assert(SPW % CH == 0, "patches must tile the K slice");
  static_assert(RED * 4 <= PATCH, "reduction buffer aliases the patches");
  static_assert(16 * XR <= 1024, "one epilogue thread per (feature slot, activation row)");
  static_assert(NW * PATCH <= 160 * 1024, "LDS per workgroup");
  __shared__ __align__(16) unsigned char lds[NW * PATCH];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * RW;
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * XR;
  const int nvalid = static_cast<int>(a.rows - row0 < XR ? a.rows - row0 : XR);

  // ---- epilogue role of this thread: feature slot en, activation row er (clamped to real ones for the loads)
  const int en = tid & 15, er = tid >> 4;
  const bool evalid = tid < 16 * XR && en < RW && n0 + en < a.out_dim && er < nvalid;
  const int efeat = evalid ? n0 + en : 0;
  const int64_t erow = row0 + (evalid ? er : 0);

  // ---- every global load of the kernel, oldest first; none is predicated (a predicated load makes the compiler
  // wait for everything in flight where the branches join): absent operands read a valid dummy address instead
  const unsigned short* bias_ptr = reinterpret_cast<const unsigned short*>(a.bias ? a.bias : a.x);
  const unsigned short* res_ptr = a.res ? reinterpret_cast<const unsigned short*>(a.res) + erow * a.res_rs + efeat
                                        : reinterpret_cast<const unsigned short*>(a.x);
  const unsigned short b_bits = bias_ptr[a.bias ? efeat : 0];
  const unsigned short r_bits = *res_ptr;
  float ws = 1.f;
  if constexpr (W8) ws = a.w_scale[efeat];
  __builtin_amdgcn_sched_barrier(0);

  const bf16x8* xg = reinterpret_cast<const bf16x8*>(a.x) + row0 * KV + wave * (SPW * 4);
  const bf16x8* wg = reinterpret_cast<const bf16x8*>(a.W) + wave * (W8 ? SPW * 2 : SPW * 4);   // 16-byte units either way
  bf16x8 xr[NCH * XL], wr[NCH * WL];
#pragma unroll
  for (int idx = 0; idx < NCH * WL; ++idx) {        // weight load idx: patch j = idx / WL, chunk slot i = idx % WL
    const int j = idx / WL, i = idx % WL;
    int e = i * 64 + lane;                           // patch chunk e -> weight row e / CPRW of the workgroup's twelve
    e = e < RW * CPRW ? e : RW * CPRW - 1;
    const int r = e / CPRW, kc = e - r * CPRW;
    int n = n0 + r;
    n = n < a.out_dim ? n : a.out_dim - 1;
    wr[idx] = __builtin_nontemporal_load(wg + static_cast<unsigned>(n) * static_cast<unsigned>(KVW) + j * CPRW + kc);
  }
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
#pragma unroll
    for (int i = 0; i < XL; ++i) {                   // patch chunk e -> activation row e / CPR, chunk e % CPR
      int e = i * 64 + lane;
      e = e < XR * CPR ? e : XR * CPR - 1;
      int r = e / CPR;
      const int kc = e - r * CPR;
      r = r < nvalid ? r : nvalid - 1;
      xr[j * XL + i] = xg[r * KV + j * CPR + kc];
    }
  }
  __builtin_amdgcn_sched_barrier(0);

  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  const int m = lane & 31, h = lane >> 5;
  unsigned char* wp = lds + wave * PATCH;            // 16 tile rows (the twelve features, four never written)
  unsigned char* xp = wp + 16 * WROW;                // XR activation rows
  const unsigned char* wfrag = wp + (m & 15) * WROW + h * 16;         // tile rows 16-31 repeat 0-15: their sums are never stored
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
        if (e < RW * CPRW) {
          *reinterpret_cast<bf16x8*>(wp + r * WROW + kc * 32) = w0;
          *reinterpret_cast<bf16x8*>(wp + r * WROW + kc * 32 + 16) = w1;
        }
      } else {
        if (e < RW * CPRW) *reinterpret_cast<bf16x8*>(wp + r * WROW + kc * 16) = wr[j * WL + i];
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

  // ---- sixteen partial tiles -> LDS as [wave][tile row][activation row]; only tile rows 0-15 (accumulator
  // registers 0-7: rows 8*(v>>2) + 4*h + (v&3)) carry features
  __syncthreads();
  float* red = reinterpret_cast<float*>(lds);
  if (m < XR) {
#pragma unroll
    for (int v = 0; v < 8; ++v) red[wave * RED + (8 * (v >> 2) + 4 * h + (v & 3)) * XR + m] = acc[v];
  }
  __syncthreads();
  if (!evalid) return;
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) s += red[w * RED + en * XR + er];
  if constexpr (W8) s *= ws;
  if (a.bias) s += __uint_as_float(static_cast<unsigned>(b_bits) << 16);
  if (a.res) s += __uint_as_float(static_cast<unsigned>(r_bits) << 16);
  a.out[erow * a.out_rs + efeat] = static_cast<bf16>(s);
}

// Any shape: one wavefront per (row, feature); 2-byte loads, shuffle reduction.
__global__ __launch_bounds__(256) void out_generic_kernel(OutArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t n = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int64_t r = blockIdx.y;
  if (n >= a.out_dim) return;
  const bf16* xrow = a.x + r * a.in_dim;
  float s = 0.f;
  if (a.w_scale) {
    const unsigned char* wrow = reinterpret_cast<const unsigned char*>(a.W) + n * a.in_dim;
    for (int k = lane; k < a.in_dim; k += 64) {
      typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
      const f32x2 w = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(wrow[k]), false);
      s = fmaf(static_cast<float>(xrow[k]), w[0], s);
    }
    s = wave_sum(s) * a.w_scale[n];
  } else {
    const bf16* wrow = reinterpret_cast<const bf16*>(a.W) + n * a.in_dim;
    for (int k = lane; k < a.in_dim; k += 64) s = fmaf(static_cast<float>(xrow[k]), static_cast<float>(wrow[k]), s);
    s = wave_sum(s);
  }
  if (lane != 0) return;
  if (a.bias) s += static_cast<float>(a.bias[n]);
  if (a.res) s += static_cast<float>(a.res[r * a.res_rs + n]);
  a.out[r * a.out_rs + n] = static_cast<bf16>(s);
}

}  // namespace tllm

using namespace tllm;

extern "C" int tllm_out_residual_decode_bf16(const void* x, const void* W, const float* w_scale, const void* bias, const void* residual,
                                             void* out, int64_t res_row_stride, int64_t out_row_stride, int64_t rows, int64_t in_dim,
                                             int64_t out_dim, void* stream) {
  TLLM_REQUIRE(rows >= 0 && in_dim >= 1 && out_dim >= 1, TLLM_E_SHAPE, "out_residual_decode: rows %lld, in_dim %lld, out_dim %lld",
               (long long)rows, (long long)in_dim, (long long)out_dim);
  TLLM_REQUIRE(in_dim < (1ll << 31) && out_dim < (1ll << 31) && in_dim * out_dim < (1ll << 40), TLLM_E_SHAPE,
               "out_residual_decode: weight too large");
  if (rows == 0) return TLLM_OK;
  TLLM_REQUIRE(x && W && out, TLLM_E_ARG, "out_residual_decode: x, W and out must not be NULL");
  TLLM_REQUIRE(out_row_stride >= out_dim && (residual == nullptr || res_row_stride >= out_dim), TLLM_E_ARG,
               "out_residual_decode: row strides must be >= out_dim");
  TLLM_REQUIRE(w_scale == nullptr || reinterpret_cast<uintptr_t>(w_scale) % 4 == 0, TLLM_E_ALIGN, "out_residual_decode: w_scale alignment");
  OutArgs a;
  a.x = (const bf16*)x;
  a.W = W;
  a.w_scale = w_scale;
  a.bias = (const bf16*)bias;
  a.res = (const bf16*)residual;
  a.out = (bf16*)out;
  a.res_rs = res_row_stride;
  a.out_rs = out_row_stride;
  a.rows = rows;
  a.in_dim = (int)in_dim;
  a.out_dim = (int)out_dim;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool w8 = w_scale != nullptr;
  if (in_dim == 4096 && out_dim % 12 == 0 && aligned16(x) && aligned16(W) && out_dim * in_dim < (1ll << 31)) {
    const int xr = rows <= 8 ? 8 : (rows <= 16 ? 16 : 32);
    const int64_t chunks = (rows + xr - 1) / xr;
    TLLM_REQUIRE(chunks <= 65535, TLLM_E_SHAPE, "out_residual_decode: rows %lld too many for the decode kernel", (long long)rows);
    dim3 grid((unsigned)(out_dim / 12), (unsigned)chunks);
    if (rows <= 8) {
      launch_out_decode_r8(grid, st, a);
      return check_launch("out_residual_decode");
    }
    if (!w8) {
      launch_out_decode_r32(dim3((unsigned)(out_dim / 12), (unsigned)((rows + 31) / 32)), st, a);
      return check_launch("out_residual_decode");
    }
#define TLLM_OUT(XR, CH)                                                                                   \
  do {                                                                                                     \
    if (w8) hipLaunchKernelGGL((out_decode_cu_kernel<XR, CH, true>), grid, dim3(1024), 0, st, a);         \
    else hipLaunchKernelGGL((out_decode_cu_kernel<XR, CH, false>), grid, dim3(1024), 0, st, a);           \
  } while (0)
    if (xr == 8) TLLM_OUT(8, 4);
    else if (xr == 16) TLLM_OUT(16, 4);
    else TLLM_OUT(32, 2);
#undef TLLM_OUT
    return check_launch("out_residual_decode");
  }
  TLLM_REQUIRE(rows <= 65535, TLLM_E_SHAPE, "out_residual_decode: rows %lld too many for the generic kernel", (long long)rows);
  hipLaunchKernelGGL(out_generic_kernel, dim3((unsigned)((out_dim + 3) / 4), (unsigned)rows), dim3(256), 0, st, a);
  return check_launch("out_residual_decode(generic)");
}
