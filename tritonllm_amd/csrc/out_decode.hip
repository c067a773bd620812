// Decode-size attention out-projection with bias and residual:  out[r, n] = sum_k x[r, k] * W[n, k] + b[n] + res[r, n]
// (out_residual_decode_forward, triton_kernels.py:1470-1517; split-K kernel :1340-1416 + reduce :1419-1467).
// One launch, no partial-sum workspace; `out` may be the residual buffer itself, as in the reference.
//
//   out_decode_r8_kernel    (out_decode_r8.hip)  in_dim == 4096, out_dim % 12 == 0 (gpt-oss: [2880, 4096]), up to 8 rows
//   out_decode_r32_kernel   (out_decode_r32.hip) the same shape, more rows in chunks of 32
//                           both: bf16 or fp8 weight, weight-streaming through LDS, twelve output features per workgroup
//   out_generic_kernel      any other shape: one wavefront per (row, feature) dot product.
//
// W8: fp8 (OCP e4m3) weight with one fp32 scale per output row, as the reference's ATTN_FP8 option
// (triton_kernels.py:1385-1408); the values are widened to bf16 (exact) on their way into LDS and the row scale
// multiplies the finished sum.
#include "out_common.h"

namespace tllm {

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
  if (in_dim == 4096 && out_dim % 12 == 0 && aligned16(x) && aligned16(W) && out_dim * in_dim < (1ll << 31)) {
    const int64_t chunks = (rows + 31) / 32;
    TLLM_REQUIRE(chunks <= 65535, TLLM_E_SHAPE, "out_residual_decode: rows %lld too many for the decode kernel", (long long)rows);
    const dim3 grid((unsigned)(out_dim / 12), (unsigned)chunks);
    if (rows <= 8) launch_out_decode_r8(grid, st, a);
    else launch_out_decode_r32(grid, st, a);
    return check_launch("out_residual_decode");
  }
  TLLM_REQUIRE(rows <= 65535, TLLM_E_SHAPE, "out_residual_decode: rows %lld too many for the generic kernel", (long long)rows);
  hipLaunchKernelGGL(out_generic_kernel, dim3((unsigned)((out_dim + 3) / 4), (unsigned)rows), dim3(256), 0, st, a);
  return check_launch("out_residual_decode(generic)");
}
