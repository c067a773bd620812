// Clamped SwiGLU: out = g * sigmoid(alpha * g) * (l + 1) with g clamped from above and l on both sides.
//
// Pure streaming (17 280 bytes per gpt-oss row): each lane loads 32 bytes of input
// (eight gate/linear pairs when interleaved), computes in fp32 and stores one 128-bit
// vector of eight bf16 outputs. The grid runs over the output vectors of the
// whole [rows, n_out] matrix, one per thread, so small and large row counts use the same kernel.
#include "common.h"

namespace tllm {

__device__ __forceinline__ float swiglu1(float g, float l, float alpha, float limit, bool has_limit) {
  if (has_limit) {
    g = g > limit ? limit : g;                 // gate: upper clamp only (NaN stays NaN, as torch.clamp)
    l = l > limit ? limit : l;                 // linear: both sides
    l = l < -limit ? -limit : l;
  }
  // g * sigmoid(alpha * g). The quotient goes through the hardware reciprocal (1 ulp): an IEEE division is ten more
  // instructions per element and this kernel has eight elements per 48 bytes of traffic to get through.
  const float s = g * __builtin_amdgcn_rcpf(1.0f + __expf(-alpha * g));
  return fmaf(s, l, s);                              // s * (l + 1)
}

// One output vector per thread, workgroups in memory order: the grid then sweeps the input like one contiguous
// read (measured at [32768, 5760]: 87 us = 6.5 TB/s; a grid-stride loop over 32 workgroups per CU 94 us, with two
// or four vectors per thread and iteration 99 / 112 us).
template <bool kInterleaved>
__global__ __launch_bounds__(256) void swiglu_vec_kernel(const bf16x8* __restrict__ x, bf16x8* __restrict__ out, int64_t rows,
                                                         int nvec_out, int64_t x_row_stride_vec, float alpha, float limit,
                                                         int has_limit) {
  const int64_t total = rows * nvec_out;
  const int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (v >= total) return;
  const int64_t row = v / nvec_out;
  const int c = static_cast<int>(v - row * nvec_out);
  const bf16x8* xr = x + row * x_row_stride_vec;
  bf16x8 a, b;
  if constexpr (kInterleaved) {
    a = __builtin_nontemporal_load(xr + 2 * c);
    b = __builtin_nontemporal_load(xr + 2 * c + 1);
  } else {
    a = __builtin_nontemporal_load(xr + c);
    b = __builtin_nontemporal_load(xr + nvec_out + c);
  }
  bf16x8 o;
  if constexpr (kInterleaved) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[j] = static_cast<bf16>(swiglu1(static_cast<float>(a[2 * j]), static_cast<float>(a[2 * j + 1]), alpha, limit, has_limit));
      o[4 + j] = static_cast<bf16>(swiglu1(static_cast<float>(b[2 * j]), static_cast<float>(b[2 * j + 1]), alpha, limit, has_limit));
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      o[j] = static_cast<bf16>(swiglu1(static_cast<float>(a[j]), static_cast<float>(b[j]), alpha, limit, has_limit));
  }
  __builtin_nontemporal_store(o, out + v);
}

// A decode batch: up to 1.5 M outputs (256 rows of 5760). Two outputs per thread, so that the chain load -> exp ->
// reciprocal -> store is as short as it gets and spread over four times as many lanes; such a launch is all latency
// ([32, 5760] 2.08 -> 1.95 us, [128, 5760] 2.21 -> 2.00, [256, 5760] 2.39 -> 2.26, level with the vector kernel at 360 rows).
template <bool kInterleaved>
__global__ __launch_bounds__(256) void swiglu_small_kernel(const bf16x2* __restrict__ x, bf16x2* __restrict__ out, unsigned total_pairs,
                                                           unsigned pairs_per_row, unsigned x_row_stride_pairs, float alpha, float limit,
                                                           int has_limit) {
  const unsigned v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v >= total_pairs) return;
  const unsigned row = v / pairs_per_row, c = v - row * pairs_per_row;
  const bf16x2* xr = x + static_cast<size_t>(row) * x_row_stride_pairs;
  bf16x2 a, b;                                            // interleaved: (g0, l0), (g1, l1); else (g0, g1), (l0, l1)
  if constexpr (kInterleaved) {
    a = xr[2 * c];
    b = xr[2 * c + 1];
  } else {
    a = xr[c];
    b = xr[pairs_per_row + c];
  }
  bf16x2 o;
  if constexpr (kInterleaved) {
    o[0] = static_cast<bf16>(swiglu1(static_cast<float>(a[0]), static_cast<float>(a[1]), alpha, limit, has_limit));
    o[1] = static_cast<bf16>(swiglu1(static_cast<float>(b[0]), static_cast<float>(b[1]), alpha, limit, has_limit));
  } else {
    o[0] = static_cast<bf16>(swiglu1(static_cast<float>(a[0]), static_cast<float>(b[0]), alpha, limit, has_limit));
    o[1] = static_cast<bf16>(swiglu1(static_cast<float>(a[1]), static_cast<float>(b[1]), alpha, limit, has_limit));
  }
  out[v] = o;
}

__global__ __launch_bounds__(256) void swiglu_scalar_kernel(const bf16* __restrict__ x, bf16* __restrict__ out, int64_t rows,
                                                            int64_t n_out, int64_t x_row_stride, float alpha, float limit,
                                                            int has_limit, int interleaved) {
  const int64_t total = rows * n_out;
  const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
    const int64_t row = i / n_out, c = i - row * n_out;
    const bf16* xr = x + row * x_row_stride;
    const float g = static_cast<float>(interleaved ? xr[2 * c] : xr[c]);
    const float l = static_cast<float>(interleaved ? xr[2 * c + 1] : xr[n_out + c]);
    out[i] = static_cast<bf16>(swiglu1(g, l, alpha, limit, has_limit));
  }
}

}  // namespace tllm

using namespace tllm;

extern "C" int tllm_swiglu_bf16(const void* x, void* out, int64_t rows, int64_t n_out, int64_t x_row_stride, float alpha, float limit,
                                int has_limit, int interleaved, void* stream) {
  TLLM_REQUIRE(rows >= 0 && n_out > 0, TLLM_E_ARG, "swiglu: rows %lld / n_out %lld invalid", (long long)rows, (long long)n_out);
  TLLM_REQUIRE(x_row_stride >= 2 * n_out, TLLM_E_ARG, "swiglu: x_row_stride %lld < 2*n_out", (long long)x_row_stride);
  if (rows == 0) return TLLM_OK;
  TLLM_REQUIRE(x && out, TLLM_E_ARG, "swiglu: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec_ok = n_out % 8 == 0 && x_row_stride % 8 == 0 && aligned16(x) && aligned16(out) && n_out / 8 < (1ll << 31);
  if (vec_ok && rows * n_out <= (3 << 18) && x_row_stride < (1ll << 32)) {
    const unsigned pairs_per_row = static_cast<unsigned>(n_out / 2), total_pairs = static_cast<unsigned>(rows) * pairs_per_row;
    dim3 grid((total_pairs + 255) / 256), block(256);
    if (interleaved)
      hipLaunchKernelGGL(swiglu_small_kernel<true>, grid, block, 0, st, (const bf16x2*)x, (bf16x2*)out, total_pairs, pairs_per_row,
                         static_cast<unsigned>(x_row_stride / 2), alpha, limit, has_limit);
    else
      hipLaunchKernelGGL(swiglu_small_kernel<false>, grid, block, 0, st, (const bf16x2*)x, (bf16x2*)out, total_pairs, pairs_per_row,
                         static_cast<unsigned>(x_row_stride / 2), alpha, limit, has_limit);
  } else if (vec_ok) {
    const int64_t total = rows * (n_out / 8);
    const int64_t blocks = (total + 255) / 256;
    TLLM_REQUIRE(blocks < (1ll << 31), TLLM_E_SHAPE, "swiglu: %lld output vectors are too many for one launch", (long long)total);
    dim3 grid(static_cast<unsigned>(blocks)), block(256);
    if (interleaved)
      hipLaunchKernelGGL(swiglu_vec_kernel<true>, grid, block, 0, st, (const bf16x8*)x, (bf16x8*)out, rows, (int)(n_out / 8),
                         x_row_stride / 8, alpha, limit, has_limit);
    else
      hipLaunchKernelGGL(swiglu_vec_kernel<false>, grid, block, 0, st, (const bf16x8*)x, (bf16x8*)out, rows, (int)(n_out / 8),
                         x_row_stride / 8, alpha, limit, has_limit);
  } else {
    const int64_t total = rows * n_out;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(swiglu_scalar_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const bf16*)x, (bf16*)out, rows, n_out,
                       x_row_stride, alpha, limit, has_limit, interleaved);
  }
  return check_launch("swiglu");
}
