// RMSNorm for bf16 rows on gfx950.
//
// Memory-bound: a row is read once (held in registers as 128-bit bf16 vectors),
// reduced in fp32, scaled and written once. Two shapes of the same idea:
//   * wave-per-row  -- many rows (prefill): each 64-lane wavefront owns a row,
//                      reduction is a pure wavefront shuffle, no LDS, no barrier;
//   * block-per-row -- few rows (decode): one 256-lane workgroup owns a row so a
//                      single row's latency is spread over four wavefronts;
//                      shuffle inside each wavefront, then a 4-entry LDS exchange.
// A scalar two-pass kernel covers hidden sizes / alignments the vector paths do not.
#include "common.h"

namespace tllm {

template <bool kScaleBf16>
__device__ __forceinline__ void load_scale8(const void* scale, int vec, float s[8]) {
  if constexpr (kScaleBf16) {
    bf16x8 sv = reinterpret_cast<const bf16x8*>(scale)[vec];
#pragma unroll
    for (int j = 0; j < 8; ++j) s[j] = static_cast<float>(sv[j]);
  } else {
    const f32x4* sp = reinterpret_cast<const f32x4*>(scale) + 2 * vec;
    f32x4 a = sp[0], b = sp[1];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      s[j] = a[j];
      s[4 + j] = b[j];
    }
  }
}

template <bool kScaleBf16>
__device__ __forceinline__ bf16x8 normalize8(bf16x8 xv, float rinv, const void* scale, int vec) {
  float s[8];
  load_scale8<kScaleBf16>(scale, vec, s);
  bf16x8 o;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = static_cast<bf16>(static_cast<float>(xv[j]) * rinv * s[j]);
  return o;
}

__device__ __forceinline__ float sumsq8(bf16x8 v) {
  float a = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float f = static_cast<float>(v[j]);
    a = fmaf(f, f, a);
  }
  return a;
}

// One wavefront per row; VPL = 16-byte vectors per lane (row length <= VPL*64*8).
template <int VPL, bool kScaleBf16>
__global__ __launch_bounds__(256) void rmsnorm_wave_kernel(const bf16x8* x, const void* __restrict__ scale,
                                                           bf16x8* out, int64_t rows, int nvec, float hidden_f, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const bf16x8* xr = x + row * nvec;
  bf16x8 v[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int idx = lane + i * 64;
    if (idx < nvec) {
      v[i] = xr[idx];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[i][j] = static_cast<bf16>(0.f);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) ss += sumsq8(v[i]);
  ss = wave_sum(ss);
  const float rinv = rsqrtf(ss / hidden_f + eps);
  bf16x8* orow = out + row * nvec;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int idx = lane + i * 64;
    if (idx < nvec) __builtin_nontemporal_store(normalize8<kScaleBf16>(v[i], rinv, scale, idx), orow + idx);   // streamed out: measured 5-18 % faster
  }
}

// One 256-lane workgroup per row; VPT = 16-byte vectors per thread.
template <int VPT, bool kScaleBf16>
__global__ __launch_bounds__(256) void rmsnorm_block_kernel(const bf16x8* x, const void* __restrict__ scale,
                                                            bf16x8* out, int nvec, float hidden_f, float eps) {
  __shared__ float part[4];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const bf16x8* xr = x + row * nvec;
  bf16x8 v[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = tid + i * 256;
    if (idx < nvec) {
      v[i] = xr[idx];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[i][j] = static_cast<bf16>(0.f);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) ss += sumsq8(v[i]);
  ss = wave_sum(ss);
  if ((tid & 63) == 0) part[tid >> 6] = ss;
  __syncthreads();
  ss = (part[0] + part[1]) + (part[2] + part[3]);
  const float rinv = rsqrtf(ss / hidden_f + eps);
  bf16x8* orow = out + row * nvec;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = tid + i * 256;
    if (idx < nvec) __builtin_nontemporal_store(normalize8<kScaleBf16>(v[i], rinv, scale, idx), orow + idx);   // streamed out: measured 5-18 % faster
  }
}

// Any hidden size / alignment: scalar loads, two passes over the row (the second hits cache).
// The row's input is fully read before any of it is overwritten only per element, which is
// all in-place use needs: element c of the output depends on element c of the input and the sum.
__global__ __launch_bounds__(256) void rmsnorm_scalar_kernel(const bf16* x, const void* __restrict__ scale,
                                                             int scale_is_bf16, bf16* out, int64_t hidden, float hidden_f,
                                                             float eps) {
  __shared__ float part[4];
  const int tid = threadIdx.x;
  const bf16* xr = x + static_cast<int64_t>(blockIdx.x) * hidden;
  bf16* orow = out + static_cast<int64_t>(blockIdx.x) * hidden;
  float ss = 0.f;
  for (int64_t c = tid; c < hidden; c += 256) {
    float f = static_cast<float>(xr[c]);
    ss = fmaf(f, f, ss);
  }
  ss = wave_sum(ss);
  if ((tid & 63) == 0) part[tid >> 6] = ss;
  __syncthreads();
  ss = (part[0] + part[1]) + (part[2] + part[3]);
  const float rinv = rsqrtf(ss / hidden_f + eps);
  for (int64_t c = tid; c < hidden; c += 256) {
    float s = scale_is_bf16 ? static_cast<float>(reinterpret_cast<const bf16*>(scale)[c]) : reinterpret_cast<const float*>(scale)[c];
    orow[c] = static_cast<bf16>(static_cast<float>(xr[c]) * rinv * s);
  }
}

template <bool kScaleBf16>
static void launch_wave(int vpl, const bf16x8* x, const void* scale, bf16x8* out, int64_t rows, int nvec, float inv_h, float eps,
                        hipStream_t st) {
  dim3 grid(static_cast<unsigned>((rows + 3) / 4)), block(256);
#define TLLM_CASE(V)                                                                                           \
  case V:                                                                                                      \
    hipLaunchKernelGGL((rmsnorm_wave_kernel<V, kScaleBf16>), grid, block, 0, st, x, scale, out, rows, nvec, inv_h, eps); \
    break;
  switch (vpl) {
    TLLM_CASE(1) TLLM_CASE(2) TLLM_CASE(3) TLLM_CASE(4) TLLM_CASE(5) TLLM_CASE(6) TLLM_CASE(7) TLLM_CASE(8)
    TLLM_CASE(9) TLLM_CASE(10) TLLM_CASE(11) TLLM_CASE(12) TLLM_CASE(13) TLLM_CASE(14) TLLM_CASE(15) TLLM_CASE(16)
  }
#undef TLLM_CASE
}

template <bool kScaleBf16>
static void launch_block(int vpt, const bf16x8* x, const void* scale, bf16x8* out, int64_t rows, int nvec, float inv_h, float eps,
                         hipStream_t st) {
  dim3 grid(static_cast<unsigned>(rows)), block(256);
#define TLLM_CASE(V)                                                                                      \
  case V:                                                                                                 \
    hipLaunchKernelGGL((rmsnorm_block_kernel<V, kScaleBf16>), grid, block, 0, st, x, scale, out, nvec, inv_h, eps); \
    break;
  switch (vpt) { TLLM_CASE(1) TLLM_CASE(2) TLLM_CASE(3) TLLM_CASE(4) }
#undef TLLM_CASE
}

}  // namespace tllm

using namespace tllm;

// Rows at or below this go to the workgroup-per-row kernel (latency), above to wave-per-row (throughput).
static constexpr int64_t kBlockPerRowMaxRows = 512;

extern "C" int tllm_rmsnorm_bf16(const void* x, const void* scale, int scale_is_bf16, void* out, int64_t rows, int64_t hidden,
                                 float eps, void* stream) {
  TLLM_REQUIRE(rows >= 0 && hidden > 0, TLLM_E_ARG, "rmsnorm: rows %lld / hidden %lld invalid", (long long)rows, (long long)hidden);
  if (rows == 0) return TLLM_OK;
  TLLM_REQUIRE(x && scale && out, TLLM_E_ARG, "rmsnorm: null pointer");
  TLLM_REQUIRE(rows < (1ll << 31), TLLM_E_SHAPE, "rmsnorm: rows %lld too large", (long long)rows);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float inv_h = static_cast<float>(hidden);  // divisor of the mean
  const bool vec_ok = hidden % 8 == 0 && aligned16(x) && aligned16(out) && aligned16(scale);
  const int64_t nvec = hidden / 8;
  if (vec_ok && rows <= kBlockPerRowMaxRows && nvec <= 4 * 256) {
    const int vpt = static_cast<int>((nvec + 255) / 256);
    if (scale_is_bf16)
      launch_block<true>(vpt, (const bf16x8*)x, scale, (bf16x8*)out, rows, (int)nvec, inv_h, eps, st);
    else
      launch_block<false>(vpt, (const bf16x8*)x, scale, (bf16x8*)out, rows, (int)nvec, inv_h, eps, st);
  } else if (vec_ok && nvec <= 16 * 64) {
    const int vpl = static_cast<int>((nvec + 63) / 64);
    if (scale_is_bf16)
      launch_wave<true>(vpl, (const bf16x8*)x, scale, (bf16x8*)out, rows, (int)nvec, inv_h, eps, st);
    else
      launch_wave<false>(vpl, (const bf16x8*)x, scale, (bf16x8*)out, rows, (int)nvec, inv_h, eps, st);
  } else {
    hipLaunchKernelGGL(rmsnorm_scalar_kernel, dim3((unsigned)rows), dim3(256), 0, st, (const bf16*)x, scale, scale_is_bf16,
                       (bf16*)out, hidden, inv_h, eps);
  }
  return check_launch("rmsnorm");
}
