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
//
// GATHER form (the first layer of a prompt: x = table[ids] followed by RMSNorm(x), model.py:920 and :476): the row
// comes from the embedding table by token id, is written out unchanged (the hidden state, bit-exact) and normalised
// from the same registers -- one launch and one read of the row instead of two of each. An id outside the table
// yields a zero row (and a zero normalised row) and sets a device flag, as in the gather kernel.
#include "common.h"

namespace tllm {

struct GatherSrc {
  const void* ids;        // [rows] int32 or int64
  int ids_is_i64;
  int64_t vocab;
  bf16x8* x_out;          // [rows, nvec]: the gathered rows
  int* oob;               // device flag or null
};

// row base in the table (null: id out of range)
__device__ __forceinline__ const bf16x8* gather_row(const GatherSrc& g, const bf16x8* table, int64_t row, int nvec, bool flag_lane) {
  const int64_t id = g.ids_is_i64 ? reinterpret_cast<const int64_t*>(g.ids)[row] : reinterpret_cast<const int*>(g.ids)[row];
  if (id < 0 || id >= g.vocab) {
    if (flag_lane && g.oob) *g.oob = 1;
    return nullptr;
  }
  return table + id * nvec;
}

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
template <int VPL, bool kScaleBf16, bool GATHER>
__global__ __launch_bounds__(256) void rmsnorm_wave_kernel(const bf16x8* x, const void* __restrict__ scale,
                                                           bf16x8* out, int64_t rows, int nvec, float hidden_f, float eps, GatherSrc g) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const bf16x8* xr = GATHER ? gather_row(g, x, row, nvec, lane == 0) : x + row * nvec;
  bf16x8 v[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int idx = lane + i * 64;
    if (idx < nvec && (!GATHER || xr != nullptr)) {
      v[i] = xr[idx];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[i][j] = static_cast<bf16>(0.f);
    }
  }
  if constexpr (GATHER) {
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int idx = lane + i * 64;
      if (idx < nvec) __builtin_nontemporal_store(v[i], g.x_out + row * nvec + idx);
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

// The scale vectors of 16-byte vector `vec` as they lie in memory (one 16-byte load for bf16, two for fp32), so that a
// kernel can request them before it needs them.
template <bool kScaleBf16>
struct ScaleRaw {
  bf16x8 b;
  f32x4 f0, f1;
  __device__ __forceinline__ void load(const void* scale, int vec) {
    if constexpr (kScaleBf16) {
      b = reinterpret_cast<const bf16x8*>(scale)[vec];
    } else {
      const f32x4* sp = reinterpret_cast<const f32x4*>(scale) + 2 * vec;
      f0 = sp[0];
      f1 = sp[1];
    }
  }
  __device__ __forceinline__ float at(int j) const {
    if constexpr (kScaleBf16) return static_cast<float>(b[j]);
    else return j < 4 ? f0[j] : f1[j - 4];
  }
};

// One 256-lane workgroup per row; VPT = 16-byte vectors per thread. The few-row case is all latency, so every load --
// the row and the scale -- goes out before anything waits (left at its use, behind the barrier, the scale's load would
// add a memory round trip to the chain: 2.36 -> 2.28 us at 8 rows, 2.43 -> 2.34 at 32, same box).
template <int VPT, bool kScaleBf16, bool GATHER>
__global__ __launch_bounds__(256) void rmsnorm_block_kernel(const bf16x8* x, const void* __restrict__ scale,
                                                            bf16x8* out, int nvec, float hidden_f, float eps, GatherSrc g) {
  __shared__ float part[4];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  ScaleRaw<kScaleBf16> sc[VPT];
  if constexpr (GATHER) {
    // the row's address hangs on the token id: the scale can travel meanwhile
#pragma unroll
    for (int i = 0; i < VPT; ++i) sc[i].load(scale, tid + i * 256 < nvec ? tid + i * 256 : 0);
  }
  const bf16x8* xr = GATHER ? gather_row(g, x, row, nvec, tid == 0) : x + row * nvec;
  bf16x8 v[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = tid + i * 256;
    if (idx < nvec && (!GATHER || xr != nullptr)) {
      v[i] = xr[idx];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[i][j] = static_cast<bf16>(0.f);
    }
  }
  if constexpr (!GATHER) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) sc[i].load(scale, tid + i * 256 < nvec ? tid + i * 256 : 0);
  }
  if constexpr (GATHER) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int idx = tid + i * 256;
      if (idx < nvec) __builtin_nontemporal_store(v[i], g.x_out + row * nvec + idx);
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
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = static_cast<bf16>(static_cast<float>(v[i][j]) * rinv * sc[i].at(j));
    if (idx < nvec) __builtin_nontemporal_store(o, orow + idx);   // streamed out: measured 5-18 % faster at prompt sizes, level at a few rows
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

template <bool kScaleBf16, bool GATHER>
static void launch_wave(int vpl, const bf16x8* x, const void* scale, bf16x8* out, int64_t rows, int nvec, float hidden_f, float eps,
                        const GatherSrc& g, hipStream_t st) {
  dim3 grid(static_cast<unsigned>((rows + 3) / 4)), block(256);
#define TLLM_CASE(V)                                                                                                             \
  case V:                                                                                                                        \
    hipLaunchKernelGGL((rmsnorm_wave_kernel<V, kScaleBf16, GATHER>), grid, block, 0, st, x, scale, out, rows, nvec, hidden_f, eps, g); \
    break;
  switch (vpl) {
    TLLM_CASE(1) TLLM_CASE(2) TLLM_CASE(3) TLLM_CASE(4) TLLM_CASE(5) TLLM_CASE(6) TLLM_CASE(7) TLLM_CASE(8)
    TLLM_CASE(9) TLLM_CASE(10) TLLM_CASE(11) TLLM_CASE(12) TLLM_CASE(13) TLLM_CASE(14) TLLM_CASE(15) TLLM_CASE(16)
  }
#undef TLLM_CASE
}

template <bool kScaleBf16, bool GATHER>
static void launch_block(int vpt, const bf16x8* x, const void* scale, bf16x8* out, int64_t rows, int nvec, float hidden_f, float eps,
                         const GatherSrc& g, hipStream_t st) {
  dim3 grid(static_cast<unsigned>(rows)), block(256);
#define TLLM_CASE(V)                                                                                                        \
  case V:                                                                                                                   \
    hipLaunchKernelGGL((rmsnorm_block_kernel<V, kScaleBf16, GATHER>), grid, block, 0, st, x, scale, out, nvec, hidden_f, eps, g); \
    break;
  switch (vpt) { TLLM_CASE(1) TLLM_CASE(2) TLLM_CASE(3) TLLM_CASE(4) }
#undef TLLM_CASE
}

}  // namespace tllm

using namespace tllm;

// The workgroup-per-row kernel is the faster one at every row count once a row keeps its 256 threads busy (hidden 2880:
// 2.65 against 4.2 us at 768 rows, 3.59 against 4.66 at 2048, 14.7 against 16.3 at 8192, 122 against 133 at 65536);
// rows narrower than 256 vectors go wavefront-per-row above this many rows.
static constexpr int64_t kBlockPerRowMaxRows = 512;

// Shared by the plain and the gather form: the two vector kernels by row count.
template <bool GATHER>
static bool launch_vector(const void* x, const void* scale, int scale_is_bf16, void* out, int64_t rows, int64_t hidden, float eps,
                          const GatherSrc& g, hipStream_t st) {
  const float hidden_f = static_cast<float>(hidden);  // divisor of the mean
  const int64_t nvec = hidden / 8;
  if ((rows <= kBlockPerRowMaxRows || nvec >= 256) && nvec <= 4 * 256) {
    const int vpt = static_cast<int>((nvec + 255) / 256);
    if (scale_is_bf16)
      launch_block<true, GATHER>(vpt, (const bf16x8*)x, scale, (bf16x8*)out, rows, (int)nvec, hidden_f, eps, g, st);
    else
      launch_block<false, GATHER>(vpt, (const bf16x8*)x, scale, (bf16x8*)out, rows, (int)nvec, hidden_f, eps, g, st);
    return true;
  }
  if (nvec <= 16 * 64) {
    const int vpl = static_cast<int>((nvec + 63) / 64);
    if (scale_is_bf16)
      launch_wave<true, GATHER>(vpl, (const bf16x8*)x, scale, (bf16x8*)out, rows, (int)nvec, hidden_f, eps, g, st);
    else
      launch_wave<false, GATHER>(vpl, (const bf16x8*)x, scale, (bf16x8*)out, rows, (int)nvec, hidden_f, eps, g, st);
    return true;
  }
  return false;
}

extern "C" int tllm_rmsnorm_bf16(const void* x, const void* scale, int scale_is_bf16, void* out, int64_t rows, int64_t hidden,
                                 float eps, void* stream) {
  TLLM_REQUIRE(rows >= 0 && hidden > 0, TLLM_E_ARG, "rmsnorm: rows %lld / hidden %lld invalid", (long long)rows, (long long)hidden);
  if (rows == 0) return TLLM_OK;
  TLLM_REQUIRE(x && scale && out, TLLM_E_ARG, "rmsnorm: null pointer");
  TLLM_REQUIRE(rows < (1ll << 31), TLLM_E_SHAPE, "rmsnorm: rows %lld too large", (long long)rows);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec_ok = hidden % 8 == 0 && aligned16(x) && aligned16(out) && aligned16(scale);
  if (!(vec_ok && launch_vector<false>(x, scale, scale_is_bf16, out, rows, hidden, eps, GatherSrc{}, st))) {
    hipLaunchKernelGGL(rmsnorm_scalar_kernel, dim3((unsigned)rows), dim3(256), 0, st, (const bf16*)x, scale, scale_is_bf16,
                       (bf16*)out, hidden, static_cast<float>(hidden), eps);
  }
  return check_launch("rmsnorm");
}

extern "C" int tllm_embed_rmsnorm_bf16(const void* table, const void* ids, int ids_is_i64, void* x_out, const void* scale,
                                       int scale_is_bf16, void* out, int64_t n_tokens, int64_t hidden, int64_t vocab, float eps,
                                       int* oob_flag, void* stream) {
  TLLM_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0, TLLM_E_ARG, "embed_rmsnorm: n_tokens %lld / hidden %lld / vocab %lld invalid",
               (long long)n_tokens, (long long)hidden, (long long)vocab);
  if (n_tokens == 0) return TLLM_OK;
  TLLM_REQUIRE(table && ids && x_out && scale && out, TLLM_E_ARG, "embed_rmsnorm: null pointer");
  TLLM_REQUIRE(n_tokens < (1ll << 31), TLLM_E_SHAPE, "embed_rmsnorm: n_tokens %lld too large", (long long)n_tokens);
  TLLM_REQUIRE(hidden % 8 == 0 && hidden <= 8192 && aligned16(table) && aligned16(x_out) && aligned16(out) && aligned16(scale), TLLM_E_SHAPE,
               "embed_rmsnorm: hidden %lld must be a multiple of 8 up to 8192 and all pointers 16-byte aligned (otherwise: the two "
               "separate calls)", (long long)hidden);
  TLLM_REQUIRE(x_out != out, TLLM_E_ARG, "embed_rmsnorm: x_out and out must be different buffers");
  GatherSrc g{ids, ids_is_i64, vocab, (bf16x8*)x_out, oob_flag};
  const bool ok = launch_vector<true>(table, scale, scale_is_bf16, out, n_tokens, hidden, eps, g, static_cast<hipStream_t>(stream));
  TLLM_REQUIRE(ok, TLLM_E_SHAPE, "embed_rmsnorm: hidden %lld not covered", (long long)hidden);
  return check_launch("embed_rmsnorm");
}
