// Shared device/host helpers for the gfx950 layer kernels.
#pragma once
#include <type_traits>

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tllm_hip.h"

namespace tllm {

typedef __bf16 bf16;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;   // 16 bytes
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;   // 8 bytes
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;   // 4 bytes
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

constexpr int kWave = 64;

// ---- host side error plumbing (abi.hip owns the storage) -------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);

#define TLLM_REQUIRE(cond, code, ...)      \
  do {                                     \
    if (!(cond)) {                         \
      ::tllm::set_error(__VA_ARGS__);      \
      return (code);                       \
    }                                      \
  } while (0)

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- device helpers --------------------------------------------------------
// Sum over the 64 lanes, the same value in every lane. Inside a row of 16 lanes through DPP operands (lane ^ 1, lane ^ 2,
// the mirrored half row, the mirrored row: four adds, no LDS crossbar), across the four rows through scalar registers.
// (Six __shfl_xor steps are six ds_bpermute round trips, ~0.2 us on the critical path of a few-row kernel.)
__device__ __forceinline__ float wave_sum(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, true));
  };
  v += dpp(v, std::integral_constant<int, 0xB1>{});        // quad_perm [1, 0, 3, 2]
  v += dpp(v, std::integral_constant<int, 0x4E>{});        // quad_perm [2, 3, 0, 1]
  v += dpp(v, std::integral_constant<int, 0x141>{});       // row_half_mirror
  v += dpp(v, std::integral_constant<int, 0x140>{});       // row_mirror
  const int b = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return (r0 + r1) + (r2 + r3);
}

// Maximum over the 64 lanes, the same value in every lane; the same route as wave_sum.
__device__ __forceinline__ float wave_max(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, true));
  };
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0xB1>{}));
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x4E>{}));
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x141>{}));
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x140>{}));
  const int b = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// The lane's own value and that of lane ^ 16 (lane ^ 32), in some order -- enough for a sum or a maximum. gfx950's row
// and half-wavefront swaps are vector-ALU instructions; __shfl_xor goes through the LDS crossbar and waits for it.
// (The two results are taken out of the returned pair as one 64-bit value: element access on it reads element 0 twice
// with this compiler.)
__device__ __forceinline__ void lane_xor16_pair(float x, float* a, float* b) {
  const int xi = __builtin_bit_cast(int, x);
  const unsigned long long u = __builtin_bit_cast(unsigned long long, __builtin_amdgcn_permlane16_swap(xi, xi, false, false));
  *a = __uint_as_float(static_cast<unsigned>(u));
  *b = __uint_as_float(static_cast<unsigned>(u >> 32));
}
__device__ __forceinline__ void lane_xor32_pair(float x, float* a, float* b) {
  const int xi = __builtin_bit_cast(int, x);
  const unsigned long long u = __builtin_bit_cast(unsigned long long, __builtin_amdgcn_permlane32_swap(xi, xi, false, false));
  *a = __uint_as_float(static_cast<unsigned>(u));
  *b = __uint_as_float(static_cast<unsigned>(u >> 32));
}
// x + (x of lane ^ 8), x + (x of lane ^ 16) + ..., as sums and maxima over the lanes that differ in the given bits
__device__ __forceinline__ float lane_xor8_value(float x) {   // row_ror:8 inside a row of 16 lanes
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128, 0xf, 0xf, true));
}
__device__ __forceinline__ float sum_over_lane_bits_16_32(float x) {
  float a, b;
  lane_xor16_pair(x, &a, &b);
  x = a + b;
  lane_xor32_pair(x, &a, &b);
  return a + b;
}
__device__ __forceinline__ float max_over_lane_bits_16_32(float x) {
  float a, b;
  lane_xor16_pair(x, &a, &b);
  x = fmaxf(a, b);
  lane_xor32_pair(x, &a, &b);
  return fmaxf(a, b);
}

// Kernel-argument copy of the rotary source (TllmRope with the YaRN block by value).
struct RopeArgs {
  const float* cos_table;
  const float* sin_table;
  int64_t table_row_stride;
  const int64_t* positions;
  const int64_t* offset;
  int64_t tokens_per_batch;
  int64_t max_ctx;
  float concentration;
  int n_freq;
  int use_yarn;
};

struct YarnFreqs {
  float v[TLLM_MAX_ROPE_FREQS];
};

// Unwrapped position of a row: only loads and an add, so it can be issued early.
__device__ __forceinline__ int64_t rope_position_raw(const RopeArgs& r, int64_t row) {
  if (r.positions) return r.positions[row];
  int64_t p = row % r.tokens_per_batch;
  if (r.offset) p += r.offset[0];
  return p;
}

// Wrap into [0, max_ctx). The common case is already in range and skips the 64-bit division.
__device__ __forceinline__ int64_t rope_wrap(int64_t p, int64_t max_ctx) {
  if (static_cast<uint64_t>(p) >= static_cast<uint64_t>(max_ctx)) {
    p %= max_ctx;
    if (p < 0) p += max_ctx;
  }
  return p;
}

__device__ __forceinline__ int64_t rope_position(const RopeArgs& r, int64_t row) {
  return rope_wrap(rope_position_raw(r, row), r.max_ctx);
}

// sin and cos of an fp32 angle up to ~3e7 rad, to ~1e-7 absolute (about one ulp of 1.0).
// Three-constant Cody-Waite reduction by pi/2 carried in FMAs (the products are exact inside the
// FMA, so the only rounding is that of the reduced argument), then the classic single-precision
// minimax polynomials on [-pi/4, pi/4] and a quadrant fix-up. A dozen registers and ~25
// instructions; the library routine's Payne-Hanek path costs five times the registers, which
// would cap the occupancy of every kernel that rotates.
__device__ __forceinline__ void sincos_reduced(float x, float* s, float* c) {
  const float kf = rintf(x * 0.636619772367581343f);
  float r = fmaf(-kf, 1.57079637050628662109375f, x);
  r = fmaf(-kf, -4.37113882867379e-8f, r);
  r = fmaf(-kf, -1.7151245e-15f, r);
  const float z = r * r;
  float sp = fmaf(z, -1.9515295891e-4f, 8.3321608736e-3f);
  sp = fmaf(z, sp, -1.6666654611e-1f);
  const float sv = fmaf(r * z, sp, r);
  float cp = fmaf(z, 2.443315711809948e-5f, -1.388731625493765e-3f);
  cp = fmaf(z, cp, 4.166664568298827e-2f);
  const float cv = fmaf(z * z, cp, fmaf(z, -0.5f, 1.0f));
  const int q = static_cast<int>(kf);
  const float ss = (q & 1) ? cv : sv;
  const float cc = (q & 1) ? sv : cv;
  *s = (q & 2) ? -ss : ss;
  *c = ((q + 1) & 2) ? -cc : cc;
}

// cos/sin of the rotary angle for (position, frequency), scaled by the concentration. The angle is
// the single fp32 product float(pos) * inv_freq, exactly as the reference's table construction forms
// it (angles reach 1.3e5 rad at the end of the context: the fast hardware sin/cos are useless here).
__device__ __forceinline__ void yarn_cos_sin(int64_t pos, float inv_freq, float concentration, float* c, float* s) {
  const float angle = __fmul_rn(static_cast<float>(pos), inv_freq);
  float sv, cv;
  sincos_reduced(angle, &sv, &cv);
  *c = cv * concentration;
  *s = sv * concentration;
}

__device__ __forceinline__ void rope_cos_sin(const RopeArgs& r, const YarnFreqs& f, int64_t pos, int i, float* c, float* s) {
  if (r.use_yarn) {
    yarn_cos_sin(pos, f.v[i], r.concentration, c, s);
  } else {
    *c = r.cos_table[pos * r.table_row_stride + i];
    *s = r.sin_table[pos * r.table_row_stride + i];
  }
}

// Eight fp8 (OCP e4m3) values in two dwords -> eight bf16, exactly (bf16 holds every e4m3 value): gfx950's packed
// conversion takes two fp8 of one 16-bit half to two bf16, times a scale of 1 -- four instructions for the eight values
// (through fp32 pairs and a byte permute it was eight). The results are taken as whole registers.
__device__ __forceinline__ bf16x8 fp8x8_to_bf16x8(unsigned lo, unsigned hi) {
  typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;
  u32x4 o;
  o[0] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false));
  o[1] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true));
  o[2] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false));
  o[3] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true));
  return __builtin_bit_cast(bf16x8, o);
}

// Host: validate a TllmRope and flatten it into kernel arguments.
int make_rope_args(const TllmRope* rope, int head_dim, RopeArgs* out, YarnFreqs* freqs);

}  // namespace tllm
