// MXFP4 -> bf16 expansion of the checkpoint's MoE weights (weights.py:68-117): a block is 16 bytes = 32 fp4 (e2m1)
// values, low nibble first, sharing one e8m0 scale byte:  value = FP4[nibble] * 2^(scale - 127).
// The arithmetic follows the
// reference's torch.ldexp on a bf16 tensor: the product is formed in fp32 and rounded once to bf16 (exact for every
// scale a checkpoint holds; scale bytes >= 255 give inf / nan there and here).
#include "common.h"

namespace tllm {

__device__ __forceinline__ float fp4_value(unsigned nib) {
  // e2m1: 0, 0.5, 1, 1.5, 2, 3, 4, 6 with the sign in bit 3 (weights.py:11-14)
  const unsigned mag = nib & 7u;
  const float m = mag < 2u ? 0.5f * static_cast<float>(mag) : static_cast<float>(2u + (mag & 1u)) * static_cast<float>(1u << ((mag >> 1) - 1u)) * 0.5f;
  return (nib & 8u) ? -m : m;
}

__device__ __forceinline__ unsigned fp4_bf16_bits(unsigned nib) {
  // the bf16 encodings of the table above: 0x3F00 + (m << 6) for the normal values m >= 2, 0.5 = 0x3F00, 0 = 0
  const unsigned m = nib & 7u;
  const unsigned mag = m == 0u ? 0u : (m == 1u ? 0x3F00u : 0x3F00u + (m << 6));
  return mag | ((nib & 8u) << 12);
}

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;

// A lane expands one dword (4 bytes -> 8 values -> one 16-byte store), so that a wave's store covers 1 KB of
// consecutive output and its load 256 consecutive bytes; a work-group takes UNROLL * 256 dwords and each lane issues its
// UNROLL loads before the first conversion.
// Scaling by 2^e is an addition of e to the bf16 exponent field as long as every nonzero product stays a normal number
// (-125 <= e <= 125): a 256-entry LDS table maps a byte to its two unscaled bf16 values plus a mask that is 0 under a
// zero value, and one packed 16-bit add applies the exponent to both. Lanes whose scale lies outside that range (no
// checkpoint holds such scales) take the fp32 product instead, which covers denormals, inf and nan.
constexpr int MX_UNROLL = 8;   // 4 and 8 measure the same, 2 and 16 are 5-8 % slower

__global__ __launch_bounds__(256) void mxfp4_dequant_kernel(const unsigned* __restrict__ blocks, const unsigned char* __restrict__ scales,
                                                            u32x4* __restrict__ out, int64_t n_dwords) {
  __shared__ uint2 lut[256];
  {
    const unsigned b = threadIdx.x;
    const unsigned lo = fp4_bf16_bits(b & 15u), hi = fp4_bf16_bits(b >> 4);
    lut[b] = make_uint2(lo | (hi << 16), ((b & 7u) ? 0xffffu : 0u) | ((b & 0x70u) ? 0xffff0000u : 0u));
  }
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (256 * MX_UNROLL) + threadIdx.x;
  unsigned w[MX_UNROLL];
  int e[MX_UNROLL];
#pragma unroll
  for (int u = 0; u < MX_UNROLL; ++u) {
    const int64_t d = base + u * 256;
    w[u] = 0;
    e[u] = 0;
    if (d < n_dwords) {
      w[u] = __builtin_nontemporal_load(blocks + d);
      e[u] = static_cast<int>(scales[d >> 2]) - 127;      // four dwords per block
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < MX_UNROLL; ++u) {
    const int64_t d = base + u * 256;
    if (d >= n_dwords) break;
    u32x4 o;
    if (e[u] >= -125 && e[u] <= 125) {
      const unsigned es = static_cast<unsigned>(e[u] << 7) & 0xffffu;
      const unsigned esp = es | (es << 16);
#pragma unroll
      for (int k = 0; k < 4; ++k) {              // byte k gives out[2k] (low nibble) and out[2k+1] (high nibble)
        const uint2 t = lut[(w[u] >> (8 * k)) & 0xffu];
        o[k] = __builtin_bit_cast(unsigned, __builtin_bit_cast(u16x2, t.x) + __builtin_bit_cast(u16x2, t.y & esp));
      }
    } else {
      // 2^e as torch.pow(2.0, e) yields it in fp32: denormal below -126, inf above 127
      const float p = e[u] > 127 ? __builtin_inff() : ldexpf(1.0f, e[u]);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const unsigned byte = (w[u] >> (8 * k)) & 0xffu;
        const bf16 lo = static_cast<bf16>(fp4_value(byte & 15u) * p), hi = static_cast<bf16>(fp4_value(byte >> 4) * p);
        o[k] = static_cast<unsigned>(__builtin_bit_cast(unsigned short, lo)) | (static_cast<unsigned>(__builtin_bit_cast(unsigned short, hi)) << 16);
      }
    }
    __builtin_nontemporal_store(o, out + d);
  }
}

}  // namespace tllm

using namespace tllm;

extern "C" int tllm_mxfp4_dequant_bf16(const void* blocks, const void* scales, void* out, int64_t n_blocks, void* stream) {
  TLLM_REQUIRE(n_blocks >= 0, TLLM_E_ARG, "mxfp4_dequant: n_blocks %lld", (long long)n_blocks);
  if (n_blocks == 0) return TLLM_OK;
  TLLM_REQUIRE(blocks && scales && out, TLLM_E_ARG, "mxfp4_dequant: null pointer");
  TLLM_REQUIRE(aligned16(blocks) && aligned16(out), TLLM_E_ALIGN, "mxfp4_dequant: blocks and out must be 16-byte aligned");
  const int64_t n_dwords = n_blocks * 4;
  const int64_t wgs = (n_dwords + 256 * MX_UNROLL - 1) / (256 * MX_UNROLL);
  TLLM_REQUIRE(wgs < (1ll << 31), TLLM_E_SHAPE, "mxfp4_dequant: %lld blocks are too many for one launch", (long long)n_blocks);
  hipLaunchKernelGGL(mxfp4_dequant_kernel, dim3((unsigned)wgs), dim3(256), 0, static_cast<hipStream_t>(stream), (const unsigned*)blocks,
                     (const unsigned char*)scales, (u32x4*)out, n_dwords);
  return check_launch("mxfp4_dequant");
}
