// Decode-size attention out-projection + bias + residual for in_dim == 4096 and 9..32 activation rows per workgroup
// (bf16 or fp8 weight): the companion of out_decode_r8.hip for the larger decode batches
//   out[r, n] = sum_k x[r, k] * W[n, k] + b[n] + res[r, n]        (out_residual_decode_forward, triton_kernels.py:1470-1517)
//
// Same skeleton: one workgroup per twelve output features (gpt-oss: 240 workgroups, one per CU), one 16-row MFMA tile
// of weight rows on M against two column blocks of 16 activation rows on N (v_mfma_f32_16x16x32_bf16), every operand
// loaded from global memory straight into LDS with the XOR swizzle chosen on the global side, fragments read back
// once, partial tiles reduced in a fixed order by epilogue wavefronts that fetched bias and residual meanwhile.
// What differs: 32 activation rows are 256 KB per workgroup, more than the LDS holds, so the activations arrive in
// phases. Four streaming wavefronts, each with 1024 of the 4096 K: 32 k32 steps in eight phases of four; in phase p
// the four together read 1024 contiguous bytes of every row (wavefront kq the 256 bytes at p * 1024 + kq * 256). A
// phase of a wavefront is 8 KB of activations (32 rows x 256 bytes) and 3 KB of weight. The weight -- the operand that
// comes from HBM -- is requested whole at the start, every phase into a place of its own (24 KB per wavefront); the
// activations, which come from the L2s, pass a ring of two 8 KB regions, a region being refilled with the phase two
// further on as soon as its fragments are in registers. A CU returns loads in the order it took them, so the third
// activation phase arrives behind the last of the weight and the rest follow one L2 round trip per pair; with the
// weight in a ring as well (three phases of both operands resident) its requests trickle out behind the MFMAs and
// the launch takes 8.5 us at 32 rows instead of 8.1 (five or six weight phases resident: 8.35 / 8.25; a third
// activation region ahead of the weight's later phases: 6.80 against 6.73 us with the fp8 weight). Two epilogue
// wavefronts, one per column block.
// W8: fp8 (OCP e4m3) weight with one fp32 scale per output row (the reference's ATTN_FP8 option,
// triton_kernels.py:1385-1408): a weight row of a phase is 128 bytes (two loads of eight rows), fragments are widened
// to bf16 (exact) between the LDS read and the MFMA, the row scale multiplies the finished sum.
// More than 32 rows: a workgroup takes up to four chunks of 32 rows one after the other against the same resident
// weight (only the first chunk requests it), so the weight is read once for up to 128 rows; between chunks the
// partial tiles pass through the first activation region behind two barriers (33 rows 13.3 -> 10.5 us, 64 rows
// 14.0 -> 11.2, where every chunk was a workgroup of its own with its own pass over the weight).
// XB = four-row activation blocks fetched per phase (rows past a chunk's last one repeat it; with fewer than 29 rows
// the blocks that would hold no real row are not fetched at all).
#include "out_common.h"

namespace tllm {

namespace r32o {
constexpr int XR = 32;            // activation rows per workgroup
constexpr int NS = 4;             // streaming wavefronts = K slices
constexpr int NE = 2;             // epilogue wavefronts = column blocks
constexpr int RW = 12;            // weight rows (output features) per workgroup
constexpr int NPH = 8;            // phases of four k32 steps
constexpr int WRING = NPH;        // every phase of the weight is requested at once and has a place of its own
constexpr int XPH = 8 * 1024;     // activations of one phase: 32 rows x four k32 steps
constexpr int WAVE_LDS = 40 * 1024;   // a wavefront's activation ring, then its weight: 2 x 8 + 8 x 3 KB
static_assert(NS * WAVE_LDS <= 160 * 1024, "the rings fit the LDS");

// Load instructions that may still be outstanding when phase p is multiplied: those requested after the phase's own
// last load. The order of requests: x(0) W(0) x(1) W(1) ... while both rings fill, then behind each phase p
// x(p + xring) (and W(p + WRING), if the weight had a ring shorter than its phases).
constexpr int younger_than_phase(int p, int xb, int lw, int xring) {
  int count = 0, last = 0;
  const int pro = xring > WRING ? xring : WRING;
  for (int i = 0; i < pro; ++i) {
    if (i < xring && i < NPH) { count += xb; if (i == p) last = count; }
    if (i < WRING && i < NPH) { count += lw; if (i == p) last = count; }
  }
  for (int q = 0; q < p; ++q) {
    if (q + xring < NPH) { count += xb; if (q + xring == p) last = count; }
    if (q + WRING < NPH) { count += lw; if (q + WRING == p) last = count; }
  }
  return count - last;
}
static_assert(NPH == 8, "the wait of each phase is spelled out below");
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "s_waitcnt vmcnt takes six bits");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
}  // namespace r32o

template <int XB, bool W8>
__global__ __launch_bounds__(384) void out_decode_r32_kernel(OutArgs a, int vec8, int cpw) {
  using namespace r32o;
  constexpr int LW = W8 ? 2 : 3;                            // weight load instructions per phase
  constexpr int XRING = 2;                                  // phases of activations resident per wavefront
  constexpr int WPH = 3 * 1024;                             // weight of one phase: 12 rows x four k32 steps (fp8: 2 KB of it)
  static_assert(XRING * XPH + WRING * WPH <= WAVE_LDS, "a wavefront's rings fit its share of the LDS");
  __shared__ __align__(1024) unsigned char ring[NS * WAVE_LDS];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * RW;
  // A workgroup takes up to `cpw` consecutive chunks of 32 rows, one after the other, against the weight it requested
  // for the first: every phase of the weight has a place of its own in LDS and stays there.
  const int64_t chunk0 = static_cast<int64_t>(blockIdx.y) * cpw;
  const int64_t chunks_left = (a.rows + XR - 1) / XR - chunk0;
  const int my_chunks = static_cast<int>(chunks_left < cpw ? chunks_left : cpw);   // >= 1 by the grid

  if (wave >= NS) {
    // ======================================================================= epilogue wavefront of column block cb
    const int cb = wave - NS;
    const int en = 16 * cb + (lane & 15), eg = lane >> 4;   // activation row of the chunk, quad of features
    for (int c = 0; c < my_chunks; ++c) {
    const int64_t row0 = (chunk0 + c) * XR;
    const int nvalid = static_cast<int>(a.rows - row0 < XR ? a.rows - row0 : XR);
    const bool evalid = eg < 3 && en < nvalid;
    const int efeat = n0 + (evalid ? 4 * eg : 0);
    const int64_t erow = row0 + (evalid ? en : 0);
    // absent operands read a valid dummy address instead of being predicated
    const bf16* bias_ptr = a.bias ? a.bias + efeat : a.x;
    const bf16* res_ptr = a.res ? a.res + erow * a.res_rs + efeat : a.x;
    bf16* out = a.out + erow * a.out_rs + efeat;
    float bv[4], rv[4];
    if (vec8) {
      const bf16x4 b4 = *reinterpret_cast<const bf16x4*>(bias_ptr);
      const bf16x4 r4 = *reinterpret_cast<const bf16x4*>(res_ptr);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bv[i] = static_cast<float>(b4[i]);
        rv[i] = static_cast<float>(r4[i]);
      }
    } else {
      bf16 b1[4], r1[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        b1[i] = bias_ptr[i];
        r1[i] = res_ptr[i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bv[i] = static_cast<float>(b1[i]);
        rv[i] = static_cast<float>(r1[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (!a.bias) bv[i] = 0.f;
      if (!a.res) rv[i] = 0.f;
    }
    float ws[4] = {1.f, 1.f, 1.f, 1.f};                    // W8: the row scales of the lane's four features
    if constexpr (W8) {
#pragma unroll
      for (int i = 0; i < 4; ++i) ws[i] = a.w_scale[efeat + i];
      asm volatile("" : "+v"(ws[0]), "+v"(ws[1]), "+v"(ws[2]), "+v"(ws[3]));
    }
    unsigned red_o = static_cast<unsigned>(cb * 1024 + lane * 16);
    // the wavefronts run alone from the barrier to the stores: everything that does not need the sums exists before it
    asm volatile("" : "+v"(bv[0]), "+v"(bv[1]), "+v"(bv[2]), "+v"(bv[3]), "+v"(rv[0]), "+v"(rv[1]), "+v"(rv[2]), "+v"(rv[3]), "+v"(out), "+v"(red_o));
    __syncthreads();                                        // partial tiles are in LDS
    f32x4 t[NS];
#pragma unroll
    for (int w = 0; w < NS; ++w) t[w] = *reinterpret_cast<const f32x4*>(ring + w * WAVE_LDS + red_o);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();                                        // ... and read: the next chunk's activations may land there
    f32x4 acc = t[0];
#pragma unroll
    for (int w = 1; w < NS; ++w) {                          // fixed order: the result does not depend on timing
      acc[0] += t[w][0];
      acc[1] += t[w][1];
      acc[2] += t[w][2];
      acc[3] += t[w][3];
    }
    if (evalid) {
      bf16x4 o;                                             // features efeat .. efeat + 3 of row en
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = static_cast<bf16>(acc[i] * ws[i] + bv[i] + rv[i]);
      if (vec8) {
        *reinterpret_cast<bf16x4*>(out) = o;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = o[i];
      }
    }
    }
    return;
  }

  // ========================================================================= streaming wavefront of K slice `kq`
  const int kq = wave;
  const int m = lane & 15, g = lane >> 4;
  unsigned char* myring = ring + wave * WAVE_LDS;

  // lane -> (row of a 4-row block, position): it fetches chunk position ^ (row & 15) of that row's 256 bytes, so that
  // the 16 rows a fragment read touches lie in 16 different bank groups
  unsigned xoff[XB], goff[LW];
  // (W8: a weight row of a phase is 128 bytes = 8 chunks and a load covers eight rows: lane -> row 8 j + lane / 8,
  // position lane % 8, chunk position ^ (row & 7); rows 12..15 of the second load repeat row 11, unread)
#pragma unroll
  for (int j = 0; j < LW; ++j) {
    if constexpr (W8) {
      int r = 8 * j + (lane >> 3);
      r = r < RW ? r : RW - 1;
      goff[j] = static_cast<unsigned>(n0 + r) * 4096u + kq * 128u + (((lane & 7) ^ (r & 7)) << 4);
    } else {
      const int r = 4 * j + (lane >> 4);
      goff[j] = static_cast<unsigned>(n0 + r) * 8192u + kq * 256u + (((lane & 15) ^ r) << 4);
    }
  }
  const unsigned char* xbase = nullptr;                     // the chunk's first row (set per chunk below)
  const unsigned char* wbase = reinterpret_cast<const unsigned char*>(a.W);
  auto lds_addr = [](const void* p) { return static_cast<unsigned>(reinterpret_cast<uintptr_t>(p)); };
  auto x_region = [&](int p) { return myring + (p % XRING) * XPH; };
  auto w_region = [&](int p) { return myring + XRING * XPH + (p % WRING) * WPH; };
  auto issue_x = [&](int p) {
    const unsigned char* xb = xbase + p * 1024;
#pragma unroll
    for (int j = 0; j < XB; ++j) {
      const unsigned dst = lds_addr(x_region(p) + j * 1024);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(xoff[j]), "s"(xb) : "memory", "m0");
    }
  };
  auto issue_w = [&](int p) {
    const unsigned char* wb = wbase + p * (W8 ? 512 : 1024);
#pragma unroll
    for (int j = 0; j < LW; ++j) {
      const unsigned dst = lds_addr(w_region(p) + j * 1024);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst), "v"(goff[j]), "s"(wb) : "memory", "m0");
    }
  };
  const int arow = m < RW ? m : m - RW;                     // tile rows past the twelfth re-read a real one (their sums are dropped)
  const unsigned a_o = arow * (W8 ? 128 : 256);
  // W8: the lane's eight fp8 of step st are bytes 32 st + 8 g of the 128-byte row: half g & 1 of chunk 2 st + g / 2,
  // which sits at position chunk ^ (row & 7)
  auto w8frag = [&](const unsigned char* reg, int st) {
    typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2;
    const u32x2 raw = *reinterpret_cast<const u32x2*>(reg + a_o + (((2 * st + (g >> 1)) ^ (arow & 7)) << 4) + (g & 1) * 8);
    return fp8x8_to_bf16x8(raw[0], raw[1]);
  };
  const unsigned b0_o = m * 256, b1_o = (16 + m) * 256;
  for (int c = 0; c < my_chunks; ++c) {
  const bool first = c == 0;                                // the weight is requested with the first chunk only
  {
    const int64_t row0 = (chunk0 + c) * XR;
    const int nvalid = static_cast<int>(a.rows - row0 < XR ? a.rows - row0 : XR);
#pragma unroll
    for (int j = 0; j < XB; ++j) {
      const int r = 4 * j + (lane >> 4);
      const int src = r < nvalid ? r : nvalid - 1;          // row inside the chunk's 32 (the base points at its first row)
      xoff[j] = static_cast<unsigned>(src * 8192 + kq * 256 + (((lane & 15) ^ (r & 15)) << 4));
    }
    xbase = reinterpret_cast<const unsigned char*>(a.x) + row0 * 8192;
  }
#pragma unroll
  for (int p = 0; p < (XRING > WRING ? XRING : WRING); ++p) {
    if (p < XRING && p < NPH) issue_x(p);
    if (first && p < WRING && p < NPH) issue_w(p);
  }
  f32x4 acc[2];                                             // [column block]
  acc[0] = f32x4{0.f, 0.f, 0.f, 0.f};
  acc[1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int p = 0; p < NPH; ++p) {
    // phase p has landed when only the loads requested after its own are outstanding (a later chunk requests no weight)
    if (first) {
      switch (p) {                                          // (p is a constant of the unrolled loop; an asm operand must be one by the language's rules)
        case 0: wait_vmcnt<younger_than_phase(0, XB, LW, XRING)>(); break;
        case 1: wait_vmcnt<younger_than_phase(1, XB, LW, XRING)>(); break;
        case 2: wait_vmcnt<younger_than_phase(2, XB, LW, XRING)>(); break;
        case 3: wait_vmcnt<younger_than_phase(3, XB, LW, XRING)>(); break;
        case 4: wait_vmcnt<younger_than_phase(4, XB, LW, XRING)>(); break;
        case 5: wait_vmcnt<younger_than_phase(5, XB, LW, XRING)>(); break;
        case 6: wait_vmcnt<younger_than_phase(6, XB, LW, XRING)>(); break;
        default: wait_vmcnt<younger_than_phase(7, XB, LW, XRING)>(); break;
      }
    } else {
      switch (p) {
        case 0: wait_vmcnt<younger_than_phase(0, XB, 0, XRING)>(); break;
        case 1: wait_vmcnt<younger_than_phase(1, XB, 0, XRING)>(); break;
        case 2: wait_vmcnt<younger_than_phase(2, XB, 0, XRING)>(); break;
        case 3: wait_vmcnt<younger_than_phase(3, XB, 0, XRING)>(); break;
        case 4: wait_vmcnt<younger_than_phase(4, XB, 0, XRING)>(); break;
        case 5: wait_vmcnt<younger_than_phase(5, XB, 0, XRING)>(); break;
        case 6: wait_vmcnt<younger_than_phase(6, XB, 0, XRING)>(); break;
        default: wait_vmcnt<younger_than_phase(7, XB, 0, XRING)>(); break;
      }
    }
    const unsigned char* reg = x_region(p);
    const unsigned char* wreg = w_region(p);
    bf16x8 fa[4], fb0[4], fb1[4];
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      if constexpr (W8) fa[st] = w8frag(wreg, st);
      else fa[st] = *reinterpret_cast<const bf16x8*>(wreg + a_o + (((4 * st + g) ^ arow) << 4));
      fb0[st] = *reinterpret_cast<const bf16x8*>(reg + b0_o + (((4 * st + g) ^ m) << 4));
      if constexpr (XB > 4) fb1[st] = *reinterpret_cast<const bf16x8*>(reg + b1_o + (((4 * st + g) ^ m) << 4));
    }
    if (p + XRING < NPH || p + WRING < NPH) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // the regions' fragments are in registers: they may be refilled
      if (p + XRING < NPH) issue_x(p + XRING);
      if (first && p + WRING < NPH) issue_w(p + WRING);
    }
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[st], fb0[st], acc[0], 0, 0, 0);
      if constexpr (XB > 4) acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[st], fb1[st], acc[1], 0, 0, 0);
    }
  }

  // ---- partial tiles -> LDS (the wavefront's own activation region 0: every region's fragments have been read by now)
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  *reinterpret_cast<f32x4*>(myring + lane * 16) = acc[0];
  *reinterpret_cast<f32x4*>(myring + 1024 + lane * 16) = acc[1];
  __syncthreads();                                          // the epilogue wavefronts take them ...
  __syncthreads();                                          // ... and have them: the region is the next chunk's again
  }
}

// in_dim 4096, out_dim % 12 == 0, bf16 weight or (a.w_scale != null) fp8; grid = (out_dim / 12, ceil(rows / 32))
void launch_out_decode_r32(dim3 grid, hipStream_t st, const OutArgs& a) {
  auto al8 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 8 == 0; };
  const int vec8 = al8(a.out) && a.out_rs % 4 == 0 && (a.res == nullptr || (al8(a.res) && a.res_rs % 4 == 0)) && (a.bias == nullptr || al8(a.bias));
  const int rows = static_cast<int>(a.rows < 32 ? a.rows : 32);          // of the fullest chunk
  // up to four chunks of 32 rows per workgroup: the weight is then read once for up to 128 rows
  const int cpw = grid.y < 4 ? static_cast<int>(grid.y) : 4;
  const dim3 g2(grid.x, (grid.y + cpw - 1) / cpw);
#define TLLM_OUT32(XB)                                                                                        \
  do {                                                                                                        \
    if (a.w_scale) hipLaunchKernelGGL((out_decode_r32_kernel<XB, true>), g2, dim3(384), 0, st, a, vec8, cpw);   \
    else hipLaunchKernelGGL((out_decode_r32_kernel<XB, false>), g2, dim3(384), 0, st, a, vec8, cpw);            \
  } while (0)
  switch ((rows + 3) / 4) {
    case 1: TLLM_OUT32(1); break;
    case 2: TLLM_OUT32(2); break;
    case 3: TLLM_OUT32(3); break;
    case 4: TLLM_OUT32(4); break;
    case 5: TLLM_OUT32(5); break;
    case 6: TLLM_OUT32(6); break;
    case 7: TLLM_OUT32(7); break;
    default: TLLM_OUT32(8); break;
  }
#undef TLLM_OUT32
}

}  // namespace tllm
