// Decode-size attention out-projection + bias + residual for in_dim == 4096 and up to 8 activation rows (bf16 or fp8 weight):
//   out[r, n] = sum_k x[r, k] * W[n, k] + b[n] + res[r, n]        (out_residual_decode_forward, triton_kernels.py:1470-1517)
// in the weight-streaming form of qkv_decode_r8.hip:
//   * one workgroup per twelve output features (gpt-oss: 240 workgroups, one per CU -- it needs most of a CU's LDS),
//     one 16-row MFMA tile (v_mfma_f32_16x16x32_bf16: weight rows on M, activation rows on N);
//   * eight streaming wavefronts, each with 512 of the 4096 K: sixteen k32 steps in four phases of four. K is dealt by
//     phase: in phase p the eight wavefronts together read 2048 contiguous bytes of every weight row (wavefront kq the
//     256 bytes at p * 2048 + kq * 256), so what a CU asks of memory at any one time is contiguous;
//   * every operand goes from global memory straight into LDS (global_load_lds_dwordx4: a load's 64 x 16 bytes land at
//     consecutive LDS addresses, which global chunk a lane fetches is free, and that freedom carries the XOR swizzle
//     chunk ^ row that makes the 16-row fragment reads conflict-free). A wavefront loads its own slice of the
//     activations (8 rows x 1 KB) and of the twelve weight rows (3 KB per phase): phases 0-2 into a ring of three
//     regions, phase 3 into the activation blocks, which are free once the activation fragments are in registers --
//     so every load is requested at once, none waits for an MFMA, and no wavefront waits for another one's loads.
//     s_waitcnt vmcnt is spelled by hand (the compiler does not see these loads); the streaming wavefronts issue no
//     other vector load;
//   * a ninth wavefront loads bias and residual while the stream runs, then adds the eight partial tiles in a fixed
//     order and stores four adjacent features of a row per lane (8-byte stores where the alignment allows).
// `out` may be the residual buffer itself: an element is read and written by the same lane.
// W8: fp8 (OCP e4m3) weight with one fp32 scale per output row (the reference's ATTN_FP8 option,
// triton_kernels.py:1385-1408): a wavefront's 512 bytes of a row arrive in two phases of eight k32 steps (256-byte
// pieces again, the same LDS layout), fragments are widened to bf16 (exact) between the LDS read and the MFMA, the row
// scale multiplies the finished sum.
#include "out_common.h"

namespace tllm {

namespace r8o {
constexpr int XR = 8;             // activation rows per workgroup
constexpr int NS = 8;             // streaming wavefronts
constexpr int RW = 12;            // weight rows (output features) per workgroup
constexpr int RING = 3;           // resident phases per wavefront
constexpr int REGION = RW * 256;  // one phase: twelve weight rows x four k32 steps
constexpr int XBLOCK = 1024;      // one activation row of a slice: 64 chunks of 16 bytes
}  // namespace r8o

template <bool W8>
__global__ __launch_bounds__(576) void out_decode_r8_kernel(OutArgs a, int vec8) {
  using namespace r8o;
  constexpr int NPH = W8 ? 2 : 4;                           // phases of PSTEPS k32 steps
  constexpr int PSTEPS = 16 / NPH;
  constexpr int RPH = W8 ? 2 : RING;                        // phases that land in the ring (the last bf16 phase lands in the activation blocks)
  constexpr int WPITCH = W8 ? 4096 : 8192;                  // bytes per weight row
  __shared__ __align__(1024) unsigned char xw[NS * XR * XBLOCK];
  __shared__ __align__(1024) unsigned char ring[NS * RING * REGION];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * RW;
  const int nvalid = static_cast<int>(a.rows < XR ? a.rows : XR);

  if (wave >= NS) {
    // ======================================================================= epilogue wavefront
    const int en = lane & 15, eg = lane >> 4;               // activation row, quad of features
    const bool evalid = eg < 3 && en < nvalid;
    const int efeat = n0 + (evalid ? 4 * eg : 0);
    const int64_t erow = evalid ? en : 0;
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
    unsigned red_o = static_cast<unsigned>(REGION + lane * 16);
    // one wavefront runs alone from the barrier to the stores: everything that does not need the sums exists before it
    asm volatile("" : "+v"(bv[0]), "+v"(bv[1]), "+v"(bv[2]), "+v"(bv[3]), "+v"(rv[0]), "+v"(rv[1]), "+v"(rv[2]), "+v"(rv[3]), "+v"(out), "+v"(red_o));
    __syncthreads();                                        // partial tiles are in LDS
    f32x4 t[NS];
#pragma unroll
    for (int w = 0; w < NS; ++w) t[w] = *reinterpret_cast<const f32x4*>(ring + w * (RING * REGION) + red_o);
    f32x4 acc = t[0];
#pragma unroll
    for (int w = 1; w < NS; ++w) {                          // fixed order: the result does not depend on timing
      acc[0] += t[w][0];
      acc[1] += t[w][1];
      acc[2] += t[w][2];
      acc[3] += t[w][3];
    }
    if (!evalid) return;
    bf16x4 o;                                               // features efeat .. efeat + 3 of row en
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = static_cast<bf16>(acc[i] * ws[i] + bv[i] + rv[i]);
    if (vec8) {
      *reinterpret_cast<bf16x4*>(out) = o;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = o[i];
    }
    return;
  }

  // ========================================================================= streaming wavefront kq
  const int kq = wave;
  const int m = lane & 15, g = lane >> 4, m1 = m & 7;
  unsigned char* myx = xw + wave * (XR * XBLOCK);
  unsigned char* myring = ring + wave * (RING * REGION);
  // byte offset inside a bf16 row of this wavefront's 16-byte chunk c (0..63): phase c / 16, chunk c % 16 of its 256 bytes
  // (of an activation row; with the fp8 weight a phase is eight steps: phase c / 32, chunk c % 32 of its 512 bytes)
  auto kb = [&](int c) { return W8 ? (c >> 5) * 4096 + kq * 512 + (c & 31) * 16 : (c >> 4) * 2048 + kq * 256 + (c & 15) * 16; };

  // activations: row n of the slice -> 1 KB block n; lane i fetches chunk i ^ 2n, the swizzle that spreads the eight
  // rows of a fragment read over the banks
  unsigned xoff[XR];
#pragma unroll
  for (int n = 0; n < XR; ++n) {
    const int src = n < nvalid ? n : nvalid - 1;
    xoff[n] = static_cast<unsigned>(src * 8192 + kb(lane ^ (2 * n)));
  }
  // weight: lane -> (row 4 j + lane / 16, position lane % 16): it fetches chunk position ^ row of that row
  unsigned goff[3];
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    const int r = 4 * j + (lane >> 4);
    const int cc = (lane & 15) ^ r;
    goff[j] = static_cast<unsigned>(n0 + r) * static_cast<unsigned>(WPITCH) + kq * 256u + cc * 16u;
  }
  const unsigned char* xbase = reinterpret_cast<const unsigned char*>(a.x);
  const unsigned char* wbase = reinterpret_cast<const unsigned char*>(a.W);
  auto lds_addr = [](const void* p) { return static_cast<unsigned>(reinterpret_cast<uintptr_t>(p)); };
  auto phase_region = [&](int p) -> unsigned char* { return p < RING ? myring + p * REGION : myx; };
  auto issue_phase = [&](int p) {
    const unsigned char* sb = wbase + p * 2048;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      const unsigned dst = lds_addr(phase_region(p) + j * 1024);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst), "v"(goff[j]), "s"(sb) : "memory", "m0");
    }
  };

  // ---- every load of this wavefront, oldest first: activations, then the weight
#pragma unroll
  for (int n = 0; n < XR; ++n) {
    // Rows past the last one are not fetched: their LDS blocks keep whatever they held, and what the MFMA makes of
    // that stays in output columns nobody stores. Fewer loads ahead of a wait only make it less strict than written.
    if (n < nvalid) {
      const unsigned dst = lds_addr(myx + n * XBLOCK);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(xoff[n]), "s"(xbase) : "memory", "m0");
    }
  }
#pragma unroll
  for (int p = 0; p < RPH; ++p) issue_phase(p);

  // ---- activation fragments into registers (the weight loads are younger and stay outstanding)
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(RPH * 3) : "memory");
  bf16x8 fb[16];
#pragma unroll
  for (int s = 0; s < 16; ++s) fb[s] = *reinterpret_cast<const bf16x8*>(myx + m1 * XBLOCK + (((4 * s + g) ^ (2 * m1)) << 4));
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the activation blocks are free from here on
  if constexpr (NPH > RPH) issue_phase(NPH - 1);

  // ---- the stream: phase by phase out of LDS into the matrix core
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const int arow = m < RW ? m : m - RW;                     // tile rows past the twelfth re-read a real one (their sums are dropped)
  const unsigned a_o = arow * 256;
  // W8: the lane's eight fp8 of step st are bytes 32 st + 8 g of the row's 256-byte piece: half g & 1 of chunk
  // 2 st + g / 2, which sits at position chunk ^ row
  auto w8frag = [&](const unsigned char* reg, int st) {
    typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2;
    const u32x2 raw = *reinterpret_cast<const u32x2*>(reg + a_o + (((2 * st + (g >> 1)) ^ arow) << 4) + (g & 1) * 8);
    return fp8x8_to_bf16x8(raw[0], raw[1]);
  };
#pragma unroll
  for (int p = 0; p < NPH; ++p) {
    // three loads per phase, every phase requested by now: phase p has landed when 3 * (NPH - 1 - p) are outstanding
    if (p == NPH - 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (p == NPH - 2) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    else if (p == NPH - 3) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
    const unsigned char* reg = phase_region(p);
    bf16x8 fa[PSTEPS];
#pragma unroll
    for (int st = 0; st < PSTEPS; ++st) {
      if constexpr (W8) fa[st] = w8frag(reg, st);
      else fa[st] = *reinterpret_cast<const bf16x8*>(reg + a_o + (((4 * st + g) ^ arow) << 4));
    }
#pragma unroll
    for (int st = 0; st < PSTEPS; ++st) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[st], fb[PSTEPS * p + st], acc, 0, 0, 0);
  }

  // ---- partial tile -> LDS (the wavefront's own region 1, long since consumed), then the epilogue wavefront takes over
  *reinterpret_cast<f32x4*>(myring + REGION + lane * 16) = acc;
  __syncthreads();
}

void launch_out_decode_r8(dim3 grid, hipStream_t st, const OutArgs& a) {
  auto al8 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 8 == 0; };
  const int vec8 = al8(a.out) && a.out_rs % 4 == 0 && (a.res == nullptr || (al8(a.res) && a.res_rs % 4 == 0)) && (a.bias == nullptr || al8(a.bias));
  if (a.w_scale) hipLaunchKernelGGL(out_decode_r8_kernel<true>, grid, dim3(576), 0, st, a, vec8);
  else hipLaunchKernelGGL(out_decode_r8_kernel<false>, grid, dim3(576), 0, st, a, vec8);
}

}  // namespace tllm
