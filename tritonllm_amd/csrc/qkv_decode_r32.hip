// Decode-size fused QKV projection + bias + rotary for hidden == 2880 and 9..32 activation rows per workgroup (bf16
// weight, activations already normalised): the companion of qkv_decode_r8.hip for the larger decode batches.
//
// Same skeleton: 256 workgroups of ten rotation pairs (20 weight rows, two 16-row MFMA tiles with the quad layout
// [lo(2i), lo(2i+1), hi(2i), hi(2i+1)]), six streaming wavefronts that each own one K slice of 480 (fifteen k32
// steps in phases of 4 + 4 + 4 + 3, a wavefront's steps being its share of each phase so that the six together read
// contiguous memory), everything loaded from global memory straight into LDS with the XOR swizzle
// chosen on the global side, fragments read back once, partial tiles reduced in a fixed order by epilogue wavefronts.
// What differs: 32 activation rows are 184 KB per workgroup, more than the LDS holds, so the activations arrive in the
// same four phases as the weight -- a phase is 8 KB of activations (32 rows x 256 bytes) and 5 KB of weight -- through
// a ring of two 13 KB regions per wavefront; a phase is multiplied (two tiles x two column blocks of 16 rows) as soon
// as it has landed and its region is then refilled with the phase after next. Four epilogue wavefronts, one per
// (tile, column block).
// W8: the weight is fp8 (OCP e4m3) with one fp32 scale per output row (triton_kernels.py:261-268, 927-965): a phase of
// weight is 20 rows x 128 bytes (three loads of eight rows), fragments are widened to bf16 (exact) between the LDS
// read and the MFMA, the row scale multiplies the finished sum.
#include "qkv_decode_stream.h"

namespace tllm {

namespace r32 {
constexpr int XR = 32;            // activation rows per workgroup
constexpr int NS = 6;             // streaming wavefronts = K slices
constexpr int NE = 4;             // epilogue wavefronts = (tile, column block)
constexpr int PAIRS = 10;         // rotation pairs per workgroup
constexpr int RING = 2;           // resident phases per wavefront
constexpr int XPH = 8 * 1024;     // activations of one phase: 32 rows x four k32 steps
constexpr int WPH = 5 * 1024;     // weight of one phase: 20 rows x four k32 steps
constexpr int REGION = XPH + WPH;
}  // namespace r32

template <bool W8>
__global__ __launch_bounds__(640) void qkv_decode_r32_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr, int out4) {
  using namespace r32;
  constexpr int LW = W8 ? 3 : 5;                            // weight load instructions per phase
  __shared__ __align__(1024) unsigned char ring[NS * RING * REGION];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int total_pairs = (a.n_q_heads + 2 * a.n_kv_heads) * 32;
  const int pair0 = blockIdx.x * PAIRS;
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * XR;
  const int nvalid = static_cast<int>(a.rows - row0 < XR ? a.rows - row0 : XR);

  if (wave >= NS) {
    // ======================================================================= epilogue wavefront of (tile, column block)
    const int tile = (wave - NS) & 1, cb = (wave - NS) >> 1;
    // L2 warm-up for the later phases. The activations were written by the kernel before this one, so no XCD's L2
    // holds them yet; the streaming wavefronts of all CUs ask for a phase at about the same time and wait for it at
    // memory latency. The first epilogue wavefront of each of the 32 workgroups of an XCD (consecutive workgroup ids go
    // to consecutive XCDs) touches 1/32 of the rows' bytes now -- a handful of loads per CU -- so that by the time
    // phases 2 and 3 are requested their lines sit in the XCD's L2.
    f32x4 warm[6];
    if (wave == NS) {
      const unsigned total = static_cast<unsigned>(nvalid) * 5760u;          // bytes of this workgroup's rows (contiguous)
      const unsigned share = ((total + 31u) / 32u + 1023u) & ~1023u;         // per workgroup of the XCD, whole 1 KB loads
      const unsigned first = ((blockIdx.x >> 3) & 31u) * share;
      const unsigned char* xr = reinterpret_cast<const unsigned char*>(a.x) + row0 * 5760;
#pragma unroll
      for (int j = 0; j < 6; ++j) {
        unsigned o = first + j * 1024u + lane * 16u;
        o = o < total - 16u ? o : total - 16u;
        warm[j] = *reinterpret_cast<const f32x4*>(xr + o);
      }
    }
    StreamEpilogueLane<W8> ep;
    ep.prepare(a, ra, fr, pair0, tile, lane >> 4, 16 * cb + (lane & 15), row0, nvalid);   // quad of the tile, activation row
    unsigned red_o = static_cast<unsigned>((2 * tile + cb) * 1024 + lane * 16);
    asm volatile("" : "+v"(red_o));
    if (wave == NS) {
#pragma unroll
      for (int j = 0; j < 6; ++j) asm volatile("" ::"v"(warm[j]));          // the values themselves are not needed
    }
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
    ep.finish(acc, out4);
    return;
  }

  // ========================================================================= streaming wavefront of K slice `kq`
  const int kq = wave;
  const int xblocks = (nvalid + 3) >> 2;                    // four-row activation blocks that hold a real row
  const int m = lane & 15, g = lane >> 4, m1 = m & 7;
  unsigned char* myring = ring + wave * (RING * REGION);

  // lane -> (row r4 of a 4-row block, position pos): it fetches chunk pos ^ (row & 15) of that row, so that the 16 rows
  // a fragment read touches lie in 16 different bank groups. Phase 3 has three steps: chunks 0..11 only.
  unsigned xoff[8], xoff3[8], goff[LW], goff3[LW];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int r = 4 * j + (lane >> 4);
    const int src = r < nvalid ? r : nvalid - 1;            // row inside the workgroup's 32 (the base below points at row0)
    const int cc = (lane & 15) ^ (r & 15);
    xoff[j] = static_cast<unsigned>(src * 5760 + kq * 256 + cc * 16);
    xoff3[j] = static_cast<unsigned>(src * 5760 + kq * 192 + (cc < 12 ? cc : 11) * 16);
  }
#pragma unroll
  // (W8: a weight row of a phase is 128 bytes = 8 chunks of 16 fp8 and a load covers eight rows: lane -> row
  // 8 j + lane / 8, position lane % 8, chunk position ^ (row & 7); rows 20..23 of the third load repeat row 19, unread)
  for (int j = 0; j < LW; ++j) {
    int row20 = W8 ? 8 * j + (lane >> 3) : 4 * j + (lane >> 4);   // 0..11 tile 0, 12..19 tile 1
    row20 = row20 < 20 ? row20 : 19;
    const int tile = row20 >= 12, trow = tile ? row20 - 12 : row20;
    const int quad = trow >> 2, q = trow & 3;
    int gp = pair0 + (tile ? 6 : 0) + 2 * quad + (q & 1);
    gp = gp < total_pairs ? gp : total_pairs - 1;
    const unsigned wrow = static_cast<unsigned>(gp >> 5) * 64u + (gp & 31) + ((q & 2) ? 32u : 0u);
    if constexpr (W8) {
      const int cc = (lane & 7) ^ (row20 & 7);
      goff[j] = wrow * 2880u + kq * 128u + cc * 16u;
      goff3[j] = wrow * 2880u + kq * 96u + (cc < 6 ? cc : 5) * 16u;
    } else {
      const int cc = (lane & 15) ^ (trow & 15);
      goff[j] = wrow * 5760u + kq * 256u + cc * 16u;
      goff3[j] = wrow * 5760u + kq * 192u + (cc < 12 ? cc : 11) * 16u;
    }
  }
  const unsigned char* xbase = reinterpret_cast<const unsigned char*>(a.x) + row0 * 5760;
  const unsigned char* wbase = reinterpret_cast<const unsigned char*>(a.W);
  auto lds_addr = [](const void* p) { return static_cast<unsigned>(reinterpret_cast<uintptr_t>(p)); };
  auto issue_phase = [&](int p) {                           // thirteen loads: the activations of the phase, then its weight
    unsigned char* reg = myring + (p % RING) * REGION;
    // phase p < 3: the six wavefronts together take 24 consecutive k32 steps (1536 contiguous bytes of every row),
    // wavefront kq steps 24 p + 4 kq .. + 4; phase 3: 18 steps, wavefront kq steps 72 + 3 kq .. + 3
    const unsigned char* xb = xbase + (p < 3 ? p * 1536 : 4608);
    const unsigned char* wb = wbase + (p < 3 ? p * 1536 : 4608) / (W8 ? 2 : 1);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      // Four-row blocks past the last row are not fetched: their LDS keeps whatever it held, and what the MFMA makes
      // of that stays in output columns nobody stores (a column depends on its own activation row only)
      // (the waits below count the loads of the phase after the one they wait for, so they depend on xblocks).
      if (j < xblocks) {
        const unsigned dst = lds_addr(reg + j * 1024);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(p == 3 ? xoff3[j] : xoff[j]), "s"(xb) : "memory", "m0");
      }
    }
#pragma unroll
    for (int j = 0; j < LW; ++j) {
      const unsigned dst = lds_addr(reg + XPH + j * 1024);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst), "v"(p == 3 ? goff3[j] : goff[j]), "s"(wb) : "memory", "m0");
    }
  };
  issue_phase(0);
  issue_phase(1);

  f32x4 acc[2][2];                                          // [tile][column block]
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int c = 0; c < 2; ++c) acc[t][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int arow0 = m < 12 ? m : m - 12;                    // tile rows past the last real one re-read a real one (their sums are dropped)
  const unsigned a0_o = XPH + arow0 * (W8 ? 128 : 256), a1_o = XPH + (12 + m1) * (W8 ? 128 : 256);
  // W8: the lane's eight fp8 of step st are bytes 32 st + 8 g of the 128-byte row: half g & 1 of chunk 2 st + g / 2,
  // which sits at position chunk ^ (row & 7)
  auto w8frag = [&](const unsigned char* reg, unsigned row_o, int row, int st) {
    typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2;
    const u32x2 raw = *reinterpret_cast<const u32x2*>(reg + row_o + (((2 * st + (g >> 1)) ^ (row & 7)) << 4) + (g & 1) * 8);
    return fp8x8_to_bf16x8(raw[0], raw[1]);
  };
  const unsigned b0_o = m * 256, b1_o = (16 + m) * 256;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    // phase p has landed when only the loads of the phase after it (if requested) are outstanding
    if (p < 3) {
      // s_waitcnt takes an immediate: one case per number of loads of a phase (xblocks activation blocks + LW of weight)
      switch (xblocks + LW) {
        case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
        case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
        case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
        case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
        case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
        case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
        case 11: asm volatile("s_waitcnt vmcnt(11)" ::: "memory"); break;
        case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(13)" ::: "memory"); break;
      }
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const unsigned char* reg = myring + (p % RING) * REGION;
    const int nst = p == 3 ? 3 : 4;
    bf16x8 fa0[4], fa1[4], fb0[4], fb1[4];
#pragma unroll
    for (int st = 0; st < nst; ++st) {
      fb0[st] = *reinterpret_cast<const bf16x8*>(reg + b0_o + (((4 * st + g) ^ m) << 4));
      fb1[st] = *reinterpret_cast<const bf16x8*>(reg + b1_o + (((4 * st + g) ^ m) << 4));
      if constexpr (W8) {
        fa0[st] = w8frag(reg, a0_o, arow0, st);
        fa1[st] = w8frag(reg, a1_o, 12 + m1, st);
      } else {
        fa0[st] = *reinterpret_cast<const bf16x8*>(reg + a0_o + (((4 * st + g) ^ arow0) << 4));
        fa1[st] = *reinterpret_cast<const bf16x8*>(reg + a1_o + (((4 * st + g) ^ m1) << 4));
      }
    }
    if (p + RING < 4) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // the region's fragments are in registers: it may be refilled
      issue_phase(p + RING);
    }
#pragma unroll
    for (int st = 0; st < nst; ++st) {
      acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa0[st], fb0[st], acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa0[st], fb1[st], acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa1[st], fb0[st], acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa1[st], fb1[st], acc[1][1], 0, 0, 0);
    }
  }

  // ---- partial tiles -> LDS: the wavefront's own region 0 (phase 2, consumed; phase 3 sat in region 1)
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int c = 0; c < 2; ++c) *reinterpret_cast<f32x4*>(myring + (2 * t + c) * 1024 + lane * 16) = acc[t][c];
  }
  __syncthreads();
}

// w8: fp8 weight with a.w_scale
void launch_qkv_decode_r32(bool w8, dim3 grid, hipStream_t st, const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr) {
  const int out4 = qkv_outputs_allow_4_byte_stores(a);
  if (w8) hipLaunchKernelGGL(qkv_decode_r32_kernel<true>, grid, dim3(640), 0, st, a, ra, fr, out4);
  else hipLaunchKernelGGL(qkv_decode_r32_kernel<false>, grid, dim3(640), 0, st, a, ra, fr, out4);
}

}  // namespace tllm
