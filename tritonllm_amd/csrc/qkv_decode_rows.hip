// Decode-size fused QKV projection + bias + rotary for hidden == 2880 and any number of activation rows, with ONE pass
// over the weight: the kernel for the batches between the 32-row streaming kernel and the prefill GEMM.
//
// Same division of the output as the other streaming kernels: 256 workgroups of ten rotation pairs (20 weight rows, two
// 16-row MFMA tiles with the quad layout [lo(2i), lo(2i+1), hi(2i), hi(2i+1)]), six streaming wavefronts that each own
// one K slice of 480 (fifteen k32 steps in phases of 4 + 4 + 4 + 3, a wavefront's steps being its share of each phase
// so that the six together read contiguous memory), partial tiles reduced in a fixed order by two epilogue wavefronts.
// What differs is which operand stays: a wavefront's share of the weight -- 20 rows x 480 K, thirty MFMA fragments --
// is brought in once (through the ring, coalesced) and stays in registers; the activations then stream past it in
// blocks of 16 rows. A block arrives in the four K phases (a unit = 16 rows x 256 bytes per wavefront, global memory straight
// into LDS with the XOR swizzle chosen on the global side) through a ring of five units per wavefront, so four units
// are in flight while one is multiplied. After a block's last unit the wavefronts park their partial tiles in one of
// two buffers and meet the epilogue wavefronts at a barrier; those finish the block (sum, bias, rotation, one
// rounding, stores) while the next block is multiplied.
// Per CU: 115 KB of weight from HBM once, and rows x 5760 bytes of activations from the L2s. A block of 16 rows costs
// ~1.4 us, most of it the streaming wavefronts' own chain (wait, fragment reads, dependent MFMAs, barrier) rather than
// the bytes; the prefill GEMM, whose tiles share activations between fewer CUs, takes over at a few hundred rows.
// W8: the weight is fp8 (OCP e4m3) with one fp32 scale per output row (triton_kernels.py:261-268, 927-965): the
// fragments are widened to bf16 (exact) once, on their way into the registers; the row scale multiplies the finished sum.
#include "qkv_decode_stream.h"

namespace tllm {

namespace rows {
constexpr int NS = 6;             // streaming wavefronts = K slices
constexpr int NE = 2;             // epilogue wavefronts = tiles
constexpr int STEPS = 15;         // k32 steps per slice
constexpr int PAIRS = 10;         // rotation pairs per workgroup
constexpr int XB = 16;            // activation rows per block
constexpr int UNIT = XB * 256;    // one phase of a block for one wavefront: 16 rows x four k32 steps
constexpr int NU = 5;             // ring slots per wavefront
constexpr int LPU = UNIT / 1024;  // load instructions per unit
constexpr int PART = 2 * 1024;    // a wavefront's two partial tiles
}  // namespace rows

template <bool W8>
__global__ __launch_bounds__(512) void qkv_decode_rows_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr, int out4) {
  using namespace rows;
  __shared__ __align__(1024) unsigned char ring[NS * NU * UNIT];
  __shared__ __align__(1024) unsigned char part[2 * NS * PART];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  {
    // the kernel arguments the first loads need, fetched in one go with the others
    const void* p0 = a.x;
    const void* p1 = a.W;
    asm volatile("" ::"s"(p0), "s"(p1));
  }
  const int total_pairs = (a.n_q_heads + 2 * a.n_kv_heads) * 32;
  const int pair0 = blockIdx.x * PAIRS;
  const int nblk = static_cast<int>((a.rows + XB - 1) / XB);
  // Every workgroup reads all of the activations; walking the blocks in the same order they would all pull on the same
  // few lines of the same L2 channels at the same time. The workgroups that share an XCD's L2 (every eighth id) start
  // at different blocks instead: the b-th block a workgroup takes is block (b + rot) mod nblk.
  const int rot = static_cast<int>((blockIdx.x >> 3) % static_cast<unsigned>(nblk));
  auto block_at = [&](int b) { return b + rot < nblk ? b + rot : b + rot - nblk; };

  if (wave >= NS) {
    // ======================================================================= epilogue wavefront of tile `tile`
    const int tile = wave - NS;
    const int eg = lane >> 4, en = lane & 15;               // quad of the tile, activation row of the block
    // Between two barriers this wavefront is the workgroup's critical path (the streaming wavefronts need ~0.5 us per
    // block), so nothing with a memory latency in it may sit there: what depends on the lane only is made once, the
    // row's position is requested two blocks ahead, its cos / sin and output address are made one block ahead (before
    // the barrier, while the streaming wavefronts multiply); between the barriers it sums, rotates and stores.
    auto row0_of = [&](int b) { return static_cast<int64_t>(block_at(b < nblk ? b : nblk - 1)) * XB; };
    auto nvalid_of = [&](int64_t row0) { return static_cast<int>(a.rows - row0 < XB ? a.rows - row0 : XB); };
    StreamEpilogueLane<W8> ep;
    ep.prepare(a, ra, fr, pair0, tile, eg, en, row0_of(0), nvalid_of(row0_of(0)));
    int64_t pos_next = ep.request_row(a, ra, en, row0_of(1), nvalid_of(row0_of(1)));
    for (int b = 0; b < nblk; ++b) {
      const int64_t row1 = row0_of(b + 1), row2 = row0_of(b + 2);   // past the end: the last block again
      StreamEpilogueLane<W8> next = ep;
      next.prepare_row(a, ra, fr, pos_next, en, row1, nvalid_of(row1));
      unsigned red_o = static_cast<unsigned>((b & 1) * (NS * PART) + tile * 1024 + lane * 16);
      asm volatile("" : "+v"(red_o));
      asm volatile("s_barrier" ::: "memory");               // the partial tiles of block b are in LDS
      f32x4 t[NS];
#pragma unroll
      for (int w = 0; w < NS; ++w) t[w] = *reinterpret_cast<const f32x4*>(part + w * PART + red_o);
      // requested before this block's stores go out: the wait for it, one round on, then does not wait for them
      const int64_t pos_after = ep.request_row(a, ra, en, row2, nvalid_of(row2));
      f32x4 acc = t[0];
#pragma unroll
      for (int w = 1; w < NS; ++w) {                        // fixed order: the result does not depend on timing
        acc[0] += t[w][0];
        acc[1] += t[w][1];
        acc[2] += t[w][2];
        acc[3] += t[w][3];
      }
      ep.finish(acc, out4);
      ep = next;
      pos_next = pos_after;
    }
    return;
  }

  // ========================================================================= streaming wavefront of K slice `kq`
  const int kq = wave;
  const int m = lane & 15, g = lane >> 4, m1 = m & 7;
  unsigned char* myring = ring + wave * (NU * UNIT);
  const int total_units = 4 * nblk;

  // ---- activations. Unit (b, p): rows 16 b .. + 16, phase p < 3: the six wavefronts together take 24 consecutive k32
  // steps (1536 contiguous bytes of every row), wavefront kq the 256 bytes at p * 1536 + kq * 256; phase 3: 18 steps,
  // wavefront kq the 192 bytes at 4608 + kq * 192. Load j of a unit covers rows 4 j .. + 4: lane -> (row 4 j + lane / 16,
  // position lane % 16), and it fetches chunk position ^ row of that row, so that the 16 rows a fragment read touches
  // lie in 16 different bank groups. Rows past the last one re-read it (a block is always fetched whole: the waits
  // below count loads; what the MFMA makes of those rows stays in output columns nobody stores).
  unsigned xoff[LPU], xoff3[LPU], xoff_last[LPU], xoff3_last[LPU];
  const int last_rows = static_cast<int>(a.rows - static_cast<int64_t>(nblk - 1) * XB);   // rows of the last block, 1..16
#pragma unroll
  for (int j = 0; j < LPU; ++j) {
    const int r = 4 * j + (lane >> 4);
    const int cc = (lane & 15) ^ r;
    const int rl = r < last_rows ? r : last_rows - 1;
    xoff[j] = static_cast<unsigned>(r * 5760 + kq * 256 + cc * 16);
    xoff3[j] = static_cast<unsigned>(r * 5760 + kq * 192 + (cc < 12 ? cc : 11) * 16);
    xoff_last[j] = static_cast<unsigned>(rl * 5760 + kq * 256 + cc * 16);
    xoff3_last[j] = static_cast<unsigned>(rl * 5760 + kq * 192 + (cc < 12 ? cc : 11) * 16);
  }
  const unsigned char* xbase = reinterpret_cast<const unsigned char*>(a.x);
  auto lds_addr = [](const void* p) { return static_cast<unsigned>(reinterpret_cast<uintptr_t>(p)); };
  auto issue_unit = [&](int u, int slot) {                  // unit u = phase u % 4 of the (u / 4)-th block, into ring slot `slot`
    const int b = block_at(u >> 2), p = u & 3;
    const unsigned char* sb = xbase + static_cast<int64_t>(b) * (XB * 5760) + (p < 3 ? p * 1536 : 4608);
    const bool last = b == nblk - 1;
#pragma unroll
    for (int j = 0; j < LPU; ++j) {
      const unsigned dst = lds_addr(myring + slot * UNIT + j * 1024);
      const unsigned off = p == 3 ? (last ? xoff3_last[j] : xoff3[j]) : (last ? xoff_last[j] : xoff[j]);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(sb) : "memory", "m0");
    }
  };
  // ---- the weight, once. It arrives like the stream of the 8-row kernel: four phases of 20 rows x 256 bytes (192 in
  // the last) land in the ring (4 x 5 KB, the whole of it), coalesced; lane -> (row 4 j + lane / 16 of the 20-row
  // patch, position lane % 16) fetches chunk position ^ (tile row & 15) of that row. Tile 0 = patch rows 0..11 (tile
  // rows 12..15 re-read 0..3, their sums are dropped), tile 1 = patch rows 12..19 (tile rows 8..15 re-read them). A
  // phase's fragments go into registers as soon as it has landed -- lane (m, g) holds of tile row m the eight K
  // elements of chunk 4 s + g of every step s -- and stay there.
  constexpr int LPW = 5;                                    // weight load instructions per phase
  constexpr int WREGION = 20 * 256;
  static_assert(4 * WREGION <= NU * UNIT, "the weight's four phases fit the ring");
  unsigned goff[LPW], goff3[LPW];
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int row20 = 4 * j + (lane >> 4);                  // 0..11 tile 0, 12..19 tile 1
    const int tile = row20 >= 12, trow = tile ? row20 - 12 : row20;
    const int quad = trow >> 2, q = trow & 3;
    int gp = pair0 + (tile ? 6 : 0) + 2 * quad + (q & 1);
    gp = gp < total_pairs ? gp : total_pairs - 1;
    const unsigned wrow = static_cast<unsigned>(gp >> 5) * 64u + (gp & 31) + ((q & 2) ? 32u : 0u);
    const int cc = (lane & 15) ^ (trow & 15);
    if constexpr (W8) {                                     // a row piece of a phase is 128 bytes of fp8: chunks 0..7 (0..5 in the last)
      goff[j] = wrow * 2880u + kq * 128u + (cc & 7) * 16u;
      goff3[j] = wrow * 2880u + kq * 96u + ((cc & 7) < 6 ? (cc & 7) : 5) * 16u;
    } else {
      goff[j] = wrow * 5760u + kq * 256u + cc * 16u;
      goff3[j] = wrow * 5760u + kq * 192u + (cc < 12 ? cc : 11) * 16u;
    }
  }
  const unsigned char* wbase = reinterpret_cast<const unsigned char*>(a.W);
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const unsigned char* sb = wbase + (p < 3 ? p * 1536 : 4608) / (W8 ? 2 : 1);
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
      const unsigned dst = lds_addr(myring + p * WREGION + j * 1024);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst), "v"(p == 3 ? goff3[j] : goff[j]), "s"(sb) : "memory", "m0");
    }
  }
  bf16x8 fa0[STEPS], fa1[STEPS];
  const int arow0 = m < 12 ? m : m - 12;
  const unsigned a0_o = arow0 * 256, a1_o = (12 + m1) * 256;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    if (p == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * LPW) : "memory");
    else if (p == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LPW) : "memory");
    else if (p == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPW) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned char* reg = myring + p * WREGION;
    const int nst = p == 3 ? 3 : 4;
#pragma unroll
    for (int st = 0; st < nst; ++st) {
      if constexpr (W8) {
        // the lane's eight fp8 of step st are bytes 32 st + 8 g of the row's 128-byte piece: half g & 1 of chunk
        // 2 st + g / 2, which sits at position (chunk ^ tile row) & 7
        typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2;
        const u32x2 r0 = *reinterpret_cast<const u32x2*>(reg + a0_o + ((((2 * st + (g >> 1)) ^ arow0) & 7) << 4) + (g & 1) * 8);
        const u32x2 r1 = *reinterpret_cast<const u32x2*>(reg + a1_o + ((((2 * st + (g >> 1)) ^ m1) & 7) << 4) + (g & 1) * 8);
        fa0[4 * p + st] = fp8x8_to_bf16x8(r0[0], r0[1]);
        fa1[4 * p + st] = fp8x8_to_bf16x8(r1[0], r1[1]);
      } else {
        fa0[4 * p + st] = *reinterpret_cast<const bf16x8*>(reg + a0_o + (((4 * st + g) ^ arow0) << 4));
        fa1[4 * p + st] = *reinterpret_cast<const bf16x8*>(reg + a1_o + (((4 * st + g) ^ m1) << 4));
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the weight is in registers: the ring is the activations' from here on
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    if (u < total_units) issue_unit(u, u);
  }

  // ---- the stream: block by block, unit by unit out of LDS into the matrix core
  int slot = 0;                                             // ring slot of the unit about to be multiplied: u % NU
  for (int b = 0; b < nblk; ++b) {
    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int u = 4 * b + p;
      // LPU loads per unit: unit u has landed when only the units issued after it are outstanding -- four of them,
      // fewer at the end of the last block
      if (b < nblk - 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NU - 1) * LPU) : "memory");
      else asm volatile("s_waitcnt vmcnt(%0)" ::"n"((3 - p) * LPU) : "memory");
      const unsigned char* reg = myring + slot * UNIT;
      const int nst = p == 3 ? 3 : 4;
      bf16x8 fb[4];
#pragma unroll
      for (int st = 0; st < nst; ++st) fb[st] = *reinterpret_cast<const bf16x8*>(reg + m * 256 + (((4 * st + g) ^ m) << 4));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // the unit's fragments are in registers: its slot may be refilled
      if (u + NU < total_units) issue_unit(u + NU, slot);
      slot = slot + 1 == NU ? 0 : slot + 1;
#pragma unroll
      for (int st = 0; st < nst; ++st) {
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa0[4 * p + st], fb[st], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa1[4 * p + st], fb[st], acc1, 0, 0, 0);
      }
    }
    // partial tiles of the block -> buffer b % 2 (the epilogue wavefronts finished reading it before the last barrier)
    unsigned char* pp = part + (b & 1) * (NS * PART) + wave * PART;
    *reinterpret_cast<f32x4*>(pp + lane * 16) = acc0;
    *reinterpret_cast<f32x4*>(pp + 1024 + lane * 16) = acc1;
    // spelled out: __syncthreads() carries a fence that would drain the four units in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }
}

// w8: fp8 weight with a.w_scale
void launch_qkv_decode_rows(bool w8, dim3 grid, hipStream_t st, const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr) {
  const int out4 = qkv_outputs_allow_4_byte_stores(a);
  if (w8) hipLaunchKernelGGL(qkv_decode_rows_kernel<true>, grid, dim3(512), 0, st, a, ra, fr, out4);
  else hipLaunchKernelGGL(qkv_decode_rows_kernel<false>, grid, dim3(512), 0, st, a, ra, fr, out4);
}

}  // namespace tllm
