// Decode-size fused (RMSNorm +) QKV projection + bias + rotary for hidden == 2880 and up to 8 activation rows per
// workgroup -- the weight-streaming kernel of the gpt-oss decode step (B <= 8) -- and, with the fused norm, up to 16.
//
// Work per CU. The 2560 rotation pairs are dealt ten at a time to 256 workgroups, each needing most of a CU's LDS, so
// exactly one lands on every CU and every CU streams 1/256 of the weight: 20 rows of 5760 bytes. The rows form two
// 16-row MFMA tiles (v_mfma_f32_16x16x32_bf16: weight rows on M, activation rows on N): tile 0 = pairs 0..5, tile 1 =
// pairs 6..9, two adjacent pairs (2i, 2i+1) occupying four tile rows [lo(2i), lo(2i+1), hi(2i), hi(2i+1)], so that one
// lane ends up with both halves of two adjacent rotation pairs.
//
// What was measured on the machine and what the kernel does about it:
//   * A CU returns vector loads in the order it took them, across wavefronts, and takes only so many at a time. A
//     barrier that waits for staged activations therefore waits for every weight load queued ahead of them. Here no
//     wavefront ever waits for another one's loads: each of the six streaming wavefronts owns one K slice of 480
//     (fifteen k32 steps, taken as its share of four phases so that the six together read contiguous memory) and
//     brings in its own slice of the activations, then its slice of the 20 weight rows.
//   * Passing the stream through registers and ds_write into operand layout costs as much time as the stream
//     itself (loads, LDS writes and LDS reads all cross the same register-file port). Here everything goes from
//     global memory straight into LDS (global_load_lds_dwordx4: a wavefront's 64 x 16 bytes land at consecutive LDS
//     addresses; which global chunk a lane fetches is free, and that freedom carries the XOR swizzle that makes the
//     fragment reads conflict-free) and is read back once, as MFMA fragments.
//   * The weight slice of a wavefront arrives in four phases (4 + 4 + 4 + 3 k32 steps) through a ring of three
//     5 KB regions; a phase is multiplied as soon as it has landed, so three steps remain when the stream ends.
//   * The six partial tiles meet in LDS; two further wavefronts (one per tile), which loaded position, bias and
//     scales and computed cos/sin while the stream ran, add them in a fixed order, add the bias, rotate, round once
//     and store two adjacent dims at a time.
// The loads of the streaming wavefronts are inline asm (the compiler cannot express "to LDS"), so their
// s_waitcnt vmcnt are spelled by hand; those wavefronts issue no other vector load once the first asm load is out.
//
// NORM: 0 = x is used as it is; 1 / 2 = x is first RMS-normalised with an fp32 / bf16 scale: the wavefronts sum the
// squares of their slices from the fragments, exchange them (one barrier) and scale the fragments in registers --
// fp32 arithmetic, one rounding to bf16: the operand the separate rmsnorm launch would hand over.
// EMB: the activation rows are gathered from an embedding table by token id (model.py:906-920 feeding the first
// block); workgroup 0 also writes the gathered rows out. An id outside the table gives a zero row and raises the flag.
// XR: 8 or 16 activation rows per workgroup. Sixteen rows (with the fused norm only; without it qkv_decode_r32.hip
// takes 9..32 rows) fill the MFMA's 16 columns and 96 KB of LDS, which leaves room for one ring region: phase 0 lands
// there and is requested before the norm; the later phases are requested after the sums are published -- by then the
// activation fragments are in registers -- and land in the activation blocks.
// W8: the weight is fp8 (OCP e4m3) with one fp32 scale per output row (triton_kernels.py:261-268, 927-965). A
// wavefront's 480 bytes of a row arrive in two phases of 8 + 7 k32 steps (256 + 224 bytes, so a row piece is as long
// as in the bf16 form and the LDS layout is the same), fragments are widened to bf16 (exact) between the LDS read and
// the MFMA, the row scale multiplies the finished sum.
#include "qkv_decode_stream.h"

namespace tllm {

namespace r8 {
constexpr int NS = 6;             // streaming wavefronts = K slices
constexpr int NE = 2;             // epilogue wavefronts = tiles
constexpr int STEPS = 15;         // k32 steps per slice
constexpr int PAIRS = 10;         // rotation pairs per workgroup
constexpr int REGION = 20 * 256;  // one phase: 20 weight rows x four k32 steps
constexpr int XBLOCK = 1024;      // one activation row of a slice: 60 chunks of 16 bytes (+ 4 spare)
constexpr int ring_regions(int xr) { return xr == 8 ? 3 : 1; }   // ring regions per wavefront
}  // namespace r8

// Set (and never cleared) by a wavefront whose bounded wait for the other wavefronts' norm sums ran out.
__device__ int g_qkv_decode_wait_expired = 0;
constexpr int kFlagPollLimit = 1 << 18;

#ifdef TLLM_R8_STAMPS
__device__ unsigned long long g_r8_stamps[256 * 8 * 8];
#define R8_STAMP(i) do { if (lane == 0 && blockIdx.y == 0 && blockIdx.x < 256) g_r8_stamps[(blockIdx.x * 8 + wave) * 8 + (i)] = wall_clock64(); } while (0)
#else
#define R8_STAMP(i) do { } while (0)
#endif

template <int XR, int NORM, bool EMB, bool W8>
__global__ __launch_bounds__(512) void qkv_decode_r8_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr, int out4) {
  using namespace r8;
  static_assert(!EMB || NORM != 0, "the fused gather exists with the fused norm only");
  static_assert(XR == 8 || (XR == 16 && NORM != 0), "sixteen rows: with the fused norm only");
  constexpr int RING = ring_regions(XR);
  constexpr int LPW = 5;                                    // weight load instructions per phase and wavefront
  constexpr int NPH = W8 ? 2 : 4;                           // phases: bf16 4 + 4 + 4 + 3 k32 steps, fp8 8 + 7
  constexpr int PSTEPS = W8 ? 8 : 4;                        // k32 steps of a full phase
  // phases that land in the ring; the others land in the activation blocks, which are free once the activation
  // fragments are in registers (8 rows: the last bf16 phase; 16 rows: every phase but the first)
  constexpr int RPH = XR == 8 ? (W8 ? 2 : RING) : 1;
  static_assert((NPH - RPH) * REGION <= XR * XBLOCK, "the phases behind the ring fit the activation blocks");
  __shared__ __align__(1024) unsigned char xw[NS * XR * XBLOCK];
  __shared__ __align__(1024) unsigned char ring[NS * RING * REGION];
  __shared__ __align__(1024) unsigned char scw[NORM ? NS * 2048 : 16];
  __shared__ float s_part[NORM ? NS * XR : 1];
  __shared__ unsigned s_flag[NORM ? NS : 1];              // s_part[w][*] of streaming wavefront w is complete

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // every kernel argument the first loads need, fetched in one go (left to its first use, the activations' base
  // arrives by a scalar load of its own, a quarter of a microsecond behind the others)
  {
    const void* p0 = EMB ? static_cast<const void*>(a.emb_table) : static_cast<const void*>(a.x);
    const void* p1 = a.W;
    const void* p2 = a.norm_scale;
    asm volatile("" ::"s"(p0), "s"(p1), "s"(p2));
  }
  const int total_pairs = (a.n_q_heads + 2 * a.n_kv_heads) * 32;
  const int pair0 = blockIdx.x * PAIRS;
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * XR;
  const int nvalid = static_cast<int>(a.rows - row0 < XR ? a.rows - row0 : XR);
  R8_STAMP(0);

  if (wave >= NS) {
    // ======================================================================= epilogue wavefront of tile `tile`
    const int tile = wave - NS;
    // the streaming wavefronts' rendezvous between their activation and weight loads (it also publishes their
    // cleared flags): met here at once, before this wavefront has anything to wait for
    if constexpr (NORM != 0) __syncthreads();
    StreamEpilogueLane<W8> ep;
    ep.prepare(a, ra, fr, pair0, tile, lane >> 4, lane & 15, row0, nvalid);   // quad of the tile, activation row
    unsigned red_o = static_cast<unsigned>((RING > 1 ? REGION : 0) + tile * 1024 + lane * 16);
    asm volatile("" : "+v"(red_o));
    __syncthreads();                                        // partial tiles are in LDS
    R8_STAMP(6);
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
    R8_STAMP(7);
    ep.finish(acc, out4);
    return;
  }

  // ========================================================================= streaming wavefront of K slice `kq`
  const int kq = wave;
  // The K slice of a wavefront is not one run of 480 but its share of each phase: in phase p < 3 the six wavefronts
  // together read 24 consecutive k32 steps (1536 contiguous bytes of every weight row), wavefront kq steps
  // 24 p + 4 kq .. + 4; in phase 3, 18 steps, wavefront kq steps 72 + 3 kq .. + 3. What a CU requests within a short
  // time is then contiguous in memory. kb(c): byte offset inside a bf16 row of this wavefront's 16-byte chunk c (0..59).
  // (With the fp8 weight the phases are 8 + 7 steps: 48 steps = 3072 bytes of an activation row, wavefront kq the 512
  // at kq * 512, then 42 steps, wavefront kq the 448 bytes at 3072 + kq * 448.)
  // (written without a branch: these offsets are all that stands between the wavefront's start and its first load)
  auto kb = [&](int c) {
    if constexpr (W8) return kq * 512 + c * 16 + (c >= 32 ? 2560 - kq * 64 : 0);
    else return (c >> 4) * 1536 + (c & 15) * 16 + kq * 256 - (c >= 48 ? kq * 64 : 0);
  };
  const int m = lane & 15, g = lane >> 4;
  const int m1 = XR == 8 ? (m & 7) : m;                     // activation row of the lane's MFMA column (8 rows: columns 8..15 repeat 0..7, never stored)
  unsigned char* myx = xw + wave * (XR * XBLOCK);
  unsigned char* myring = ring + wave * (RING * REGION);

  // activations: row n of the slice -> 1 KB block n; lane i fetches chunk i ^ 2n (60 real chunks, the rest re-read
  // chunk 59), the swizzle that spreads the eight rows of a fragment read over the banks
  unsigned xoff[XR];
  // 32-bit lane offsets from a scalar base: the workgroup's first row, or (EMB) the table, whose size the host checks
  const unsigned char* xbase = EMB ? reinterpret_cast<const unsigned char*>(a.emb_table) : reinterpret_cast<const unsigned char*>(a.x) + row0 * 5760;
  bool xok_m1 = true;                                       // EMB: is the id of the row this lane's fragments belong to inside the table?
  static_assert(2 * (XR - 1) < 64, "the row swizzle stays inside a 1 KB block");
  {
    int64_t src_row[XR];
#pragma unroll
    for (int n = 0; n < XR; ++n) src_row[n] = (EMB ? row0 : 0) + (n < nvalid ? n : nvalid - 1);   // EMB: index into the ids; else row inside the workgroup
    if constexpr (EMB) {
      int64_t id[XR];
#pragma unroll
      for (int n = 0; n < XR; ++n) {                        // all ids first: nothing between these loads that could order them
        id[n] = a.emb_ids_i64 ? reinterpret_cast<const int64_t*>(a.emb_ids)[src_row[n]]
                              : static_cast<int64_t>(reinterpret_cast<const int*>(a.emb_ids)[src_row[n]]);
      }
      bool any_bad = false;
#pragma unroll
      for (int n = 0; n < XR; ++n) {
        const bool ok = id[n] >= 0 && id[n] < a.emb_vocab;
        any_bad |= !ok;
        if (n == m1) xok_m1 = ok;
        src_row[n] = id[n] < 0 ? 0 : (id[n] < a.emb_vocab ? id[n] : a.emb_vocab - 1);
      }
      if (any_bad && a.emb_oob && lane == 0) *a.emb_oob = 1;
    }
#pragma unroll
    for (int n = 0; n < XR; ++n) {
      int c = lane ^ (2 * n);
      c = c < 60 ? c : 59;
      xoff[n] = static_cast<unsigned>(src_row[n] * 5760 + kb(c));
    }
  }
  // weight: lane -> (row r4 of a 4-row block, position pos): it fetches chunk pos ^ (tile row & 15) of that row
  unsigned goff[LPW], goff3[LPW];                           // full phases / the short last phase (bf16: chunks 0..11 only, fp8: 0..13)
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int row20 = 4 * j + (lane >> 4);                  // 0..11 tile 0, 12..19 tile 1
    const int tile = row20 >= 12, trow = tile ? row20 - 12 : row20;
    const int quad = trow >> 2, q = trow & 3;
    int gp = pair0 + (tile ? 6 : 0) + 2 * quad + (q & 1);
    gp = gp < total_pairs ? gp : total_pairs - 1;
    const unsigned wrow = static_cast<unsigned>(gp >> 5) * 64u + (gp & 31) + ((q & 2) ? 32u : 0u);
    const int cc = (lane & 15) ^ (trow & 15);
    if constexpr (W8) {                                     // a chunk is 16 fp8; a full phase is again 256 bytes per row and wavefront
      goff[j] = wrow * 2880u + kq * 256u + cc * 16u;
      goff3[j] = wrow * 2880u + kq * 224u + (cc < 14 ? cc : 13) * 16u;
    } else {
      goff[j] = wrow * 5760u + kq * 256u + cc * 16u;
      goff3[j] = wrow * 5760u + kq * 192u + (cc < 12 ? cc : 11) * 16u;
    }
  }
  const unsigned char* wbase = reinterpret_cast<const unsigned char*>(a.W);
  auto lds_addr = [](const void* p) { return static_cast<unsigned>(reinterpret_cast<uintptr_t>(p)); };
  // The first RPH phases land in the wavefront's ring regions, the others in its activation blocks, which are free as
  // soon as the activation fragments are in registers -- so no weight load ever waits for an MFMA.
  auto phase_region = [&](int p) -> unsigned char* { return p < RPH ? myring + p * REGION : myx + (p - RPH) * REGION; };
  auto issue_phase = [&](int p) {
    const unsigned char* sb = wbase + p * 1536;            // the six wavefronts' pieces of a full phase: 6 x 256 bytes of every row
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
      const unsigned dst = lds_addr(phase_region(p) + j * 1024);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst), "v"(p == NPH - 1 ? goff3[j] : goff[j]), "s"(sb) : "memory", "m0");
    }
  };

  // ---- every load of this wavefront, oldest first: activations, norm scale, then the weight
#pragma unroll
  for (int n = 0; n < XR; ++n) {
    // Rows past the last one are not fetched: their LDS blocks keep whatever they held, and what the MFMA makes of
    // that stays in output columns nobody stores (a column depends on its own activation row only). Fewer loads ahead
    // of a wait only make it less strict than written: the counts below are relative to the youngest loads.
    if (n < nvalid) {
      const unsigned dst = lds_addr(myx + n * XBLOCK);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(xoff[n]), "s"(xbase) : "memory", "m0");
    }
  }
  constexpr int NSC = NORM == 1 ? 2 : (NORM == 2 ? 1 : 0);   // scale loads: 480 fp32 = 120 chunks, 480 bf16 = 60 chunks
  if constexpr (NORM != 0) {
    const unsigned char* sbase = reinterpret_cast<const unsigned char*>(a.norm_scale);
#pragma unroll
    for (int t = 0; t < NSC; ++t) {
      int c = 64 * t + lane;                                // 16-byte chunk of the slice's scale: 4 fp32 or 8 bf16 values
      const int cmax = NORM == 1 ? 119 : 59;
      c = c < cmax ? c : cmax;
      const unsigned off = NORM == 1 ? 2u * kb(c >> 1) + (c & 1) * 16u : static_cast<unsigned>(kb(c));
      const unsigned dst = lds_addr(scw + wave * 2048 + t * 1024);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(sbase) : "memory", "m0");
    }
  }
  // A CU takes only so many loads at a time; a wavefront that issues one more simply stalls until the queue has
  // drained that far. Without the norm that costs nothing: everything is requested at once. With it, the wavefronts
  // must see their activations, exchange sums and scale before the first MFMA, and one stuck issuing weight loads
  // would hold the others up at the barrier: so all activation loads go first (the rendezvous puts them at the head
  // of the CU's queue, which returns loads in the order it took them), one phase of weight keeps the memory system
  // busy meanwhile, and the other three phases are requested after the norm.
  constexpr int EARLY = NORM != 0 ? 1 : RPH;
  if constexpr (NORM != 0) {
    if (lane == 0) s_flag[wave] = 0;
    __syncthreads();
  }
#pragma unroll
  for (int p = 0; p < EARLY; ++p) issue_phase(p);
  R8_STAMP(1);

  // ---- activation fragments into registers (the weight loads issued so far are younger and stay outstanding)
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(EARLY * LPW) : "memory");
  R8_STAMP(2);
  bf16x8 fb[STEPS];
  auto xfrag = [&](int s) { return *reinterpret_cast<const bf16x8*>(myx + m1 * XBLOCK + (((4 * s + g) ^ (2 * m1)) << 4)); };
  if constexpr (NORM == 0) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) fb[s] = xfrag(s);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if constexpr (NPH > RPH) issue_phase(NPH - 1);
  } else {
    // The six slices' sums meet through LDS, but not at a barrier: a wavefront publishes its sums, raises its flag and
    // goes on to request the rest of its weight (where it may sit for a microsecond until the CU's queue takes the
    // loads); only then does it wait for the other five flags, which by that time are long up.
    // Every streaming wavefront raises its flag before it gets here and none returns early, so the flags are up
    // after a few polls. The wait is bounded all the same: a wavefront that has polled kFlagPollLimit times (tens of
    // milliseconds) records that in g_qkv_decode_wait_expired and carries on to the kernel's barriers and exit with
    // whatever sums it has -- a wrong result the host can see instead of a workgroup that never ends.
    auto publish_and_meet = [&](float ssq) {                // ssq: sum of squares of row `lane` of this slice, in lanes 0 .. XR - 1
      if (lane < XR) s_part[wave * XR + lane] = ssq;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");   // LDS only: the loads in flight are none of its business
      if (lane == 0) __hip_atomic_store(&s_flag[wave], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
      for (int p = EARLY; p < NPH; ++p) issue_phase(p);
      for (int polls = 0;; ++polls) {
        const unsigned f = lane < NS ? __hip_atomic_load(&s_flag[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) : 1u;
        if (__all(f != 0u)) break;
        if (polls >= kFlagPollLimit) {
          if (lane == 0) g_qkv_decode_wait_expired = 1;
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
      float ss = 0.f;
#pragma unroll
      for (int w = 0; w < NS; ++w) ss += s_part[w * XR + m1];
      return rsqrtf(ss * (1.0f / 2880.0f) + a.norm_eps);
    };
    const unsigned char* sc = scw + wave * 2048;
    auto scaled = [&](bf16x8 v, int sj, float rinv) {       // bf16(x * rinv * scale), fp32 arithmetic, one rounding
      f32x4 s_lo, s_hi;
      if constexpr (NORM == 1) {
        s_lo = *reinterpret_cast<const f32x4*>(sc + (4 * sj + g) * 32);
        s_hi = *reinterpret_cast<const f32x4*>(sc + (4 * sj + g) * 32 + 16);
      } else {
        const bf16x8 t = *reinterpret_cast<const bf16x8*>(sc + (4 * sj + g) * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          s_lo[q] = static_cast<float>(t[q]);
          s_hi[q] = static_cast<float>(t[4 + q]);
        }
      }
      bf16x8 t;
#pragma unroll
      for (int q = 0; q < 8; ++q) t[q] = static_cast<bf16>(static_cast<float>(v[q]) * rinv * (q < 4 ? s_lo[q] : s_hi[q - 4]));
      return t;
    };
    auto sumsq = [](bf16x8 v) {
      float part = 0.f;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float f = static_cast<float>(v[q]);
        part = fmaf(f, f, part);
      }
      return part;
    };
    if constexpr (XR == 16) {
      // all sixteen MFMA columns are real rows: every lane fetches and scales the fifteen fragments of its own row
#pragma unroll
      for (int s = 0; s < STEPS; ++s) fb[s] = xfrag(s);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // the activation blocks are free from here on
      if constexpr (EMB) {
        if (!xok_m1) {
#pragma unroll
          for (int s = 0; s < STEPS; ++s) {
#pragma unroll
            for (int q = 0; q < 8; ++q) fb[s][q] = static_cast<bf16>(0.f);
          }
        }
        if (blockIdx.x == 0 && m1 < nvalid) {               // the gathered rows, as the residual stream: every lane its own fragments
          bf16x8* xo = reinterpret_cast<bf16x8*>(a.emb_out) + (row0 + m1) * 360;
#pragma unroll
          for (int s = 0; s < STEPS; ++s) xo[kb(4 * s + g) >> 4] = fb[s];
        }
      }
      float ssq = 0.f;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) ssq += sumsq(fb[s]);
      ssq = sum_over_lane_bits_16_32(ssq);
      const float rinv = publish_and_meet(ssq);             // lanes 0..15: row m1 == lane
#ifdef TLLM_R8_STAMPS
      R8_STAMP(3);
#endif
#pragma unroll
      for (int s = 0; s < STEPS; ++s) fb[s] = scaled(fb[s], s, rinv);
    } else {
      // Columns 8..15 of the MFMA are never stored, so lanes m >= 8 are free to do half of the norm's arithmetic: a
      // lane fetches and scales the fragments of the steps of its own parity (h = bit 3 of the lane), and the lanes
      // m < 8 then take the other parity's from their partner 8 lanes up (one DPP move per register).
      const int h = (lane >> 3) & 1;
      typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;
      bf16x8 own[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int sj = 2 * j + h;
        own[j] = xfrag(sj < STEPS ? sj : STEPS - 2);          // (h = 1, j = 7) has no step: re-reads step 13, masked below
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // the activation blocks are free from here on
      if constexpr (EMB) {
        if (!xok_m1) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
#pragma unroll
            for (int q = 0; q < 8; ++q) own[j][q] = static_cast<bf16>(0.f);
          }
        }
        if (blockIdx.x == 0 && m1 < nvalid) {               // the gathered rows, as the residual stream: every lane its own fragments
          bf16x8* xo = reinterpret_cast<bf16x8*>(a.emb_out) + (row0 + m1) * 360;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            if (2 * j + h < STEPS) xo[kb(4 * (2 * j + h) + g) >> 4] = own[j];
          }
        }
      }
      float ssq = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) ssq += (j == 7 && h == 1) ? 0.f : sumsq(own[j]);
      ssq += lane_xor8_value(ssq);
      ssq = sum_over_lane_bits_16_32(ssq);
      const float rinv = publish_and_meet(ssq);             // lanes 0..7: row m1 == lane
#ifdef TLLM_R8_STAMPS
      R8_STAMP(3);
#endif
#pragma unroll
      for (int j = 0; j < 8; ++j) own[j] = scaled(own[j], 2 * j + h < STEPS ? 2 * j + h : STEPS - 2, rinv);
      // lanes m < 8 (h = 0): even steps are their own, odd steps come from lane + 8; lanes m >= 8 end up with a mix
      // that only feeds the unused columns
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        fb[2 * j] = own[j];
        if (2 * j + 1 < STEPS) {
          const u32x4 mine = __builtin_bit_cast(u32x4, own[j]);
          u32x4 theirs;
#pragma unroll
          for (int q = 0; q < 4; ++q) theirs[q] = __builtin_amdgcn_update_dpp(0u, mine[q], 0x128 /* row_ror:8 */, 0xf, 0xf, false);
          fb[2 * j + 1] = __builtin_bit_cast(bf16x8, theirs);
        }
      }
    }
#ifdef TLLM_R8_STAMPS
    R8_STAMP(4);
#endif
  }

  // ---- the stream: phase by phase out of LDS into the matrix core
  f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  const int arow0 = m < 12 ? m : m - 12;                    // tile rows past the last real one re-read a real one (their sums are dropped)
  const unsigned a0_o = arow0 * 256, a1_o = (12 + m1) * 256;
  // W8: the lane's eight fp8 of step st are bytes 32 st + 8 g of the row's 256-byte piece: half g & 1 of chunk
  // 2 st + g / 2, which sits at position chunk ^ (tile row & 15)
  auto w8frag = [&](const unsigned char* reg, unsigned row_o, int trow, int st) {
    typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2;
    const u32x2 raw = *reinterpret_cast<const u32x2*>(reg + row_o + (((2 * st + (g >> 1)) ^ trow) << 4) + (g & 1) * 8);
    return fp8x8_to_bf16x8(raw[0], raw[1]);
  };
#pragma unroll
  for (int p = 0; p < NPH; ++p) {
    // LPW loads per phase, every phase requested by now: phase p has landed when LPW * (NPH - 1 - p) are outstanding
    if (p == NPH - 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (p == NPH - 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPW) : "memory");
    else if (p == NPH - 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LPW) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * LPW) : "memory");
    if (NORM == 0 && p == 0) R8_STAMP(3);
    if (NORM == 0 && p == NPH - 1) R8_STAMP(4);
    const unsigned char* reg = phase_region(p);
    bf16x8 fa0[PSTEPS], fa1[PSTEPS];
    const int nst = p == NPH - 1 ? PSTEPS - 1 : PSTEPS;
#pragma unroll
    for (int st = 0; st < nst; ++st) {                      // all fragment reads of the phase in one go, then its MFMAs
      if constexpr (W8) {
        fa0[st] = w8frag(reg, a0_o, arow0, st);
        fa1[st] = w8frag(reg, a1_o, m1, st);
      } else {
        fa0[st] = *reinterpret_cast<const bf16x8*>(reg + a0_o + (((4 * st + g) ^ arow0) << 4));
        fa1[st] = *reinterpret_cast<const bf16x8*>(reg + a1_o + (((4 * st + g) ^ m1) << 4));
      }
    }
#pragma unroll
    for (int st = 0; st < nst; ++st) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa0[st], fb[PSTEPS * p + st], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa1[st], fb[PSTEPS * p + st], acc1, 0, 0, 0);
    }
  }

  // ---- partial tiles -> LDS (a ring region of the wavefront's own, long since consumed), then the epilogue wavefronts take over
  unsigned char* part = myring + (RING > 1 ? REGION : 0);
  *reinterpret_cast<f32x4*>(part + lane * 16) = acc0;
  *reinterpret_cast<f32x4*>(part + 1024 + lane * 16) = acc1;
  R8_STAMP(5);
  __syncthreads();
}

// Host side: pick the instantiation. xr = 8 or 16 rows per workgroup (16: fused norm only); norm = 0 / 1 (fp32 scale) / 2
// (bf16 scale); w8: fp8 weight with a.w_scale.
void launch_qkv_decode_r8(int xr, int norm, bool emb, bool w8, dim3 grid, hipStream_t st, const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr) {
  const int out4 = qkv_outputs_allow_4_byte_stores(a);
#define TLLM_R8(XRR, NORM, EMBF)                                                                                             \
  do {                                                                                                                       \
    if (w8) hipLaunchKernelGGL((qkv_decode_r8_kernel<XRR, NORM, EMBF, true>), grid, dim3(512), 0, st, a, ra, fr, out4);      \
    else hipLaunchKernelGGL((qkv_decode_r8_kernel<XRR, NORM, EMBF, false>), grid, dim3(512), 0, st, a, ra, fr, out4);        \
  } while (0)
  if (xr == 16) {
    if (emb) {
      if (norm == 1) TLLM_R8(16, 1, true);
      else TLLM_R8(16, 2, true);
    } else if (norm == 1) TLLM_R8(16, 1, false);
    else TLLM_R8(16, 2, false);
  } else if (emb) {
    if (norm == 1) TLLM_R8(8, 1, true);
    else TLLM_R8(8, 2, true);
  } else if (norm == 0) TLLM_R8(8, 0, false);
  else if (norm == 1) TLLM_R8(8, 1, false);
  else TLLM_R8(8, 2, false);
#undef TLLM_R8
}

}  // namespace tllm

extern "C" int tllm_qkv_decode_wait_expired(int32_t* expired) {
  TLLM_REQUIRE(expired != nullptr, TLLM_E_ARG, "qkv_decode_wait_expired: expired is NULL");
  int v = 0;
  const hipError_t e = hipMemcpyFromSymbol(&v, HIP_SYMBOL(tllm::g_qkv_decode_wait_expired), sizeof(v));
  TLLM_REQUIRE(e == hipSuccess, TLLM_E_LAUNCH, "qkv_decode_wait_expired: %s", hipGetErrorString(e));
  *expired = v;
  return TLLM_OK;
}

#ifdef TLLM_R8_STAMPS
extern "C" int tllm_debug_r8_stamps(void* host, size_t bytes) { return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(tllm::g_r8_stamps), bytes); }
#endif
