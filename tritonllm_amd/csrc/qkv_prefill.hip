// Prefill-size fused QKV projection + bias + rotary: an LDS-staged bf16 MFMA GEMM.
//
//   D[T, 5120] = X[T, 2880] . W[5120, 2880]^T      (both operands K-contiguous)
//
// Tiling for 256 CUs: a workgroup computes a 128-token x 320-column tile (five whole heads),
// so T = 2048 is exactly 16 x 16 = 256 tiles -- one per CU, no tail wave -- and T = 8192 is
// exactly four per CU. Eight wavefronts form a 4 x 2 grid (two per SIMD); each owns 32 x 160 of the tile as
// 1 x 5 v_mfma_f32_32x32x16_bf16 blocks (80 fp32 accumulators per lane) and reads 6 operand
// fragments from LDS per 5 MFMAs. K is walked in slices of 64 (one 128-byte line per row) through
// two LDS stages filled by direct global->LDS loads (global_load_lds_dwordx4: no staging registers,
// no ds_write). Such a load puts the 64 lanes' 16-byte chunks at consecutive LDS addresses, so rows
// cannot be padded; instead the chunk order inside each row is XOR-swizzled with the row index --
// applied by choosing which *global* chunk a lane fetches -- and the fragment reads undo it, which
// keeps the 128-bit fragment reads of 16 consecutive rows conflict-free.
// With one tile per CU nothing but the kernel's own schedule overlaps anything:
//   * the one barrier per slice sits before the slice's last k16 step; the stage just finished is handed to
//     the slice after next, whose loads go out one per MFMA behind that step and the next (never all in a row:
//     a CU's load queue is bounded and a wavefront that overflows it stalls, MFMAs included);
//   * the fragment reads of the next k16 step are pinned between the MFMAs of the current one
//     (sched_group_barrier): hoisted to the top of the iteration, as the compiler does by itself, the
//     wavefronts read a slice's fragments in one burst with no MFMA running;
//   * an L2 miss still costs more than a slice of MFMAs and LDS has no room for a third stage, so
//     three slices ahead every workgroup touches (one dword per line) its share of the lines its
//     XCD's tiles are going to need, which pulls them into that XCD's L2 in time (86 % L2 hits counted).
// Where the time goes at T = 2048 (66 us; builds with parts of the loop compiled out): the MFMAs, barriers,
// prologue and epilogue alone take 43 us (30 us of MFMAs at the 1.9 GHz this load clocks at), adding the
// fragment reads 55 us, the global->LDS loads alone (no MFMA, no fragment read) 56 us, everything 66 us. The
// loads are the wall: with two stages the loads of slice i+2 cannot start before slice i has been read by
// everyone and must have landed before slice i+1 has been, so every slice pays its 56 KB through the CU's
// 64 B/clk address unit (~900 cycles) plus an L2 round trip inside one slice's 1280 cycles of MFMAs, and a third
// stage of this tile does not fit (3 x 56 KB > 160 KB). Measured without gain: the 2 x 2 grid of 64 x 160
// wavefronts this kernel started with (70 us: one wavefront per SIMD, nothing to cover a stalled load issue),
// pairs of 64 x 160 wavefronts taking alternate k16 steps (fewer fragment reads, 68 us), four extra wavefronts that
// only load (71-75 us), K slices of 32 in a four-stage ring (77 us), a four-deep feed with two more slices in flight
// into registers and written to LDS by ds_write (70.6 us -- so the two-stage window above is not the whole story),
// other spreads of the loads over the steps and other prefetch distances (+-1 us).
// The feed itself: 256 tiles x 2.58 MB = 660 MB through the L2s in those 44 us (~15 TB/s, 7.1 M requests of 128 B);
// doubling the requests (every wavefront touching its own lines ahead of time) cost 13 %, so only fewer bytes per
// flop -- a larger tile, which T = 2048 on 256 CUs does not allow -- would lift the wall.
//
// The rotary pair (d, d+32) has to sit in one lane. The weights go on the MFMA's M side, so in
// a 32x32 block a lane owns one token and sixteen output columns (four runs of four); for a
// whole head the pair is the same register of two neighbouring blocks. 160 columns per
// wavefront are 2.5 heads; the tile's middle head is therefore split by *dims*: wavefront
// column 0 takes dims [0,16) u [32,48), column 1 takes [16,32) u [48,64), packed into one
// "mixed" block whose pair partner is sixteen rows down, i.e. register v + 8 of the same lane.
// The W rows are permuted accordingly when they are copied into LDS, which costs nothing.
//
// Epilogue: cos/sin of the tile's 128 positions x 32 frequencies are computed once per
// workgroup from the YaRN parameters into their own LDS region while the first slices are in
// flight; after the loop every lane adds the bias to its fp32 accumulators, rotates q/k pairs,
// rounds once to bf16 into an LDS image of the tile, and the image leaves as coalesced 128-bit
// stores straight into the separate q / k / v outputs (no split / contiguous copies afterwards).
#include "qkv_common.h"

namespace tllm {

namespace {
constexpr int BM = 128;            // tokens per tile
constexpr int HPT = 5;             // heads per tile
constexpr int BN = HPT * 64;       // 320 columns per tile
constexpr int BK = 64;             // K slice: one 128-byte line per row
constexpr int NS = 2;              // LDS stages
constexpr int kTouchDist = 3;      // slices of lead of the L2 warm-up
constexpr int KS = BK / 16;        // k16 MFMA steps per slice
constexpr int CHUNKS = BK / 8;     // 16-byte chunks per LDS row
constexpr int LROW = BK * 2;       // LDS row, bytes (unpadded: rows are swizzled instead)
constexpr int RPB = 1024 / LROW;   // rows per 1 KiB block (one load instruction)
constexpr int A_BYTES = BM * LROW;
constexpr int STAGE = (BM + BN) * LROW;
constexpr int OROW = BN + 4;       // epilogue staging row, elements (648 B: an odd number of 8-byte units)
constexpr int CSROW = 34;                  // float2 per row of the cos/sin table: 32 frequencies + padding, so that
                                           // lanes reading the same frequency of 32 different rows spread over the banks
constexpr int CS_BYTES = BM * CSROW * 8;   // cos/sin of (tile row, frequency) as float2
constexpr int BIAS_BYTES = BN * 4;         // the tile's bias as fp32, head-local column order
constexpr int SMEM = NS * STAGE + CS_BYTES + BIAS_BYTES;
static_assert(BM * OROW * 2 <= NS * STAGE, "the epilogue's output image reuses the stage ring");
static_assert(SMEM <= 160 * 1024, "LDS per workgroup");
constexpr int BLOCKS = STAGE / 1024;      // 1 KiB blocks per stage
static_assert(KS % 2 == 0 && BLOCKS % 8 == 0 && CHUNKS == 8 && NS == 2, "the schedule and the swizzle below are written for BK = 64, two stages");
}  // namespace

// Chunk swizzle of LDS row r: the 16-byte chunk c of the row is stored at chunk position c ^ swz(r).
// Chosen so that the 16 consecutive rows one fragment read touches land in 16 different bank groups.
__device__ __forceinline__ int swz(int r) { return (r ^ (r >> 3)) & 7; }

// LDS row i of the W tile -> (head within tile, dim within head); see the header comment.
__device__ __forceinline__ void w_tile_row(int i, int* head_local, int* dim) {
  const int w = i >= 160 ? 1 : 0;
  const int j = i - 160 * w;
  if (j < 128) {
    *head_local = 3 * w + (j >> 6);
    *dim = j & 63;
  } else {
    const int jj = j - 128;
    *head_local = 2;
    *dim = (jj < 16) ? (16 * w + jj) : (32 + 16 * w + (jj - 16));
  }
}

// WROWS wavefront rows x 2 wavefront columns: 4 x 2 (two wavefronts per SIMD, 32 x 160 each) is what is launched;
// 2 x 2 (one per SIMD, 64 x 160 each) compiles from the same source.
template <int WROWS>
__global__ __launch_bounds__(WROWS * 128) void qkv_prefill_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr, int tiles_m, int tiles_n, int swizzle) {
  constexpr int NW = WROWS * 2;             // wavefronts
  constexpr int NT = NW * 64;               // threads
  constexpr int MB = BM / (32 * WROWS);     // 32-token blocks per wavefront
  constexpr int LPW = BLOCKS / NW;          // load instructions per wavefront per stage
  constexpr int NMF = MB * 5;               // MFMAs per k16 step
  constexpr int NRD = MB + 5;               // fragment reads per k16 step
  constexpr int NL_LAST = LPW < NMF ? LPW : NMF;   // loads handed out behind a slice's last step ...
  constexpr int NL_FIRST = LPW - NL_LAST;          // ... and behind the next slice's first step
  static_assert(NL_FIRST <= NMF, "a slice's loads fit behind two k16 steps");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  // ---- tile assignment: XCD-aware. Consecutive block ids go to different XCDs (8 of them, each
  // with its own L2), so give every XCD a compact 8 x 4 super-block of tiles to maximise L2 reuse.
  int tile_m, tile_n, share_q = -1, share_p = -1;     // position inside the XCD's super-block (-1: unknown)
  {
    const int b = blockIdx.x;
    if (swizzle) {
      const int per = (tiles_m * tiles_n) >> 3;
      const int id = (b & 7) * per + (b >> 3);
      const int sb = id >> 5, in = id & 31;
      const int sbm = tiles_m >> 3;
      tile_m = (sb % sbm) * 8 + (in & 7);
      tile_n = (sb / sbm) * 4 + (in >> 3);
      share_q = in >> 3;
      share_p = in & 7;
    } else {
      tile_m = b % tiles_m;
      tile_n = b / tiles_m;
    }
  }
  const int64_t row0 = static_cast<int64_t>(tile_m) * BM;
  const int head0 = tile_n * HPT;
  const int total_heads = a.n_q_heads + 2 * a.n_kv_heads;
  const int kvec = a.hidden >> 3;
  const int n_iter = a.hidden / BK;

  // ---- loader setup. Load instruction j of wavefront w fills LDS block w*LPW + j (RPB rows of LROW bytes);
  // lane L lands at row RPB*blk + L/CHUNKS, chunk position L%CHUNKS, so it fetches global chunk (L%CHUNKS) ^ swz(row).
  // The tiles that share an XCD's L2 walk K in lockstep and four or eight of them want the same lines;
  // each starts its round of blocks at a different one so that at any moment they pull on different
  // rows (different L2 channels) instead of queueing on the same line.
  const int rot = (blockIdx.x >> 3) % LPW;
  const bf16x8* src[LPW];
  int blk_off[LPW];                                          // LDS byte offset of load j's block inside the wavefront's share
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int bj = (j + rot) % LPW;
    blk_off[j] = bj * 1024;
    const int r = (wave * LPW + bj) * RPB + lane / CHUNKS;  // LDS row: 0..127 activations, 128..447 weights
    const int c = (lane % CHUNKS) ^ swz(r);
    if (r < BM) {
      int64_t gr = row0 + r;
      if (gr >= a.rows) gr = a.rows - 1;                // clamp: valid memory, result rows are never stored
      src[j] = reinterpret_cast<const bf16x8*>(a.x) + gr * kvec + c;
    } else {
      int hl, dim;
      w_tile_row(r - BM, &hl, &dim);
      int h = head0 + hl;
      if (h >= total_heads) h = total_heads - 1;        // clamp for a ragged last tile
      src[j] = reinterpret_cast<const bf16x8*>(a.W) + (static_cast<int64_t>(h) * 64 + dim) * kvec + c;
    }
  }
  // L2 warm-up. With one tile per CU an L2 miss stalls the whole pipeline for longer than a slice of MFMAs
  // lasts, and LDS has room for only two stages of BK = 64. So three slices ahead each workgroup touches
  // (one dword per 128-byte line) its share of the lines its XCD's 32 tiles will need: a quarter of its
  // activation rows (four tiles share them) and an eighth of its weight rows (eight tiles share them) --
  // 72 lanes of one load. Nothing waits for these loads; they only pull the lines into the XCD's L2.
  // Every wavefront issues exactly one such load per slice (18 working lanes each; idle lanes and
  // unswizzled launches re-touch a line that is needed anyway), so the wait counts below are constants.
  constexpr int TPW = 72 / NW;                        // touch lanes per wavefront
  const int tch = lane < TPW ? wave * TPW + lane : 72;
  const unsigned char* touch_ptr = reinterpret_cast<const unsigned char*>(src[0]);
  if (share_q >= 0 && tch < 72) {
    if (tch < 32) {
      int64_t gr = row0 + 32 * share_q + tch;
      if (gr >= a.rows) gr = a.rows - 1;
      touch_ptr = reinterpret_cast<const unsigned char*>(a.x) + gr * a.hidden * 2;
    } else {
      int hl, dim;
      w_tile_row(40 * share_p + (tch - 32), &hl, &dim);
      int h = head0 + hl;
      if (h >= total_heads) h = total_heads - 1;
      touch_ptr = reinterpret_cast<const unsigned char*>(a.W) + (static_cast<int64_t>(h) * 64 + dim) * a.hidden * 2;
    }
  }
  // The destination register must stay reserved for as long as a touch may be in flight (the data lands
  // whenever it lands): it is threaded through every asm as read-write and consumed after the final drain.
  unsigned touch_sink = 0;
  auto issue_touch = [&](int it) {
    const int itc = it < n_iter ? it : n_iter - 1;
    asm volatile("global_load_dword %0, %1, off" : "+v"(touch_sink) : "v"(touch_ptr + itc * (BK * 2)) : "memory");
  };
  constexpr int kTouch = 1;                              // touch loads per wavefront per slice
  auto issue_loads = [&](int it) {                      // slice `it` -> stage it % NS; past the end: re-read the last slice (never consumed)
    unsigned char* dst = smem + (it % NS) * STAGE + wave * (LPW * 1024);
    const int itc = it < n_iter ? it : n_iter - 1;
#pragma unroll
    for (int j = 0; j < LPW; ++j)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[j] + itc * CHUNKS),
                                       (__attribute__((address_space(3))) void*)(dst + blk_off[j]), 16, 0, 0);
  };

  f32x16 acc[MB][5];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < 5; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mb][nb][v] = 0.f;

  // fragment addressing: byte offset of (row, chunk c) inside a stage is row*LROW + ((c ^ swz(row)) << 4)
  const int fa_row = 32 * MB * wm + l32, fb_row = BM + 160 * wn + l32;
  int fa_off[KS][MB], fb_off[KS][5];                     // [k16 step within the slice][block]
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) fa_off[kk][mb] = (fa_row + 32 * mb) * LROW + (((2 * kk + lh) ^ swz(fa_row + 32 * mb)) << 4);
#pragma unroll
    for (int nb = 0; nb < 5; ++nb) fb_off[kk][nb] = (fb_row + 32 * nb) * LROW + (((2 * kk + lh) ^ swz(fb_row + 32 * nb)) << 4);
  }
  auto load_frags = [&](const unsigned char* st, int kk, bf16x8 (&fa)[MB], bf16x8 (&fb)[5]) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) fa[mb] = *reinterpret_cast<const bf16x8*>(st + fa_off[kk][mb]);
#pragma unroll
    for (int nb = 0; nb < 5; ++nb) fb[nb] = *reinterpret_cast<const bf16x8*>(st + fb_off[kk][nb]);
  };
  auto issue_load = [&](int it, int j) {                // one load instruction of slice `it`
    unsigned char* dst = smem + (it % NS) * STAGE + wave * (LPW * 1024);
    const int itc = it < n_iter ? it : n_iter - 1;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[j] + itc * CHUNKS),
                                     (__attribute__((address_space(3))) void*)(dst + blk_off[j]), 16, 0, 0);
  };
  // One k16 step: ten MFMAs on the fragments in buffer `cur`. Behind MFMA m goes the LDS read of fragment m of
  // the next step (seven of them, into buffer cur ^ 1) and, for m < n, one global->LDS load instruction
  // (j0 + m) of slice `lit`. The interleaving is pinned with sched_group_barrier, for two reasons:
  //   * left alone, the compiler hoists all 28 fragment reads of a slice to the top of the iteration; the four
  //     wavefronts then read 112 KB from LDS in one burst (~900 cycles with no MFMA running) and do their 40
  //     MFMAs afterwards -- the two costs add up instead of overlapping;
  //   * a CU takes only so many loads into its queue and a wavefront that issues one more stalls, MFMAs
  //     included (there is one wavefront per SIMD), until the queue has drained that far; fourteen loads in a
  //     row do exactly that. Handed out one per MFMA (32 cycles) they never find the queue full.
  bf16x8 fa[2][MB], fb[2][5];
  auto read_frag = [&](int cur, const unsigned char* nst, int nkk, int i) {   // fragment i of the next step: activations first
    if (i < MB) fa[cur ^ 1][i < MB ? i : 0] = *reinterpret_cast<const bf16x8*>(nst + fa_off[nkk][i < MB ? i : 0]);
    else fb[cur ^ 1][i - MB] = *reinterpret_cast<const bf16x8*>(nst + fb_off[nkk][i - MB]);
  };
  auto step = [&](int cur, const unsigned char* nst, int nkk, int lit, int j0, int n) {
#pragma unroll
    for (int m = 0; m < NMF; ++m) {
      const int mb = m / 5, nb = m % 5;
      acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][nb], fa[cur][mb], acc[mb][nb], 0, 0, 0);   // weights on M, tokens on N
      // NRD reads over NMF MFMAs: one each (7 over 10), or two behind the first when there are more reads than MFMAs (6 over 5)
      constexpr int EXTRA = NRD > NMF ? NRD - NMF : 0;
      const int r0 = m == 0 ? 0 : m + EXTRA, nr = m == 0 ? 1 + EXTRA : (m + EXTRA < NRD ? 1 : 0);
#pragma unroll
      for (int i = 0; i < nr; ++i) read_frag(cur, nst, nkk, r0 + i);
      if (m < n) issue_load(lit, j0 + m);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // one MFMA
      if (nr == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // its LDS reads
      if (nr == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      if (m < n) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);      // one VMEM read
    }
  };

  // prologue: slices 0..NS-2 in flight, slice 0 landed
#pragma unroll
  for (int i = 0; i < NS - 1; ++i) issue_loads(i);
  // cos/sin of (tile row, frequency) for the epilogue, computed from the YaRN parameters into its own
  // LDS region while the first slices are in flight (the positions are global loads: all 16 are issued
  // before any is used).
  float2* cs_tab = reinterpret_cast<float2*>(smem + NS * STAGE);
  // the tile's 320 bias values, widened once (fetched per group inside the epilogue they were twenty dependent
  // global loads per lane, each waited for)
  float* bias_s = reinterpret_cast<float*>(smem + NS * STAGE + CS_BYTES);
  if (tid < BN) {
    int h = head0 + (tid >> 6);
    if (h >= total_heads) h = total_heads - 1;
    bias_s[tid] = a.bias ? static_cast<float>(a.bias[h * 64 + (tid & 63)]) : 0.f;
  }
  if (a.has_rope) {
    const int f = tid & 31;
    constexpr int RPP = NT / 32;                       // rows per pass
    int64_t pos[BM / RPP];
#pragma unroll
    for (int j = 0; j < BM / RPP; ++j) {
      int64_t grow = row0 + (tid >> 5) + RPP * j;
      if (grow >= a.rows) grow = a.rows - 1;
      pos[j] = rope_position_raw(ra, grow);
    }
#pragma unroll
    for (int j = 0; j < BM / RPP; ++j) {
      float c, sn;
      rope_cos_sin(ra, fr, rope_wrap(pos[j], ra.max_ctx), f, &c, &sn);
      cs_tab[((tid >> 5) + RPP * j) * CSROW + f] = make_float2(c, sn);
    }
  }
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * LPW) : "memory");
  __syncthreads();
  load_frags(smem, 0, fa[0], fb[0]);

  // Steady state: slices it+1 .. it+NS-1 are in flight or landed while slice it is multiplied. The one
  // barrier per slice sits before the slice's last k16 step; from there on the stage of slice `it` is free
  // (all reads of it have been issued) and is handed to slice it+NS, whose loads go out behind the MFMAs of
  // this last step (ten of them) and of the next slice's first step (the other four) -- a whole slice of
  // MFMAs before they are needed.
  issue_loads(NS - 1);
  issue_touch(kTouchDist);
  for (int it = 0; it < n_iter; ++it) {
    const unsigned char* st = smem + (it % NS) * STAGE;
    const unsigned char* nx = smem + ((it + 1) % NS) * STAGE;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      if (kk + 1 < KS) {
        if (kk == 0 && it > 0) {
          step(kk & 1, st, kk + 1, it + NS - 1, NL_LAST, NL_FIRST);
          issue_touch(it + kTouchDist);             // youngest in the queue: the wait below leaves it outstanding
        } else {
          step(kk & 1, st, kk + 1, 0, 0, 0);
        }
      } else {
        // Slice it+1 has landed (this wavefront's share; the touch stays in flight), then the barrier: everyone's
        // share has, and everyone has issued its last reads of slice it. Spelled out, because __syncthreads()
        // carries a fence that drains every load in flight, the look-ahead ones included.
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((NS - 2) * (LPW + kTouch) + kTouch) : "memory");
        step(kk & 1, nx, 0, it + NS, 0, NL_LAST);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(touch_sink)::"memory");   // drain the look-ahead loads before LDS is reused
  __syncthreads();
  if (touch_sink == 0x7fc12345u && tid == 1023) a.q[0] = static_cast<bf16>(0.f);   // keeps the sink register alive; never true

  // ---- epilogue -------------------------------------------------------------------------------
  // The stage ring is idle now and becomes a bf16 image of the output tile (rows padded to 656 B so the
  // two half-wavefronts of a store hit different banks). Every lane finishes its accumulators (bias,
  // rotation with the cos/sin table, one RNE) into the image; then the tile leaves as coalesced
  // 128-bit stores, eight columns of one head per lane.
  bf16* img = reinterpret_cast<bf16*>(smem);

  // Accumulator layout (weights on the MFMA's M side): the lane owns token l32 of each 32-token block and,
  // in each 32-column block, columns 8*(v>>2) + 4*lh + (v&3) -- runs of four consecutive columns, so
  // bias, cos/sin and the image stores all move in 4-element vectors. A whole head is two blocks (low
  // dims, their partners: same register index); the mixed block holds the wavefront's 16 low dims of
  // the middle head in rows 0-15 and their partners in rows 16-31 (register v and v + 8).
#pragma unroll
  for (int hp = 0; hp < 3; ++hp) {
    const int hl = (hp < 2) ? (3 * wn + hp) : 2;
    int head = head0 + hl;
    if (head >= total_heads) head = total_heads - 1;        // ragged last tile: computed, never copied out
    const bool rotate = a.has_rope && head < a.n_q_heads + a.n_kv_heads;
    const int ngrp = hp < 2 ? 4 : 2;                         // groups of four (lo, hi) pairs per lane
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (g >= ngrp) continue;
      // first of the four consecutive low dims of this group, and where its partner lives
      const int d0 = hp < 2 ? (8 * g + 4 * lh) : (16 * wn + 8 * g + 4 * lh);
      const f32x4 b_lo = *reinterpret_cast<const f32x4*>(bias_s + hl * 64 + d0);
      const f32x4 b_hi = *reinterpret_cast<const f32x4*>(bias_s + hl * 64 + 32 + d0);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int r = 32 * MB * wm + 32 * mb + l32;
        float lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (hp < 2) {
            lo[j] = acc[mb][2 * hp][4 * g + j] + b_lo[j];
            hi[j] = acc[mb][2 * hp + 1][4 * g + j] + b_hi[j];
          } else {
            lo[j] = acc[mb][4][4 * g + j] + b_lo[j];
            hi[j] = acc[mb][4][8 + 4 * g + j] + b_hi[j];
          }
        }
        bf16x4 olo, ohi;
        if (rotate) {                                      // uniform per wavefront and head
          const f32x4 c01 = *reinterpret_cast<const f32x4*>(cs_tab + r * CSROW + d0);       // (cos, sin) of dims d0, d0 + 1
          const f32x4 c23 = *reinterpret_cast<const f32x4*>(cs_tab + r * CSROW + d0 + 2);   // ... d0 + 2, d0 + 3
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float c = j < 2 ? c01[2 * j] : c23[2 * j - 4], sn = j < 2 ? c01[2 * j + 1] : c23[2 * j - 3];
            olo[j] = static_cast<bf16>(lo[j] * c - hi[j] * sn);
            ohi[j] = static_cast<bf16>(hi[j] * c + lo[j] * sn);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            olo[j] = static_cast<bf16>(lo[j]);
            ohi[j] = static_cast<bf16>(hi[j]);
          }
        }
        *reinterpret_cast<bf16x4*>(img + r * OROW + hl * 64 + d0) = olo;
        *reinterpret_cast<bf16x4*>(img + r * OROW + hl * 64 + 32 + d0) = ohi;
      }
    }
  }
  __syncthreads();

  // copy-out: chunk = 8 consecutive dims of one head of one row
  const int64_t slot_off = qkv_slot(a, ra) * a.kv_slot_stride;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(a.q) % 16 == 0) && (reinterpret_cast<uintptr_t>(a.k) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(a.v) % 16 == 0) && a.q_rs % 8 == 0 && a.k_rs % 8 == 0 && a.v_rs % 8 == 0 &&
                      a.kv_slot_stride % 8 == 0;
#pragma unroll 4
  for (int ch = tid; ch < BM * (BN / 8); ch += NT) {
    const int r = ch / (BN / 8), cc = ch - r * (BN / 8);
    const int hl = cc >> 3, d8 = (cc & 7) * 8;
    const int head = head0 + hl;
    const int64_t grow = row0 + r;
    if (head >= total_heads || grow >= a.rows) continue;
    bf16* dst;
    if (head < a.n_q_heads)
      dst = a.q + grow * a.q_rs + static_cast<int64_t>(head) * 64 + d8;
    else if (head < a.n_q_heads + a.n_kv_heads)
      dst = a.k + grow * a.k_rs + slot_off + static_cast<int64_t>(head - a.n_q_heads) * 64 + d8;
    else
      dst = a.v + grow * a.v_rs + slot_off + static_cast<int64_t>(head - a.n_q_heads - a.n_kv_heads) * 64 + d8;
    bf16x8 val;
    {
      const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(img + r * OROW + cc * 8), v1 = *reinterpret_cast<const bf16x4*>(img + r * OROW + cc * 8 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        val[e] = v0[e];
        val[4 + e] = v1[e];
      }
    }
    if (vec_ok) {
      *reinterpret_cast<bf16x8*>(dst) = val;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[e] = val[e];
    }
  }
}

}  // namespace tllm

using namespace tllm;

extern "C" int tllm_qkv_rope_prefill_bf16(const void* x, const void* W, const void* b, void* q, void* k, void* v, int64_t q_row_stride,
                                          int64_t k_row_stride, int64_t v_row_stride, int64_t kv_slot_stride, int64_t rows,
                                          int64_t hidden, int n_q_heads, int n_kv_heads, int head_dim, const TllmRope* rope,
                                          void* stream) {
  QkvArgs a;
  RopeArgs ra;
  YarnFreqs fr;
  int rc = qkv_validate("qkv_rope_prefill", x, W, q, k, v, q_row_stride, k_row_stride, v_row_stride, kv_slot_stride, rows, hidden,
                        n_q_heads, n_kv_heads, head_dim, rope, &a, &ra, &fr);
  if (rc != TLLM_OK) return rc;
  a.bias = (const bf16*)b;
  if (rows == 0) return TLLM_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool fast = head_dim == 64 && hidden % BK == 0 && aligned16(x) && aligned16(W);
  if (!fast) {
    launch_qkv_generic(a, ra, fr, st);
    return check_launch("qkv_rope_prefill(generic)");
  }
  constexpr int WROWS = 4;
  static bool attr_set = false;   // raising the dynamic-LDS limit is idempotent; a benign race at worst repeats it
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_prefill_kernel<WROWS>), hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
    TLLM_REQUIRE(e == hipSuccess, TLLM_E_LAUNCH, "qkv_rope_prefill: cannot raise LDS limit: %s", hipGetErrorString(e));
    attr_set = true;
  }
  const int heads = n_q_heads + 2 * n_kv_heads;
  const int64_t tiles_m = (rows + BM - 1) / BM;
  const int tiles_n = (heads + HPT - 1) / HPT;
  const int64_t tiles = tiles_m * tiles_n;
  TLLM_REQUIRE(tiles < (1ll << 31), TLLM_E_SHAPE, "qkv_rope_prefill: too many tiles");
  const int swizzle = (tiles_m % 8 == 0 && tiles_n % 4 == 0) ? 1 : 0;
  hipLaunchKernelGGL(qkv_prefill_kernel<WROWS>, dim3((unsigned)tiles), dim3(WROWS * 128), SMEM, st, a, ra, fr, (int)tiles_m, tiles_n, swizzle);
  return check_launch("qkv_rope_prefill");
}
