// Prefill-size fused QKV projection + bias + rotary: an LDS-staged bf16 MFMA GEMM.
//
//   D[T, 5120] = X[T, 2880] . W[5120, 2880]^T      (both operands K-contiguous)
//
// Tiling for 256 CUs: a workgroup computes a 128-token x 320-column tile (five whole heads),
// so T = 2048 is exactly 16 x 16 = 256 tiles -- one per CU, no tail wave (longer inputs take 256-token tiles, see
// the end of this comment). Eight wavefronts form a 4 x 2 grid (two per SIMD); each owns 32 x 160 of the tile as
// 1 x 5 v_mfma_f32_32x32x16_bf16 blocks (80 fp32 accumulators per lane) and reads 6 operand
// fragments from LDS per 5 MFMAs. K is walked in slices of 64 (one 128-byte line per row) through
// LDS stage rings filled by direct global->LDS loads (global_load_lds_dwordx4: no staging registers,
// no ds_write): two stages of 16 KB for the tile's activations, three of 40 KB for its weight. Such a load puts
// the 64 lanes' 16-byte chunks at consecutive LDS addresses, so rows
// cannot be padded; instead the chunk order inside each row is XOR-swizzled with the row index --
// applied by choosing which *global* chunk a lane fetches -- and the fragment reads undo it, which
// keeps the 128-bit fragment reads of 16 consecutive rows conflict-free.
// With one tile per CU nothing but the kernel's own schedule overlaps anything:
//   * the one barrier per slice sits before the slice's last k16 step; the stages just finished are handed on
//     (activations: to the slice after next; weight: to the slice three on), the loads going out one per MFMA behind
//     that step and the next (never all in a row: a CU's load queue is bounded and a wavefront that overflows it
//     stalls, MFMAs included);
//   * the fragment reads of the next k16 step are pinned between the MFMAs of the current one
//     (sched_group_barrier): hoisted to the top of the iteration, as the compiler does by itself, the
//     wavefronts read a slice's fragments in one burst with no MFMA running.
// Where the time goes at T = 2048 (builds with parts of the loop compiled out, two 56 KB stages): the MFMAs,
// barriers, prologue and epilogue alone take 43 us (30 us of MFMAs at the 1.9 GHz this load clocks at), adding the
// fragment reads 55 us, the global->LDS loads alone (no MFMA, no fragment read) 56 us, everything 64-66 us. Two things
// bound it. The feed: what a CU receives is its bytes in flight over the latency of a slice (every slice contains
// lines nobody in the XCD has touched yet, and a CU returns loads in order, so a slice completes at miss latency,
// 1.2-2 us); two symmetric stages keep one slice (56 KB) in flight, 46 GB/s per CU. The third weight stage (which
// fits once the cos/sin table no longer sits next to the stages) keeps two weight slices in flight; a probe of the
// feed with dummy MFMAs went from 59 to 46 us with it -- the kernel itself only from 64-70 to 63-68.5 us, because
// behind the feed sits the LDS: 8 wavefronts x 6 fragment reads x 4 steps x 8 clocks + 448 clocks of stage writes per
// slice are 1984 clocks against 1280 of MFMAs. Measured without gain: the 2 x 2 grid of 64 x 160
// wavefronts this kernel started with (70 us, 75 us with the three-stage ring: one wavefront per SIMD, nothing to cover
// a stalled load issue), pairs of 64 x 160 wavefronts taking alternate k16 steps (fewer fragment reads, 68 us), four
// extra wavefronts that only load (71-75 us), K slices of 32 in a four-stage ring (77 us), a four-deep feed with two
// more slices in flight into registers and written to LDS by ds_write (70.6 us), an L2 warm-up by a ninth wavefront
// (its loads sit in the same in-order queue), other spreads of the loads over the steps (+-1 us).
// From T = 4096 up there are enough tokens for 256 x 320 tiles (BM = 256: eight wavefronts of 64 x 160, 36 % fewer
// bytes per flop through the L2s): 238 -> 202-205 us at T = 8192. Its 160 accumulators leave room for
// single-buffered weight fragments only, its stages (2 x 32 KB + 2 x 40 KB) for no third weight stage, and the
// epilogue runs in two passes of 128 rows. Neither tile has LDS left for the cos/sin table next to the stages: it is
// built after the K loop inside the idle ring.
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
constexpr int HPT = 5;             // heads per tile
constexpr int BN = HPT * 64;       // 320 columns per tile
constexpr int BK = 64;             // K slice: one 128-byte line per row
constexpr int XS = 2;              // LDS stages of the activations
constexpr int KS = BK / 16;        // k16 MFMA steps per slice
constexpr int CHUNKS = BK / 8;     // 16-byte chunks per LDS row
constexpr int LROW = BK * 2;       // LDS row, bytes (unpadded: rows are swizzled instead)
constexpr int RPB = 1024 / LROW;   // rows per 1 KiB block (one load instruction)
constexpr int W_STAGE = BN * LROW;                               // one LDS stage of the weight: 320 rows of one K slice
constexpr int x_stage(int bm) { return bm * LROW; }              // ... of a bm-token tile's activations
// A 128-token tile has room for a third weight stage (3 x 40 KB + 2 x 16 KB), a 256-token tile has not (2 x 40 + 2 x 32).
constexpr int w_stages(int bm) { return bm == 128 ? 3 : 2; }
constexpr int ring_bytes(int bm) { return w_stages(bm) * W_STAGE + XS * x_stage(bm); }
constexpr int OROW = BN + 4;       // epilogue staging row, elements (648 B: an odd number of 8-byte units)
constexpr int CSROW = 34;                  // float2 per row of the cos/sin table: 32 frequencies + padding, so that
                                           // lanes reading the same frequency of 32 different rows spread over the banks
constexpr int EROWS = 128;                 // rows the epilogue finishes per pass (one pass for a 128-token tile, two for 256)
constexpr int CS_BYTES = EROWS * CSROW * 8;   // cos/sin of (row, frequency) as float2
constexpr int IMG_BYTES = (EROWS * OROW * 2 + 1023) / 1024 * 1024;   // bf16 image of a pass's rows
constexpr int BIAS_BYTES = BN * 4;         // the tile's bias as fp32, head-local column order
// The stages leave no room for the cos/sin table: it is built inside the idle stage ring after the K loop -- by a
// 128-token tile from values computed while the first slices were in flight and kept in registers, by a 256-token tile
// (no registers to spare) per pass from the rows' positions parked in LDS.
constexpr int prefill_smem(int bm) { return ring_bytes(bm) + BIAS_BYTES + bm * 8; }
static_assert(IMG_BYTES + CS_BYTES <= ring_bytes(128) && IMG_BYTES + CS_BYTES <= ring_bytes(256), "the epilogue reuses the stage ring");
static_assert(prefill_smem(128) <= 160 * 1024 && prefill_smem(256) <= 160 * 1024, "LDS per workgroup");
static_assert(KS % 2 == 0 && W_STAGE % 8192 == 0 && x_stage(128) % 8192 == 0 && CHUNKS == 8 && XS == 2,
              "the schedule and the swizzle below are written for BK = 64");
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
// BM: tokens per tile. 128 makes T = 2048 one tile per CU; 256 (from T = 4096 up) reads each weight slice for twice
// the tokens: 36 % fewer bytes per flop through the L2s, which is what bounds the 128-token tile.
template <int BM, int WROWS>
__global__ __launch_bounds__(WROWS * 128) void qkv_prefill_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr, int tiles_m, int tiles_n, int swizzle) {
  constexpr int WS = w_stages(BM);          // weight stages
  constexpr int XSTAGE = x_stage(BM);
  constexpr int NW = WROWS * 2;             // wavefronts
  constexpr int NT = NW * 64;               // threads
  constexpr int MB = BM / (32 * WROWS);     // 32-token blocks per wavefront
  constexpr int LPX = XSTAGE / 1024 / NW;   // load instructions (1 KiB blocks) per wavefront per slice: activations ...
  constexpr int LPWW = W_STAGE / 1024 / NW; // ... weight
  constexpr int LPW = LPX + LPWW;           // ... together
  constexpr int NMF = MB * 5;               // MFMAs per k16 step
  constexpr int NRD = MB + 5;               // fragment reads per k16 step
  constexpr int NL_LAST = LPW < NMF ? LPW : NMF;   // loads handed out behind a slice's last step ...
  constexpr int NL_FIRST = LPW - NL_LAST;          // ... and behind the next slice's first step
  static_assert(NL_FIRST <= NMF, "a slice's loads fit behind two k16 steps");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // a scalar: which operand a load belongs to is then a scalar choice
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  // ---- tile assignment: XCD-aware. Consecutive block ids go to different XCDs (8 of them, each
  // with its own L2), so give every XCD a compact 8 x 4 super-block of tiles to maximise L2 reuse.
  int tile_m, tile_n;
  {
    const int b = blockIdx.x;
    if (swizzle) {
      // `swizzle` = token tiles per super-block (SM); a super-block is SM x (32 / SM) tiles
      const int per = (tiles_m * tiles_n) >> 3;
      const int id = (b & 7) * per + (b >> 3);
      const int sb = id >> 5, in = id & 31;
      const int sm = swizzle, sn = 32 / swizzle;
      const int sbm = tiles_m / sm;
      tile_m = (sb % sbm) * sm + (in % sm);
      tile_n = (sb / sbm) * sn + (in / sm);
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

  // ---- loader setup. A slice's activations (BM rows) and weight (320 rows) land in separate stage rings; within its
  // operand, load instruction j of wavefront w fills 1 KiB block w * n + j (RPB rows of LROW bytes); lane L lands at
  // row RPB * blk + L / CHUNKS, chunk position L % CHUNKS, so it fetches global chunk (L % CHUNKS) ^ swz(row).
  // A wavefront's loads of a period are numbered activations first (j < LPX), then weight.
  // The tiles that share an XCD's L2 walk K in lockstep and four or eight of them want the same lines;
  // each starts its round of blocks at a different one so that at any moment they pull on different
  // rows (different L2 channels) instead of queueing on the same line.
  const int rotx = (blockIdx.x >> 3) % LPX, rotw = (blockIdx.x >> 3) % LPWW;
  // A load's source is a scalar base (the tile's first activation row, or the weight) plus a 32-bit byte offset per
  // lane: half the registers of a pointer per load, and the loads can use the scalar-base addressing form.
  const unsigned char* const x_base = reinterpret_cast<const unsigned char*>(a.x) + row0 * a.hidden * 2;
  const unsigned char* const w_base = reinterpret_cast<const unsigned char*>(a.W);
  unsigned char* const wring = smem;                         // WS stages of W_STAGE bytes
  unsigned char* const xring = smem + WS * W_STAGE;          // XS stages of XSTAGE bytes
  unsigned soff[LPW];
  int blk_off[LPW];                                          // LDS byte offset of load j's block inside its operand's stage
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    if (j < LPX) {
      const int bj = wave * LPX + (j + rotx) % LPX;
      blk_off[j] = bj * 1024;
      const int r = bj * RPB + lane / CHUNKS;                // activation row of the tile
      const int c = (lane % CHUNKS) ^ swz(r);
      int64_t lr = r;
      if (row0 + lr >= a.rows) lr = a.rows - 1 - row0;       // clamp: valid memory, result rows are never stored
      soff[j] = static_cast<unsigned>((lr * kvec + c) * 16);
    } else {
      const int bj = wave * LPWW + (j - LPX + rotw) % LPWW;
      blk_off[j] = bj * 1024;
      const int r = bj * RPB + lane / CHUNKS;                // weight row of the tile (LDS order)
      const int c = (lane % CHUNKS) ^ swz(r);
      int hl, dim;
      w_tile_row(r, &hl, &dim);
      int h = head0 + hl;
      if (h >= total_heads) h = total_heads - 1;             // clamp for a ragged last tile
      soff[j] = static_cast<unsigned>(((static_cast<int64_t>(h) * 64 + dim) * kvec + c) * 16);
    }
  }

  f32x16 acc[MB][5];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < 5; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mb][nb][v] = 0.f;

  // fragment addressing: byte offset of (row, chunk c) inside a stage is row*LROW + ((c ^ swz(row)) << 4)
  const int fa_row = 32 * MB * wm + l32, fb_row = 160 * wn + l32;   // rows inside the activation / the weight stage
  // The k16 step kk wants chunks 2 kk + lh of the row; with the row's swizzle that is position (2 kk + lh) ^ swz(row),
  // and because a row starts on a 128-byte boundary the step enters as an XOR of bits 5-6 of the byte offset: one
  // register per 32-row block instead of one per block and step.
  int fa_o[MB], fb_o[5];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) fa_o[mb] = (fa_row + 32 * mb) * LROW + ((lh ^ swz(fa_row + 32 * mb)) << 4);
#pragma unroll
  for (int nb = 0; nb < 5; ++nb) fb_o[nb] = (fb_row + 32 * nb) * LROW + ((lh ^ swz(fb_row + 32 * nb)) << 4);
  auto load_frags = [&](const unsigned char* stx, const unsigned char* stw, int kk, bf16x8 (&fa)[MB], bf16x8 (&fb)[5]) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) fa[mb] = *reinterpret_cast<const bf16x8*>(stx + (fa_o[mb] ^ (kk << 5)));
#pragma unroll
    for (int nb = 0; nb < 5; ++nb) fb[nb] = *reinterpret_cast<const bf16x8*>(stw + (fb_o[nb] ^ (kk << 5)));
  };
  // Period `per` = the loads that go out when slice `per` has been consumed: the activations of slice per + 2 into the
  // activation stage that slice just vacated, the weight of slice per + WS into the weight stage it vacated.
  auto issue_load = [&](int per, int j) {                // one load instruction of period `per`
    const bool is_x = j < LPX;                            // known at compile time wherever j is
    const int sl = per + (is_x ? XS : WS);
    const int slc = sl < n_iter ? sl : n_iter - 1;        // look-ahead past the end re-reads the last slice (never used)
    unsigned char* dst = is_x ? xring + (sl % XS) * XSTAGE : wring + (sl % WS) * W_STAGE;
    // Spelled out rather than through __builtin_amdgcn_global_load_lds: this is the scalar-base form (64-bit base in
    // SGPRs, 32-bit lane offset, LDS block address in M0), where the builtin builds a 64-bit address per lane; 14 / 13
    // fewer registers in the two tile heights and 2-3 % faster. The lanes' 16 bytes land at M0 + 16 * lane.
    const unsigned lds_off = static_cast<unsigned>(reinterpret_cast<uintptr_t>(dst + blk_off[j]));
    const unsigned char* sb = (is_x ? x_base : w_base) + static_cast<int64_t>(slc) * (BK * 2);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_off), "v"(soff[j]), "s"(sb) : "memory", "m0");
  };
  auto issue_period = [&](int per) {
#pragma unroll
    for (int j = 0; j < LPW; ++j) issue_load(per, j);
  };
  // One k16 step: NMF MFMAs on the fragments in buffer `cur`. Behind the MFMAs go the LDS reads of the next step's
  // fragments (into buffer cur ^ 1) and, for m < n, one global->LDS load instruction (j0 + m) of slice `lit`.
  // The interleaving is pinned with sched_group_barrier, for two reasons:
  //   * left alone, the compiler hoists all fragment reads of a slice to the top of the iteration; the wavefronts
  //     then read them from LDS in one burst with no MFMA running and do their MFMAs afterwards -- the two costs
  //     add up instead of overlapping;
  //   * a CU takes only so many loads into its queue and a wavefront that issues one more stalls, MFMAs
  //     included, until the queue has drained that far; a slice's loads in a row do exactly that. Handed out one
  //     per MFMA (32 cycles) they never find the queue full.
  bf16x8 fa[2][MB], fb[2][5];
  auto read_frag = [&](int cur, const unsigned char* nstx, const unsigned char* nstw, int nkk, int i) {   // fragment i of the next step: activations first
    if (i < MB) fa[cur ^ 1][i < MB ? i : 0] = *reinterpret_cast<const bf16x8*>(nstx + (fa_o[i < MB ? i : 0] ^ (nkk << 5)));
    else fb[cur ^ 1][i - MB] = *reinterpret_cast<const bf16x8*>(nstw + (fb_o[i - MB] ^ (nkk << 5)));
  };
  auto step = [&](int cur, const unsigned char* nstx, const unsigned char* nstw, int nkk, int lit, int j0, int n) {
    if constexpr (MB == 2) {
      // 64 x 160 per wavefront: the two MFMAs that share a weight fragment are issued back to back and the fragment is
      // reloaded for the next step right behind them (weight fragments single-buffered: 20 registers instead of 40, which
      // is what keeps this variant's 160 accumulators + fragments inside 256 registers); the activation fragments of the
      // next step go into their second buffer behind the first two pairs.
#pragma unroll
      for (int nb = 0; nb < 5; ++nb) {
        acc[0][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[0][nb], fa[cur][0], acc[0][nb], 0, 0, 0);
        acc[1][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[0][nb], fa[cur][1], acc[1][nb], 0, 0, 0);
        fb[0][nb] = *reinterpret_cast<const bf16x8*>(nstw + (fb_o[nb] ^ (nkk << 5)));
        if (nb < 2) fa[cur ^ 1][nb] = *reinterpret_cast<const bf16x8*>(nstx + (fa_o[nb] ^ (nkk << 5)));
        if (2 * nb < n) issue_load(lit, j0 + 2 * nb);
        if (2 * nb + 1 < n) issue_load(lit, j0 + 2 * nb + 1);
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        if (nb < 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        else __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (2 * nb + 1 < n) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
        else if (2 * nb < n) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      return;
    }
#pragma unroll
    for (int m = 0; m < NMF; ++m) {
      const int mb = m / 5, nb = m % 5;
      acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][nb], fa[cur][mb], acc[mb][nb], 0, 0, 0);   // weights on M, tokens on N
      // NRD reads over NMF MFMAs: one each (7 over 10), or two behind the first when there are more reads than MFMAs (6 over 5)
      constexpr int EXTRA = NRD > NMF ? NRD - NMF : 0;
      const int r0 = m == 0 ? 0 : m + EXTRA, nr = m == 0 ? 1 + EXTRA : (m + EXTRA < NRD ? 1 : 0);
#pragma unroll
      for (int i = 0; i < nr; ++i) read_frag(cur, nstx, nstw, nkk, r0 + i);
      if (m < n) issue_load(lit, j0 + m);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // one MFMA
      if (nr == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // its LDS reads
      if (nr == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      if (m < n) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);      // one VMEM read
    }
  };

  // prologue: slice 0 requested first (period -XS asks for activations 0, period -WS for weight 0)
#pragma unroll
  for (int j = 0; j < LPW; ++j) issue_load(j < LPX ? -XS : -WS, j);
  // cos/sin of (row, frequency) for the epilogue, computed from the YaRN parameters. There is no LDS for the table
  // next to the stages; it is built inside the idle stage ring after the K loop. A 128-token tile computes the values
  // here, while the first slices are in flight (the positions are global loads: all of them are issued before any is
  // used), and keeps them in registers until then; a 256-token tile (no registers to spare) only parks the rows'
  // positions in LDS now and computes the table after the loop, 128 rows at a time.
  constexpr bool CS_REGS = BM == EROWS;
  constexpr int CS_OFF = IMG_BYTES;
  constexpr int BIAS_OFF = ring_bytes(BM);
  float2* cs_tab = reinterpret_cast<float2*>(smem + CS_OFF);
  // the tile's 320 bias values, widened once (fetched per group inside the epilogue they were twenty dependent
  // global loads per lane, each waited for)
  float* bias_s = reinterpret_cast<float*>(smem + BIAS_OFF);
  int64_t* pos_s = reinterpret_cast<int64_t*>(smem + BIAS_OFF + BIAS_BYTES);   // 256-token tile only
  if (tid < BN) {
    int h = head0 + (tid >> 6);
    if (h >= total_heads) h = total_heads - 1;
    bias_s[tid] = a.bias ? static_cast<float>(a.bias[h * 64 + (tid & 63)]) : 0.f;
  }
  constexpr int RPP = NT / 32;                         // table rows per round of the whole workgroup
  constexpr int CSN = EROWS / RPP;                     // table entries per thread: rows tid / 32 + RPP * j, frequency tid % 32
  float2 csr[CS_REGS ? CSN : 1];
  auto compute_cs = [&](auto&& pos_of, auto&& sink) {  // pos_of(row) -> raw position; sink(j, cos, sin)
    const int f = tid & 31;
    int64_t pos[CSN];
#pragma unroll
    for (int j = 0; j < CSN; ++j) pos[j] = pos_of((tid >> 5) + RPP * j);
#pragma unroll
    for (int j = 0; j < CSN; ++j) {
      float c, sn;
      rope_cos_sin(ra, fr, rope_wrap(pos[j], ra.max_ctx), f, &c, &sn);
      sink(j, c, sn);
    }
  };
  auto store_cs = [&](int j, float c, float sn) { cs_tab[((tid >> 5) + RPP * j) * CSROW + (tid & 31)] = make_float2(c, sn); };
  if (a.has_rope) {
    if constexpr (CS_REGS) {
      compute_cs(
          [&](int r) {
            int64_t grow = row0 + r;
            if (grow >= a.rows) grow = a.rows - 1;
            return rope_position_raw(ra, grow);
          },
          [&](int j, float c, float sn) { csr[j] = make_float2(c, sn); });
    } else {
      for (int r = tid; r < BM; r += NT) {
        int64_t grow = row0 + r;
        if (grow >= a.rows) grow = a.rows - 1;
        pos_s[r] = rope_position_raw(ra, grow);
      }
    }
  }
  // The rest of the look-ahead, oldest first: (three weight stages: weight 1,) then period -1 = activations 1 and the
  // weight of slice WS - 1. Requested only now: the compiler waits for its own loads above (positions, bias) by
  // count, which would have made it wait for these as well.
  if constexpr (WS == 3) {
#pragma unroll
    for (int j = LPX; j < LPW; ++j) issue_load(-2, j);
  }
  issue_period(-1);
  // slice 0 has landed when only those are outstanding
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"((WS - 2) * LPWW + LPW) : "memory");
  __syncthreads();
  load_frags(xring, wring, 0, fa[0], fb[0]);

  // Steady state. While slice `it` is multiplied, outstanding or landed, oldest first: (three weight stages: the
  // weight of slice it + 1,) the activations of slice it + 1, the weight of slice it + WS - 1. The one barrier per
  // slice sits before the slice's last k16 step; from there on the stages of slice `it` are free (all reads of them
  // have been issued) and period `it` goes out behind the MFMAs of this last step and, what does not fit there, of the
  // next slice's first step: the activations of slice it + 2 -- a whole slice of MFMAs before they are needed -- and
  // the weight of slice it + WS -- with the third stage, two slices.
  for (int it = 0; it < n_iter; ++it) {
    const unsigned char* stx = xring + (it % XS) * XSTAGE;
    const unsigned char* stw = wring + (it % WS) * W_STAGE;
    const unsigned char* nxx = xring + ((it + 1) % XS) * XSTAGE;
    const unsigned char* nxw = wring + ((it + 1) % WS) * W_STAGE;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      if (kk + 1 < KS) {
        if (kk == 0 && it > 0) {
          step(kk & 1, stx, stw, kk + 1, it - 1, NL_LAST, NL_FIRST);
        } else {
          step(kk & 1, stx, stw, kk + 1, 0, 0, 0);
        }
      } else {
        // Slice it + 1 has landed (this wavefront's share: everything but the newest weight slice of a three-stage
        // ring), then the barrier: everyone's share has, and everyone has issued its last reads of slice it.
        // Spelled out, because __syncthreads() carries a fence that drains every load in flight, the look-ahead ones
        // included.
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((WS - 2) * LPWW) : "memory");
        step(kk & 1, nxx, nxw, 0, it, 0, NL_LAST);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // drain the look-ahead loads before LDS is reused
  __syncthreads();

  // ---- epilogue -------------------------------------------------------------------------------
  // The stage ring is idle now and becomes a bf16 image of the output tile (rows padded to 656 B so the
  // two half-wavefronts of a store hit different banks). Every lane finishes its accumulators (bias,
  // rotation with the cos/sin table, one RNE) into the image; then the tile leaves as coalesced
  // 128-bit stores, eight columns of one head per lane.
  bf16* img = reinterpret_cast<bf16*>(smem);
  const int64_t slot_off = qkv_slot(a, ra) * a.kv_slot_stride;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(a.q) % 16 == 0) && (reinterpret_cast<uintptr_t>(a.k) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(a.v) % 16 == 0) && a.q_rs % 8 == 0 && a.k_rs % 8 == 0 && a.v_rs % 8 == 0 &&
                      a.kv_slot_stride % 8 == 0;

  // Accumulator layout (weights on the MFMA's M side): the lane owns token l32 of each 32-token block and,
  // in each 32-column block, columns 8*(v>>2) + 4*lh + (v&3) -- runs of four consecutive columns, so
  // bias, cos/sin and the image stores all move in 4-element vectors. A whole head is two blocks (low
  // dims, their partners: same register index); the mixed block holds the wavefront's 16 low dims of
  // the middle head in rows 0-15 and their partners in rows 16-31 (register v and v + 8).
  // A pass finishes EROWS rows: the wavefronts that hold them write the image, then everyone copies it out.
  if constexpr (CS_REGS) {
    if (a.has_rope) {
#pragma unroll
      for (int j = 0; j < CSN; ++j) store_cs(j, csr[j].x, csr[j].y);
    }
    __syncthreads();
  }
#pragma unroll
  for (int pass = 0; pass < BM / EROWS; ++pass) {
  if constexpr (!CS_REGS) {
    if (pass > 0) __syncthreads();                        // the previous pass's image and table have been read
    if (a.has_rope) compute_cs([&](int r) { return pos_s[EROWS * pass + r]; }, store_cs);
    __syncthreads();
  }
  const bool my_pass = (32 * MB * wm) / EROWS == pass;     // uniform per wavefront
#pragma unroll
  for (int hp = 0; hp < 3; ++hp) {
    if (!my_pass) break;
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
        const int r = 32 * MB * wm + 32 * mb + l32 - EROWS * pass;   // row inside the pass
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
#pragma unroll 4
  for (int ch = tid; ch < EROWS * (BN / 8); ch += NT) {
    const int r = ch / (BN / 8), cc = ch - r * (BN / 8);
    const int hl = cc >> 3, d8 = (cc & 7) * 8;
    const int head = head0 + hl;
    const int64_t grow = row0 + EROWS * pass + r;
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
  }   // pass
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
  // the kernel addresses a tile's rows and the weight with 32-bit byte offsets
  const bool fast = head_dim == 64 && hidden % BK == 0 && aligned16(x) && aligned16(W) &&
                    static_cast<int64_t>(n_q_heads + 2 * n_kv_heads) * 64 * hidden * 2 < (1ll << 32) && 256 * hidden * 2 < (1ll << 32);
  if (!fast) {
    launch_qkv_generic(a, ra, fr, st);
    return check_launch("qkv_rope_prefill(generic)");
  }
  constexpr int WROWS = 4;
  static bool attr_set = false;   // raising the dynamic-LDS limit is idempotent; a benign race at worst repeats it
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_prefill_kernel<128, WROWS>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, prefill_smem(128));
    if (e == hipSuccess)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_prefill_kernel<256, WROWS>), hipFuncAttributeMaxDynamicSharedMemorySize,
                              prefill_smem(256));
    TLLM_REQUIRE(e == hipSuccess, TLLM_E_LAUNCH, "qkv_rope_prefill: cannot raise LDS limit: %s", hipGetErrorString(e));
    attr_set = true;
  }
  const int heads = n_q_heads + 2 * n_kv_heads;
  // Tile height by a two-number cost model: a round of 128-token tiles over the 256 CUs takes ~65 us, a round of
  // 256-token tiles ~109 us (3 : 5); whichever needs less in total. T = 2048 is one round of 128s; anything that would
  // need a second round of 128s is one round of 256s instead, T = 8192 two rounds of 256s instead of four of 128s.
  const int64_t tn = (heads + HPT - 1) / HPT;
  const int64_t rounds128 = (((rows + 127) / 128) * tn + 255) / 256, rounds256 = (((rows + 255) / 256) * tn + 255) / 256;
  const int BM = rounds256 * 5 < rounds128 * 3 ? 256 : 128;
  const int64_t tiles_m = (rows + BM - 1) / BM;
  const int tiles_n = (heads + HPT - 1) / HPT;
  const int64_t tiles = tiles_m * tiles_n;
  TLLM_REQUIRE(tiles < (1ll << 31), TLLM_E_SHAPE, "qkv_rope_prefill: too many tiles");
  // Super-block of tiles per XCD: 8 x 4 (token tiles x column tiles). Measured at T = 2048: 8 x 4 and 16 x 2 66 us,
  // 4 x 8 71 us, 2 x 16 and no grouping 75 us; from T = 4096 up (256-token tiles) the shape makes no difference.
  const int swizzle = (tiles_m % 8 == 0 && tiles_n % 4 == 0) ? 8 : 0;
  if (BM == 256)
    hipLaunchKernelGGL((qkv_prefill_kernel<256, WROWS>), dim3((unsigned)tiles), dim3(WROWS * 128), prefill_smem(256), st, a, ra, fr,
                       (int)tiles_m, tiles_n, swizzle);
  else
    hipLaunchKernelGGL((qkv_prefill_kernel<128, WROWS>), dim3((unsigned)tiles), dim3(WROWS * 128), prefill_smem(128), st, a, ra, fr,
                       (int)tiles_m, tiles_n, swizzle);
  return check_launch("qkv_rope_prefill");
}
