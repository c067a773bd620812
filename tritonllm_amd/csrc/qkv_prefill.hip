// Prefill-size fused QKV projection + bias + rotary: an LDS-staged bf16 MFMA GEMM.
//
//   D[T, 5120] = X[T, 2880] . W[5120, 2880]^T      (both operands K-contiguous)
//
// A workgroup of eight wavefronts computes a tile of 128 tokens x 320 columns (five whole heads), so T = 2048 is
// exactly 16 x 16 = 256 tiles -- one per CU, no tail wave; from T = 4096 up a tile is 256 tokens x 320 columns (36 %
// fewer operand bytes per flop through the L2s). Tiles are handed to the XCDs in compact 8 x 4 super-blocks (each XCD
// has its own L2). K is walked in slices of 64 (one 128-byte line per row) through LDS stage rings filled by direct
// global->LDS loads (global_load_lds_dwordx4: no staging registers, no ds_write). Such a load puts the 64 lanes'
// 16-byte chunks at consecutive LDS addresses, so rows cannot be padded; instead the chunk order inside each row is
// XOR-swizzled with the row index -- applied by choosing which *global* chunk a lane fetches -- and the fragment reads
// undo it. One hand-spelled s_waitcnt + s_barrier per slice; the loads that refill a freed stage are handed out one
// behind an MFMA at a time (a CU's load queue is bounded: a wavefront that overflows it stalls, MFMAs included), and
// the LDS reads of the next step's fragments are pinned between the MFMAs of the current one (sched_group_barrier).
//
// The 128-token tile (qkv_prefill_quads_kernel): wavefronts as 2 (tokens) x 4 (columns), 64 x 80 each, on
// v_mfma_f32_16x16x32_bf16 -- 144 operand rows read from LDS per K step and wavefront, against 192 for a 32 x 160
// wavefront. Three weight stages (40 KB) + two activation stages (16 KB): two weight slices and one activation slice
// are in flight while a slice is multiplied. Weight rows sit on the MFMA's M side: a lane owns one token of a
// 16-token block and four consecutive weight rows of a 16-row block, and the weight rows are dealt to LDS rows so that
// those four are [lo(p), lo(p+1), hi(p), hi(p+1)] of two adjacent rotation pairs (d, d + 32) -- the rotation never
// leaves the lane, and every 16-row block is laid out alike, so 80 columns (1.25 heads) need no special case.
// What the LDS wants from the fragment reads: a 128-bit read is served 16 lanes at a time, lanes 0-7 together with
// 32-39, 8-15 with 40-47 and so on; see the comment at the fragment addressing.
//
// The 256-token tile (qkv_prefill_kernel256): wavefronts as 4 x 2, 64 x 160 each, on v_mfma_f32_32x32x16_bf16 (160
// accumulators per lane leave room for single-buffered weight fragments only); two stages of each operand. 160 columns
// are 2.5 heads: the tile's middle head is split by *dims* between the two wavefront columns (column 0 takes dims
// [0,16) u [32,48), column 1 [16,32) u [48,64)), packed into one "mixed" 32-row block whose pair partner is sixteen
// rows down, i.e. register v + 8 of the same lane.
//
// Epilogue of both: cos/sin of the tile's positions x 32 frequencies come from the YaRN parameters (in the 128-token
// tile computed while the first slices are in flight and kept in registers; there is no LDS for the table next to
// the stages, it is built inside the idle ring after the K loop); every lane adds the bias to its fp32 accumulators,
// rotates q/k pairs, rounds once to bf16 into an LDS image of the tile, and the image leaves as coalesced 128-bit
// stores straight into the separate q / k / v outputs (no split / contiguous copies afterwards).
#include "qkv_common.h"

namespace tllm {

namespace {
constexpr int HPT = 5;             // heads per tile
constexpr int BN = HPT * 64;       // 320 columns per tile
constexpr int BK = 64;             // K slice: one 128-byte line per row
constexpr int XS = 2;              // LDS stages of the activations
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
                                           // lanes reading the same frequency of different rows spread over the banks
constexpr int EROWS = 128;                 // rows the epilogue finishes per pass (one pass for a 128-token tile, two for 256)
constexpr int CS_BYTES = EROWS * CSROW * 8;   // cos/sin of (row, frequency) as float2
constexpr int IMG_BYTES = (EROWS * OROW * 2 + 1023) / 1024 * 1024;   // bf16 image of a pass's rows
constexpr int BIAS_BYTES = BN * 4;         // the tile's bias as fp32, head-local column order
// Behind the ring: the bias, and (256-token tile) the rows' positions.
constexpr int prefill_smem(int bm) { return ring_bytes(bm) + BIAS_BYTES + bm * 8; }
static_assert(IMG_BYTES + CS_BYTES <= ring_bytes(128) && IMG_BYTES + CS_BYTES <= ring_bytes(256), "the epilogue reuses the stage ring");
static_assert(prefill_smem(128) <= 160 * 1024 && prefill_smem(256) <= 160 * 1024, "LDS per workgroup");
static_assert(W_STAGE % 8192 == 0 && x_stage(128) % 8192 == 0 && CHUNKS == 8 && XS == 2, "the schedules and the swizzle below are written for BK = 64");
}  // namespace

// Chunk swizzle of LDS row r: the 16-byte chunk c of the row is stored at chunk position c ^ swz(r). Eight consecutive
// rows of one chunk land on the eight chunk positions, and rows r, r + 8 on positions that differ in bit 0.
__device__ __forceinline__ int swz(int r) { return (r ^ (r >> 3)) & 7; }

// Tile of a workgroup, XCD-aware: consecutive block ids go to different XCDs (8 of them, each with its own L2), so
// every XCD gets a compact super-block of `swizzle` x (32 / swizzle) tiles (token tiles x column tiles).
__device__ __forceinline__ void prefill_tile_of_block(int b, int tiles_m, int tiles_n, int swizzle, int* tile_m, int* tile_n) {
  if (swizzle) {
    const int per = (tiles_m * tiles_n) >> 3;
    const int id = (b & 7) * per + (b >> 3);
    const int sb = id >> 5, in = id & 31;
    const int sm = swizzle, sn = 32 / swizzle;
    const int sbm = tiles_m / sm;
    *tile_m = (sb % sbm) * sm + (in % sm);
    *tile_n = (sb / sbm) * sn + (in / sm);
  } else {
    *tile_m = b % tiles_m;
    *tile_n = b / tiles_m;
  }
}

// The epilogue's last phase, shared by both tile heights: rows [pass_row0, pass_row0 + EROWS) of the tile sit in LDS as
// a bf16 image (OROW elements per row); a chunk = 8 consecutive dims of one head of one row goes out as one 128-bit store.
template <int NT>
__device__ __forceinline__ void prefill_copy_out(const QkvArgs& a, const bf16* img, int tid, int head0, int total_heads, int64_t pass_row0,
                                                 int64_t slot_off) {
  const bool vec_ok = (reinterpret_cast<uintptr_t>(a.q) % 16 == 0) && (reinterpret_cast<uintptr_t>(a.k) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(a.v) % 16 == 0) && a.q_rs % 8 == 0 && a.k_rs % 8 == 0 && a.v_rs % 8 == 0 &&
                      a.kv_slot_stride % 8 == 0;
#pragma unroll 4
  for (int ch = tid; ch < EROWS * (BN / 8); ch += NT) {
    const int r = ch / (BN / 8), cc = ch - r * (BN / 8);
    const int hl = cc >> 3, d8 = (cc & 7) * 8;
    const int head = head0 + hl;
    const int64_t grow = pass_row0 + r;
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

// ===================================================================================== the 128-token tile
// LDS row i of the W tile -> (head within tile, dim within head): block b = i / 16 (0..19) holds pairs 8 (b % 4) .. + 8
// of head b / 4; row i % 16 of the block is pair 8 (b % 4) + 2 (i16 / 4) + (i16 & 1), half (i16 >> 1) & 1.
__device__ __forceinline__ void w_tile_row_quads(int i, int* head_local, int* dim) {
  const int b = i >> 4, i16 = i & 15;
  *head_local = b >> 2;
  *dim = 8 * (b & 3) + 2 * (i16 >> 2) + (i16 & 1) + 32 * ((i16 >> 1) & 1);
}

// Unwrapped rotary positions of 16 consecutive rows starting at row g0 (the same in every lane; rows past the last one
// repeat it), read through the scalar cache: positions and offset were written before this kernel started and nothing
// writes them while it runs, and a scalar load does not involve the vector-memory counter the look-ahead loads are
// waited for with. Without a positions tensor the result is offset[0] alone and the caller adds row % tokens_per_batch.
__device__ __forceinline__ void rope_positions_16_uniform(const RopeArgs& r, const void* any_valid, int64_t g0, int64_t rows, int64_t (&pos_even)[8],
                                                          int64_t (&pos_odd)[8]) {
  typedef const int64_t __attribute__((address_space(4))) * const_i64_ptr;
  // branch-free (an absent tensor reads a valid dummy address), so that the sixteen values stay in scalar registers
  const_i64_ptr pp = reinterpret_cast<const_i64_ptr>(reinterpret_cast<uintptr_t>(r.positions ? static_cast<const void*>(r.positions) : any_valid));
  const_i64_ptr po = reinterpret_cast<const_i64_ptr>(reinterpret_cast<uintptr_t>(r.offset ? static_cast<const void*>(r.offset) : any_valid));
  const int64_t off_ld = po[0];
  const int64_t off = r.offset ? off_ld : 0;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int64_t gi = g0 + j < rows ? g0 + j : rows - 1;
    const int64_t ld = pp[r.positions ? gi : 0];
    // two arrays: a lane picks row 2 i or 2 i + 1 by a select between them (of one array the compiler makes an
    // indexed access, and the array then lives in scratch memory)
    if (j & 1) pos_odd[j >> 1] = r.positions ? ld : off;
    else pos_even[j >> 1] = r.positions ? ld : off;
  }
}

// TABLE: cos / sin come from the caller's tables (two loads per value) instead of the YaRN parameters.
template <bool TABLE>
__global__ __launch_bounds__(512) void qkv_prefill_quads_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr, int tiles_m, int tiles_n, int swizzle) {
  constexpr int BM = 128;
  constexpr int WS = w_stages(BM);          // weight stages (3)
  constexpr int XSTAGE = x_stage(BM);
  constexpr int NW = 8, NT = 512;
  constexpr int TB = BM / 2 / 16;           // 16-token blocks per wavefront (4)
  constexpr int RB = 5;                     // 16-row weight blocks per wavefront
  constexpr int KSTEPS = BK / 32;           // k32 MFMA steps per slice (2)
  constexpr int LPX = XSTAGE / 1024 / NW;   // load instructions (1 KiB blocks) per wavefront per slice: activations (2) ...
  constexpr int LPWW = W_STAGE / 1024 / NW; // ... weight (5)
  constexpr int LPW = LPX + LPWW;
  constexpr int NMF = TB * RB;              // MFMAs per k32 step (20)
  constexpr int NRD = TB + RB;              // fragment reads per k32 step (9)
  static_assert(WS == 3 && KSTEPS == 2 && 2 * LPW <= NMF && 2 * NRD <= NMF, "the schedule below: two steps per slice, reads and loads behind alternate MFMAs");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // a scalar: which operand a load belongs to is then a scalar choice
  const int wm = wave >> 2, wn = wave & 3;
  const int m16 = lane & 15, g = lane >> 4;

  int tile_m, tile_n;
  prefill_tile_of_block(blockIdx.x, tiles_m, tiles_n, swizzle, &tile_m, &tile_n);
  const int64_t row0 = static_cast<int64_t>(tile_m) * BM;
  const int head0 = tile_n * HPT;
  const int total_heads = a.n_q_heads + 2 * a.n_kv_heads;
  const int kvec = a.hidden >> 3;
  const int n_iter = a.hidden / BK;

  // ---- loader setup. A slice's activations (128 rows) and weight (320 rows) land in separate stage rings; within its
  // operand, load instruction j of wavefront w fills 1 KiB block w * n + j (RPB rows of LROW bytes); lane L lands at
  // row RPB * blk + L / CHUNKS, chunk position L % CHUNKS, so it fetches global chunk (L % CHUNKS) ^ swz(row).
  // A wavefront's loads of a period are numbered activations first (j < LPX), then weight.
  // The tiles that share an XCD's L2 walk K in lockstep and four or eight of them want the same lines; each starts
  // its round of blocks at a different one so that at any moment they pull on different rows (different L2 channels).
  const int rotx = (blockIdx.x >> 3) % LPX, rotw = (blockIdx.x >> 3) % LPWW;
  // A load's source is a scalar base (the tile's first activation row, or the weight) plus a 32-bit byte offset per lane.
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
      w_tile_row_quads(r, &hl, &dim);
      int h = head0 + hl;
      if (h >= total_heads) h = total_heads - 1;             // clamp for a ragged last tile
      soff[j] = static_cast<unsigned>(((static_cast<int64_t>(h) * 64 + dim) * kvec + c) * 16);
    }
  }
  // Period `per` = the loads that go out when slice `per` has been consumed: the activations of slice per + 2 into the
  // activation stage that slice just vacated, the weight of slice per + 3 into the weight stage it vacated.
  auto issue_load = [&](int per, int j) {
    const bool is_x = j < LPX;                            // known at compile time wherever j is
    const int sl = per + (is_x ? XS : WS);
    const int slc = sl < n_iter ? sl : n_iter - 1;        // look-ahead past the end re-reads the last slice (never used)
    unsigned char* dst = is_x ? xring + (sl % XS) * XSTAGE : wring + (sl % WS) * W_STAGE;
    // Spelled out rather than through __builtin_amdgcn_global_load_lds: this is the scalar-base form (64-bit base in
    // SGPRs, 32-bit lane offset, LDS block address in M0), where the builtin builds a 64-bit address per lane. The
    // lanes' 16 bytes land at M0 + 16 * lane; the s_nop is the wait state an M0 write needs before an LDS-DMA load reads it.
    const unsigned lds_off = static_cast<unsigned>(reinterpret_cast<uintptr_t>(dst + blk_off[j]));
    const unsigned char* sb = (is_x ? x_base : w_base) + static_cast<int64_t>(slc) * (BK * 2);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_off), "v"(soff[j]), "s"(sb) : "memory", "m0");
  };

  f32x4 acc[RB][TB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) acc[rb][tb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Fragment addressing. Lane group g = lane / 16 supplies k = 8 g .. 8 g + 7 of a k32 step; which 16-byte chunk of
  // the step's 64 bytes that is does not matter as long as both operands agree (a dot product does not care about the
  // order of its terms), and it is chosen for the LDS banks: a 128-bit read is served 16 lanes at a time, lanes
  // 0-7 together with 32-39, 8-15 with 40-47 and so on, i.e. groups g and g + 2 of eight consecutive rows. Under the
  // row swizzle those two must read chunks that differ in bit 0: group g reads chunk 4 kk + (g >> 1 | (g & 1) << 1)
  // (with chunk 4 kk + g half of all LDS cycles of this kernel were bank conflicts). With the row's swizzle that is
  // position chunk ^ swz(row), and the step enters as an XOR of bit 6 of the byte offset.
  const int gc = (g >> 1) | ((g & 1) << 1);
  int fx_o[TB], fw_o[RB];
#pragma unroll
  for (int tb = 0; tb < TB; ++tb) {
    const int r = 64 * wm + 16 * tb + m16;
    fx_o[tb] = r * LROW + ((gc ^ swz(r)) << 4);
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int r = 80 * wn + 16 * rb + m16;
    fw_o[rb] = r * LROW + ((gc ^ swz(r)) << 4);
  }
  bf16x8 fx[2][TB], fw[2][RB];
  auto read_frag = [&](int cur, const unsigned char* nstx, const unsigned char* nstw, int nkk, int i) {   // fragment i of the next step
    if (i < TB) fx[cur ^ 1][i < TB ? i : 0] = *reinterpret_cast<const bf16x8*>(nstx + (fx_o[i < TB ? i : 0] ^ (nkk << 6)));
    else fw[cur ^ 1][i - TB] = *reinterpret_cast<const bf16x8*>(nstw + (fw_o[i - TB] ^ (nkk << 6)));
  };
  // One k32 step: 20 MFMAs on the fragments in buffer `cur` (weights on M, tokens on N). Behind every even MFMA goes one
  // LDS read of the next step's fragments (into buffer cur ^ 1), behind the first n odd ones one global->LDS load of
  // period `lit`. The interleaving is pinned with sched_group_barrier: left alone, the compiler hoists all fragment
  // reads to the top of the iteration, where the wavefronts read them in one burst with no MFMA running; and a slice's
  // loads in a row overflow the CU's load queue.
  auto step = [&](int cur, const unsigned char* nstx, const unsigned char* nstw, int nkk, int lit, int n) {
#pragma unroll
    for (int m = 0; m < NMF; ++m) {
      const int rb = m / TB, tb = m % TB;
      acc[rb][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[cur][rb], fx[cur][tb], acc[rb][tb], 0, 0, 0);
      const bool rd = (m % 2 == 0) && (m / 2 < NRD);
      const bool ld = (m % 2 == 1) && (m / 2 < n);
      if (rd) read_frag(cur, nstx, nstw, nkk, m / 2);
      if (ld) issue_load(lit, m / 2);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);           // one MFMA
      if (rd) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // its LDS read
      if (ld) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // its VMEM read
    }
  };

  // ---- prologue. Nothing in it may wait for a vector load before the first slice is needed: a wait counts back from
  // the youngest load, so it would also wait for every look-ahead load issued before it. Hence: the one vector load
  // of the prologue (a bias value per thread) goes out first and is not looked at until the epilogue; the rows'
  // positions come through the scalar cache (a wavefront computes the cos/sin of 16 whole rows, so their indices are
  // uniform); then all look-ahead loads, oldest first: slice 0, weight 1, activations 1, weight 2.
  constexpr int CS_OFF = IMG_BYTES;
  constexpr int BIAS_OFF = ring_bytes(BM);
  float2* cs_tab = reinterpret_cast<float2*>(smem + CS_OFF);
  float* bias_s = reinterpret_cast<float*>(smem + BIAS_OFF);
  bf16 bias_raw;
  {
    const int c = tid < BN ? tid : BN - 1;
    int h = head0 + (c >> 6);
    if (h >= total_heads) h = total_heads - 1;
    const bf16* bp = a.bias ? a.bias : a.W;                 // absent: a valid dummy address instead of a branch around the load
    bias_raw = bp[h * 64 + (c & 63)];
  }
#pragma unroll
  for (int j = 0; j < LPW; ++j) issue_load(j < LPX ? -XS : -WS, j);
#pragma unroll
  for (int j = LPX; j < LPW; ++j) issue_load(-2, j);
#pragma unroll
  for (int j = 0; j < LPW; ++j) issue_load(-1, j);
  // cos/sin of (row, frequency) for the epilogue, computed while the first slices are in flight and kept in registers.
  // Wavefront w: rows 16 w .. 16 w + 15 of the tile; lane: frequency lane % 32, rows 16 w + 2 j + lane / 32.
  constexpr int CSN = 8;
  static_assert(NW * 2 * CSN == EROWS && EROWS == BM, "eight wavefronts x two rows x eight rounds cover the tile");
  float2 csr[CSN];
  if (TABLE || a.has_rope) {
    const int f = lane & 31;
    int64_t pos_even[CSN], pos_odd[CSN];
    rope_positions_16_uniform(ra, a.W, row0 + 16 * wave, a.rows, pos_even, pos_odd);
    // TABLE: the loads go out whether there is a rotation or not (without one they read the weight's first bytes), so
    // that the waits below can count on them, and no branch surrounds a load.
    const float* cos_t = a.has_rope ? ra.cos_table : reinterpret_cast<const float*>(a.W);
    const float* sin_t = a.has_rope ? ra.sin_table : reinterpret_cast<const float*>(a.W);
#pragma unroll
    for (int j = 0; j < CSN; ++j) {
      int64_t p = lane < 32 ? pos_even[j] : pos_odd[j];
      if (!ra.positions) {                                  // uniform
        int64_t grow = row0 + 16 * wave + 2 * j + (lane >> 5);
        if (grow >= a.rows) grow = a.rows - 1;
        p += grow < ra.tokens_per_batch ? grow : grow % ra.tokens_per_batch;
      }
      if constexpr (TABLE) {
        const int64_t at = a.has_rope ? rope_wrap(p, ra.max_ctx) * ra.table_row_stride + f : f;
        // The youngest loads of the prologue: every wait below is for older loads and so at most stricter than it
        // needs to be until these have landed, which they have by the loop's second slice.
        csr[j] = make_float2(cos_t[at], sin_t[at]);
      } else {
        float c, sn;
        yarn_cos_sin(rope_wrap(p, ra.max_ctx), fr.v[f], ra.concentration, &c, &sn);
        csr[j] = make_float2(c, sn);
      }
    }
  }
  // slice 0 has landed when only those are outstanding
  // (TABLE: the sixteen table loads are younger still and are not counted in, so this wait also takes some of the
  // look-ahead loads in -- measured: no difference -- and does not depend on how many loads the compiler makes of them)
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"((WS - 2) * LPWW + LPW) : "memory");
  __syncthreads();
#pragma unroll
  for (int tb = 0; tb < TB; ++tb) fx[0][tb] = *reinterpret_cast<const bf16x8*>(xring + fx_o[tb]);
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) fw[0][rb] = *reinterpret_cast<const bf16x8*>(wring + fw_o[rb]);

  // ---- steady state. While slice `it` is multiplied, outstanding or landed, oldest first: the weight of slice it + 1,
  // the activations of slice it + 1, the weight of slice it + 2. Step 0 of a slice reads the fragments of its step 1;
  // then the slice's one barrier (this wavefront's share of slice it + 1 has landed -- everything but the newest weight
  // slice --, then: everyone's has, and everyone has issued its last reads of slice it; spelled out, because
  // __syncthreads() carries a fence that drains every load in flight, the look-ahead ones included); step 1 reads the
  // fragments of the next slice's step 0 and hands the freed stages on.
  for (int it = 0; it < n_iter; ++it) {
    const unsigned char* stx = xring + (it % XS) * XSTAGE;
    const unsigned char* stw = wring + (it % WS) * W_STAGE;
    const unsigned char* nxx = xring + ((it + 1) % XS) * XSTAGE;
    const unsigned char* nxw = wring + ((it + 1) % WS) * W_STAGE;
    step(0, stx, stw, 1, 0, 0);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((WS - 2) * LPWW) : "memory");
    step(1, nxx, nxw, 0, it, LPW);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // drain the look-ahead loads before LDS is reused
  __syncthreads();

  // ---- epilogue: the cos/sin table and the bias into the idle ring; bias, rotation, one rounding into a bf16 image of
  // the tile (rows padded to 648 B); coalesced copy-out. The lane owns token m16 of each of its 16-token blocks and, in
  // 16-row block b = 5 wn + rb of the tile, [lo(p), lo(p+1), hi(p), hi(p+1)] of head b / 4 with p = 8 (b % 4) + 2 g.
  bf16* img = reinterpret_cast<bf16*>(smem);
  const int64_t slot_off = qkv_slot(a, ra) * a.kv_slot_stride;
  if (a.has_rope) {
#pragma unroll
    for (int j = 0; j < CSN; ++j) cs_tab[(16 * wave + 2 * j + (lane >> 5)) * CSROW + (lane & 31)] = csr[j];
  }
  if (tid < BN) bias_s[tid] = a.bias ? static_cast<float>(bias_raw) : 0.f;
  __syncthreads();
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int b = RB * wn + rb;
    const int hl = b >> 2;
    int head = head0 + hl;
    if (head >= total_heads) head = total_heads - 1;        // ragged last tile: computed, never copied out
    const bool rotate = a.has_rope && head < a.n_q_heads + a.n_kv_heads;   // uniform per wavefront and block
    const int p = 8 * (b & 3) + 2 * g;
    const float2 b_lo = *reinterpret_cast<const float2*>(bias_s + hl * 64 + p);
    const float2 b_hi = *reinterpret_cast<const float2*>(bias_s + hl * 64 + 32 + p);
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
      const int r = 64 * wm + 16 * tb + m16;
      float lo0 = acc[rb][tb][0] + b_lo.x, lo1 = acc[rb][tb][1] + b_lo.y;
      float hi0 = acc[rb][tb][2] + b_hi.x, hi1 = acc[rb][tb][3] + b_hi.y;
      if (rotate) {
        const f32x4 cs = *reinterpret_cast<const f32x4*>(cs_tab + r * CSROW + p);   // cos p, sin p, cos p+1, sin p+1
        const float r0 = lo0 * cs[0] - hi0 * cs[1], r2 = hi0 * cs[0] + lo0 * cs[1];
        const float r1 = lo1 * cs[2] - hi1 * cs[3], r3 = hi1 * cs[2] + lo1 * cs[3];
        lo0 = r0;
        lo1 = r1;
        hi0 = r2;
        hi1 = r3;
      }
      bf16x2 olo, ohi;
      olo[0] = static_cast<bf16>(lo0);
      olo[1] = static_cast<bf16>(lo1);
      ohi[0] = static_cast<bf16>(hi0);
      ohi[1] = static_cast<bf16>(hi1);
      *reinterpret_cast<bf16x2*>(img + r * OROW + hl * 64 + p) = olo;
      *reinterpret_cast<bf16x2*>(img + r * OROW + hl * 64 + 32 + p) = ohi;
    }
  }
  __syncthreads();
  prefill_copy_out<NT>(a, img, tid, head0, total_heads, row0, slot_off);
}

// ===================================================================================== the 256-token tile
// LDS row i of the W tile -> (head within tile, dim within head): wavefront column w = i / 160 holds heads 3 w, 3 w + 1
// whole (rows 0..127 of its 160) and its half of the tile's middle head (rows 128..159: 16 low dims, then their partners).
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

template <bool TABLE>
__global__ __launch_bounds__(512) void qkv_prefill_kernel256(QkvArgs a, RopeArgs ra, YarnFreqs fr, int tiles_m, int tiles_n, int swizzle) {
  constexpr int BM = 256;
  constexpr int WS = w_stages(BM);          // weight stages (2)
  constexpr int KS = BK / 16;               // k16 MFMA steps per slice
  constexpr int XSTAGE = x_stage(BM);
  constexpr int NW = 8, NT = 512;
  constexpr int MB = 2;                     // 32-token blocks per wavefront
  constexpr int LPX = XSTAGE / 1024 / NW;   // load instructions (1 KiB blocks) per wavefront per slice: activations ...
  constexpr int LPWW = W_STAGE / 1024 / NW; // ... weight
  constexpr int LPW = LPX + LPWW;           // ... together
  constexpr int NMF = MB * 5;               // MFMAs per k16 step
  constexpr int NL_LAST = LPW < NMF ? LPW : NMF;   // loads handed out behind a slice's last step ...
  constexpr int NL_FIRST = LPW - NL_LAST;          // ... and behind the next slice's first step
  static_assert(WS == 2 && NL_FIRST <= NMF && KS % 2 == 0, "a slice's loads fit behind two k16 steps");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  int tile_m, tile_n;
  prefill_tile_of_block(blockIdx.x, tiles_m, tiles_n, swizzle, &tile_m, &tile_n);
  const int64_t row0 = static_cast<int64_t>(tile_m) * BM;
  const int head0 = tile_n * HPT;
  const int total_heads = a.n_q_heads + 2 * a.n_kv_heads;
  const int kvec = a.hidden >> 3;
  const int n_iter = a.hidden / BK;

  // ---- loader setup: as in the 128-token kernel
  const int rotx = (blockIdx.x >> 3) % LPX, rotw = (blockIdx.x >> 3) % LPWW;
  const unsigned char* const x_base = reinterpret_cast<const unsigned char*>(a.x) + row0 * a.hidden * 2;
  const unsigned char* const w_base = reinterpret_cast<const unsigned char*>(a.W);
  unsigned char* const wring = smem;
  unsigned char* const xring = smem + WS * W_STAGE;
  unsigned soff[LPW];
  int blk_off[LPW];
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    if (j < LPX) {
      const int bj = wave * LPX + (j + rotx) % LPX;
      blk_off[j] = bj * 1024;
      const int r = bj * RPB + lane / CHUNKS;
      const int c = (lane % CHUNKS) ^ swz(r);
      int64_t lr = r;
      if (row0 + lr >= a.rows) lr = a.rows - 1 - row0;
      soff[j] = static_cast<unsigned>((lr * kvec + c) * 16);
    } else {
      const int bj = wave * LPWW + (j - LPX + rotw) % LPWW;
      blk_off[j] = bj * 1024;
      const int r = bj * RPB + lane / CHUNKS;
      const int c = (lane % CHUNKS) ^ swz(r);
      int hl, dim;
      w_tile_row(r, &hl, &dim);
      int h = head0 + hl;
      if (h >= total_heads) h = total_heads - 1;
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

  // fragment addressing: byte offset of (row, chunk c) inside a stage is row*LROW + ((c ^ swz(row)) << 4). The k16 step
  // kk wants chunks 2 kk + lh of the row; because a row starts on a 128-byte boundary the step enters as an XOR of bits
  // 5-6 of the byte offset: one register per 32-row block instead of one per block and step. (Lanes 0-7 and 32-39,
  // served together, read chunks 2 kk and 2 kk + 1 of eight consecutive rows: conflict-free under the swizzle.)
  const int fa_row = 32 * MB * wm + l32, fb_row = 160 * wn + l32;
  int fa_o[MB], fb_o[5];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) fa_o[mb] = (fa_row + 32 * mb) * LROW + ((lh ^ swz(fa_row + 32 * mb)) << 4);
#pragma unroll
  for (int nb = 0; nb < 5; ++nb) fb_o[nb] = (fb_row + 32 * nb) * LROW + ((lh ^ swz(fb_row + 32 * nb)) << 4);
  // Period `per`: the activations of slice per + 2 and the weight of slice per + 2 into the stages slice `per` vacated.
  auto issue_load = [&](int per, int j) {
    const bool is_x = j < LPX;
    const int sl = per + (is_x ? XS : WS);
    const int slc = sl < n_iter ? sl : n_iter - 1;
    unsigned char* dst = is_x ? xring + (sl % XS) * XSTAGE : wring + (sl % WS) * W_STAGE;
    const unsigned lds_off = static_cast<unsigned>(reinterpret_cast<uintptr_t>(dst + blk_off[j]));
    const unsigned char* sb = (is_x ? x_base : w_base) + static_cast<int64_t>(slc) * (BK * 2);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_off), "v"(soff[j]), "s"(sb) : "memory", "m0");
  };
  // One k16 step, 64 x 160 per wavefront: the two MFMAs that share a weight fragment are issued back to back and the
  // fragment is reloaded for the next step right behind them (weight fragments single-buffered: 20 registers instead of
  // 40, which is what keeps 160 accumulators + fragments inside 256 registers); the activation fragments of the next
  // step go into their second buffer behind the first two pairs; for m < n one global->LDS load (j0 + m) of period `lit`.
  bf16x8 fa[2][MB], fb[5];
  auto step = [&](int cur, const unsigned char* nstx, const unsigned char* nstw, int nkk, int lit, int j0, int n) {
#pragma unroll
    for (int nb = 0; nb < 5; ++nb) {
      acc[0][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[nb], fa[cur][0], acc[0][nb], 0, 0, 0);   // weights on M, tokens on N
      acc[1][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[nb], fa[cur][1], acc[1][nb], 0, 0, 0);
      fb[nb] = *reinterpret_cast<const bf16x8*>(nstw + (fb_o[nb] ^ (nkk << 5)));
      if (nb < 2) fa[cur ^ 1][nb] = *reinterpret_cast<const bf16x8*>(nstx + (fa_o[nb] ^ (nkk << 5)));
      if (2 * nb < n) issue_load(lit, j0 + 2 * nb);
      if (2 * nb + 1 < n) issue_load(lit, j0 + 2 * nb + 1);
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      if (nb < 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      else __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if (2 * nb + 1 < n) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
      else if (2 * nb < n) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
  };

  // prologue: slice 0 requested first; the rows' positions are parked in LDS for the epilogue (no registers to spare
  // for cos/sin values), the bias widened once; then slice 1.
  constexpr int CS_OFF = IMG_BYTES;
  constexpr int BIAS_OFF = ring_bytes(BM);
  float2* cs_tab = reinterpret_cast<float2*>(smem + CS_OFF);
  float* bias_s = reinterpret_cast<float*>(smem + BIAS_OFF);
  int64_t* pos_s = reinterpret_cast<int64_t*>(smem + BIAS_OFF + BIAS_BYTES);
#pragma unroll
  for (int j = 0; j < LPW; ++j) issue_load(-2, j);
  if (tid < BN) {
    int h = head0 + (tid >> 6);
    if (h >= total_heads) h = total_heads - 1;
    bias_s[tid] = a.bias ? static_cast<float>(a.bias[h * 64 + (tid & 63)]) : 0.f;
  }
  if (a.has_rope) {
    for (int r = tid; r < BM; r += NT) {
      int64_t grow = row0 + r;
      if (grow >= a.rows) grow = a.rows - 1;
      pos_s[r] = rope_position_raw(ra, grow);
    }
  }
#pragma unroll
  for (int j = 0; j < LPW; ++j) issue_load(-1, j);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPW) : "memory");   // slice 0 has landed when only slice 1 is outstanding
  __syncthreads();
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) fa[0][mb] = *reinterpret_cast<const bf16x8*>(xring + fa_o[mb]);
#pragma unroll
  for (int nb = 0; nb < 5; ++nb) fb[nb] = *reinterpret_cast<const bf16x8*>(wring + fb_o[nb]);

  // Steady state. The one barrier per slice sits before the slice's last k16 step; from there on the stages of slice
  // `it` are free (all reads of them have been issued) and period `it` goes out behind the MFMAs of this last step
  // and, what does not fit there, of the next slice's first step.
  for (int it = 0; it < n_iter; ++it) {
    const unsigned char* stx = xring + (it % XS) * XSTAGE;
    const unsigned char* stw = wring + (it % WS) * W_STAGE;
    const unsigned char* nxx = xring + ((it + 1) % XS) * XSTAGE;
    const unsigned char* nxw = wring + ((it + 1) % WS) * W_STAGE;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      if (kk + 1 < KS) {
        if (kk == 0 && it > 0) step(kk & 1, stx, stw, kk + 1, it - 1, NL_LAST, NL_FIRST);
        else step(kk & 1, stx, stw, kk + 1, 0, 0, 0);
      } else {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        step(kk & 1, nxx, nxw, 0, it, 0, NL_LAST);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // ---- epilogue, in two passes of 128 rows: the wavefronts that hold the pass's rows write the image, then everyone
  // copies it out. Accumulator layout: the lane owns token l32 of each 32-token block and, in each 32-column block,
  // columns 8*(v>>2) + 4*lh + (v&3) -- runs of four consecutive columns. A whole head is two blocks (low dims, their
  // partners: same register index); the mixed block holds the wavefront's 16 low dims of the middle head in rows 0-15
  // and their partners in rows 16-31 (register v and v + 8).
  bf16* img = reinterpret_cast<bf16*>(smem);
  const int64_t slot_off = qkv_slot(a, ra) * a.kv_slot_stride;
#pragma unroll
  for (int pass = 0; pass < BM / EROWS; ++pass) {
    if (pass > 0) __syncthreads();                        // the previous pass's image and table have been read
    if (a.has_rope) {
      // table rows tid / 32 + 16 j, frequency tid % 32
      const int f = tid & 31;
      int64_t pos[EROWS / 16];
#pragma unroll
      for (int j = 0; j < EROWS / 16; ++j) pos[j] = pos_s[EROWS * pass + (tid >> 5) + 16 * j];
      if constexpr (TABLE) {
        float c[EROWS / 16], sn[EROWS / 16];                   // all sixteen loads out before the first is looked at
#pragma unroll
        for (int j = 0; j < EROWS / 16; ++j) {
          const int64_t at = rope_wrap(pos[j], ra.max_ctx) * ra.table_row_stride + f;
          c[j] = ra.cos_table[at];
          sn[j] = ra.sin_table[at];
        }
#pragma unroll
        for (int j = 0; j < EROWS / 16; ++j) cs_tab[((tid >> 5) + 16 * j) * CSROW + f] = make_float2(c[j], sn[j]);
      } else {
#pragma unroll
        for (int j = 0; j < EROWS / 16; ++j) {
          float c, sn;
          yarn_cos_sin(rope_wrap(pos[j], ra.max_ctx), fr.v[f], ra.concentration, &c, &sn);
          cs_tab[((tid >> 5) + 16 * j) * CSROW + f] = make_float2(c, sn);
        }
      }
    }
    __syncthreads();
    const bool my_pass = (32 * MB * wm) / EROWS == pass;     // uniform per wavefront
#pragma unroll
    for (int hp = 0; hp < 3; ++hp) {
      if (!my_pass) break;
      const int hl = (hp < 2) ? (3 * wn + hp) : 2;
      int head = head0 + hl;
      if (head >= total_heads) head = total_heads - 1;
      const bool rotate = a.has_rope && head < a.n_q_heads + a.n_kv_heads;
      const int ngrp = hp < 2 ? 4 : 2;                         // groups of four (lo, hi) pairs per lane
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (g >= ngrp) continue;
        const int d0 = hp < 2 ? (8 * g + 4 * lh) : (16 * wn + 8 * g + 4 * lh);   // first of the four consecutive low dims
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
          if (rotate) {
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
    prefill_copy_out<NT>(a, img, tid, head0, total_heads, row0 + EROWS * pass, slot_off);
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
  // the kernels address a tile's rows and the weight with 32-bit byte offsets
  const bool fast = head_dim == 64 && hidden % BK == 0 && aligned16(x) && aligned16(W) &&
                    static_cast<int64_t>(n_q_heads + 2 * n_kv_heads) * 64 * hidden * 2 < (1ll << 32) && 256 * hidden * 2 < (1ll << 32);
  if (!fast) {
    launch_qkv_generic(a, ra, fr, st);
    return check_launch("qkv_rope_prefill(generic)");
  }
  static bool attr_set = false;   // raising the dynamic-LDS limit is idempotent; a benign race at worst repeats it
  if (!attr_set) {
    const void* k128[] = {reinterpret_cast<const void*>(qkv_prefill_quads_kernel<false>), reinterpret_cast<const void*>(qkv_prefill_quads_kernel<true>)};
    const void* k256[] = {reinterpret_cast<const void*>(qkv_prefill_kernel256<false>), reinterpret_cast<const void*>(qkv_prefill_kernel256<true>)};
    for (int t = 0; t < 2; ++t) {
      hipError_t e = hipFuncSetAttribute(k128[t], hipFuncAttributeMaxDynamicSharedMemorySize, prefill_smem(128));
      if (e == hipSuccess) e = hipFuncSetAttribute(k256[t], hipFuncAttributeMaxDynamicSharedMemorySize, prefill_smem(256));
      TLLM_REQUIRE(e == hipSuccess, TLLM_E_LAUNCH, "qkv_rope_prefill: cannot raise LDS limit: %s", hipGetErrorString(e));
    }
    attr_set = true;
  }
  const int heads = n_q_heads + 2 * n_kv_heads;
  // Tile height by a two-number cost model: a round of 128-token tiles over the 256 CUs takes ~62 us, a round of
  // 256-token tiles ~105 us (3 : 5); whichever needs less in total. T = 2048 is one round of 128s; anything that would
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
  // cos / sin from the caller's tables or, with YaRN parameters, computed in the kernel
  const bool table = !ra.use_yarn;
  const dim3 grid((unsigned)tiles), block(512);
  if (BM == 256) {
    if (table)
      hipLaunchKernelGGL(qkv_prefill_kernel256<true>, grid, block, prefill_smem(256), st, a, ra, fr, (int)tiles_m, tiles_n, swizzle);
    else
      hipLaunchKernelGGL(qkv_prefill_kernel256<false>, grid, block, prefill_smem(256), st, a, ra, fr, (int)tiles_m, tiles_n, swizzle);
  } else {
    if (table)
      hipLaunchKernelGGL(qkv_prefill_quads_kernel<true>, grid, block, prefill_smem(128), st, a, ra, fr, (int)tiles_m, tiles_n, swizzle);
    else
      hipLaunchKernelGGL(qkv_prefill_quads_kernel<false>, grid, block, prefill_smem(128), st, a, ra, fr, (int)tiles_m, tiles_n, swizzle);
  }
  return check_launch("qkv_rope_prefill");
}
