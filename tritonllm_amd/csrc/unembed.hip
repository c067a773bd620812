// Decode-size unembedding: logits[r, v] = sum_k x[r, k] * W[v, k] over the whole vocabulary, and its fused
// greedy-sampling form that returns argmax_v instead of the logits
// (unembedding_decode_forward triton_kernels.py:111-197, unembedding_decode_argmax_forward :305-401, the fp8-weight
// twins :200-302 and :404-512). With W = [201088, 2880] bf16 this is a 1.16 GB stream per token -- the largest
// single read of a decode step -- so the kernel is built around keeping HBM busy and nothing else:
//
//   * one workgroup of ten (eight) wavefronts per CU, alive for the whole launch; the few activation rows sit in LDS,
//     read once per workgroup;
//   * a wavefront owns whole 32-row vocabulary tiles (dealt round-robin, so every CU gets the same share +-1) and
//     walks K in steps of 64: four 1 KB loads per step, each lane fetching 16 bytes so that eight lanes cover one
//     128-byte line of one row (fully coalesced), three steps (12 KB per wavefront, 120 KB per CU) always in
//     flight, the stream running on across tile boundaries;
//   * a step's 32 x 64 block goes through a wavefront-private LDS patch into MFMA operand layout:
//     v_mfma_f32_32x32x16_bf16 with the activations on M and the vocabulary rows on N, so a lane owns one
//     vocabulary row and the logits of one batch row leave as 64-byte runs;
//   * no wavefront ever waits for another: no barrier after the prologue, no cross-wavefront reduction.
//
// ARGMAX: instead of storing logits every lane keeps the best (value, index) it has seen per batch row (fp32
// accumulator values, as the reference compares them); one shuffle reduction per wavefront at the end, one
// (value, index) pair per wavefront and batch row into a small workspace, and a second tiny kernel picks the
// winner. Ties go to the lowest index.
//
// W8: fp8 (OCP e4m3) weight with one fp32 scale per vocabulary row (triton_kernels.py:261-268): widened to bf16
// on the way into the patch, the row scale multiplies the finished sum. Half the bytes. With an even vocabulary the
// weight is streamed as pairs of rows (SR, below), whose bytes are whole cache lines.
#include <mutex>

#include "common.h"

namespace tllm {

struct UnembedArgs {
  const bf16* x;          // [rows, hidden]
  const void* W;          // [vocab, hidden] bf16, or fp8 bytes when w_scale != null
  const float* w_scale;   // [vocab] or null
  bf16* logits;           // [rows, vocab] with row stride ld (logits form)
  int64_t ld;
  float* part_max;        // [gridDim.y][gridDim.x * UNW][XR] (argmax form)
  int* part_idx;
  int64_t rows;
  int hidden, vocab;
  int pair_stores;        // the logits rows allow 4-byte stores at even columns
};

__host__ __device__ constexpr int unembed_patch(int ks) { return 32 * (ks * 2 + 16); }   // wavefront patch: 32 rows of KS bf16 + padding

__host__ __device__ constexpr int unembed_xrow(int hidden) { return hidden * 2 + 16; }   // activation row in LDS, bytes

// UNW wavefronts per workgroup and UD steps in flight: see the table at unembed_nw() below.
// SR (fp8 weight, even vocabulary): a row of fp8 is hidden bytes, 22.5 cache lines at gpt-oss's width, so that row pieces
// never line up with cache lines; two neighbouring rows together are 2 * hidden bytes -- whole lines. The weight is then
// read as [vocab / 2, 2 * hidden]: a tile is 32 such pairs (64 vocabulary rows), a step is 128 bytes = one aligned line of
// every pair (the bf16 kernel's pattern exactly, streamed with the nontemporal hint), and the bytes of a step belong to
// the pair's first row while they lie below `hidden` and to its second row from there on -- two accumulator tiles, the
// K offset into the activations chosen per MFMA. A lane ends up with the logits of rows 2p and 2p + 1: one 4-byte store,
// whole 128-byte lines per wavefront. (A bare read in this pattern: 86 us for the 580 MB; in 192-byte row pieces: 96-98.)
template <int XR, int UNW, int KS, int UD, bool W8, bool ARGMAX, bool SR = false>
__global__ __launch_bounds__(UNW * 64) void unembed_kernel(UnembedArgs a) {
  static_assert(!SR || (W8 && KS == 128), "pairs of rows: fp8 weight, 128 bytes per pair and step");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  const int xrow_b = unembed_xrow(a.hidden);
  unsigned char* xs = smem;                                   // [XR][xrow_b]
  constexpr int UPROW = KS * 2 + 16, UPATCH = unembed_patch(KS);
  unsigned char* patch = smem + XR * xrow_b + wave * UPATCH;  // this wavefront's [32][UPROW]
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * XR;
  const int nvalid = static_cast<int>(a.rows - row0 < XR ? a.rows - row0 : XR);
  const int kvec = a.hidden >> 3;                             // 16-byte chunks per activation row
  const int nsteps = SR ? 2 * a.hidden / KS : a.hidden / KS;  // K steps of a tile

  // ---- this wavefront's tiles, one per round of G = all wavefronts of the launch. Within a round the tiles go
  // wavefront index first, workgroup second: when the tiles do not divide evenly (201088 rows are 6284 tiles for 4096
  // wavefronts) the ones that take one tile more are the first wavefronts of EVERY workgroup, not all the wavefronts of
  // the first workgroups -- every CU then streams to the end of the launch.
  const int G = gridDim.x * UNW;
  // The logits of a tile leave as 64-byte runs, half a cache line: neighbouring tiles go to neighbouring wavefronts of
  // one workgroup, which reach the end of their tiles at about the same time, so that the two halves of a line meet in
  // the same L2 and leave it as one write (182.8 -> 178.9 us; four or eight neighbouring tiles per workgroup are slower,
  // 184 / 194 us: their reads then pull on the same memory pages). A pair of wavefronts (2q, 2q + 1) of all workgroups
  // covers a row of 2 * gridDim.x tiles per round; a row that the vocabulary does not fill is dealt one tile per
  // workgroup instead, so that no CU takes two tiles more than another. The argmax form stores nothing and deals singly.
  constexpr bool ADJ2 = !ARGMAX && !SR;                       // (pairs of rows leave as whole lines anyway)
  const int nwg = static_cast<int>(gridDim.x), wg = static_cast<int>(blockIdx.x);
  const int nunits = SR ? a.vocab >> 1 : a.vocab;            // rows (pairs of rows) of the weight as it is streamed
  const int ntiles = (nunits + 31) >> 5;
  auto tile_of = [&](int round) {
    const int base = round * G + (wave >> 1) * (2 * nwg);     // first tile of this wavefront pair's row
    if (ADJ2 && ntiles - base >= 2 * nwg) return base + 2 * wg + (wave & 1);
    return base + (wave & 1) * nwg + wg;
  };
  const int full_rounds = ntiles / G;                         // rounds in which every wavefront has a tile
  const int my_tiles = full_rounds + (tile_of(full_rounds) < ntiles ? 1 : 0);
  const int gw = wave * nwg + wg;                             // this wavefront's number (its slot in the argmax workspace)
  const int total = my_tiles * nsteps;                        // steps of the whole stream

  // One load instruction moves 1 KB; the 32 x (KS elements) block of a step is dealt to the lanes as 16-byte
  // chunks in row-major order, so consecutive lanes cover consecutive bytes of a row (KS = 64: eight lanes per
  // 128-byte line; KS = 192: 24 lanes per 384-byte run).
  constexpr int CPS = (W8 ? KS : KS * 2) / 16;                // 16-byte chunks per row per step, as the weight lies in memory
  constexpr int LPS = 32 * CPS / 64;                          // load instructions per step
  const int64_t wrow_vec = (W8 && !SR) ? (a.hidden >> 4) : (a.hidden >> 3);   // 16-byte chunks per weight row (pair of rows)
  const bf16x8* wv = reinterpret_cast<const bf16x8*>(a.W);
  auto row_base = [&](int tile, int i) -> const bf16x8* {    // first chunk this lane fetches of load i in tile `tile`
    const int c = i * 64 + lane;
    int v = tile * 32 + c / CPS;
    v = v < nunits ? v : nunits - 1;                          // ragged last tile: repeat the last row (never stored)
    return wv + static_cast<int64_t>(v) * wrow_vec + (c % CPS);
  };

  bf16x8 buf[UD][LPS];
  const bf16x8* lp[LPS];                                      // load cursor: row bases of the tile being requested
  int l_round = 0, l_tile = tile_of(0), l_step = 0, l_count = 0;
#pragma unroll
  for (int i = 0; i < LPS; ++i) lp[i] = row_base(my_tiles > 0 ? l_tile : 0, i);
  // Unconditional on purpose (a load under a branch makes the compiler wait for it where the paths join): past
  // the end of the stream the cursor simply stays on the last step and re-requests it.
  auto issue = [&](int d) {                                   // request the next step of the stream into buf[d]
#pragma unroll
    for (int i = 0; i < LPS; ++i) {
      // fp8 rows are 22.5 lines long, so a step's row pieces share lines with the next step's: read through the cache
      // they are fetched from HBM once (FETCH_SIZE 601 MB for 580 MB of weight; with the streaming hint 730 MB)
      if constexpr (W8 && !SR) buf[d][i] = lp[i][l_step * CPS];
      else buf[d][i] = __builtin_nontemporal_load(lp[i] + l_step * CPS);
    }
    if (l_count + 1 < total) {
      ++l_count;
      if (++l_step == nsteps) {
        l_step = 0;
        l_tile = tile_of(++l_round);
#pragma unroll
        for (int i = 0; i < LPS; ++i) lp[i] = row_base(l_tile < ntiles ? l_tile : ntiles - 1, i);
      }
    }
  };
#pragma unroll
  for (int d = 0; d < UD; ++d) issue(d);

  // ---- the activation rows into LDS (rows past the end repeat the last one; never stored), behind the first weight
  // requests: those take the longest to come back, and the first multiply needs both
  for (int c = tid; c < XR * kvec; c += UNW * 64) {
    int r = c / kvec;
    const int kc = c - r * kvec;
    const int rs = r < nvalid ? r : nvalid - 1;
    *reinterpret_cast<bf16x8*>(xs + r * xrow_b + kc * 16) = reinterpret_cast<const bf16x8*>(a.x)[(row0 + rs) * kvec + kc];
  }
  __syncthreads();

  f32x16 acc, acc2;                                           // acc2 (SR): the pair's second row
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = acc2[v] = 0.f;
  constexpr int NB = XR / 2;                                  // accumulator registers that carry batch rows: row(v) = 8*(v>>2) + 4*h + (v&3)
  float best[NB];
  int best_i[NB];
#pragma unroll
  for (int v = 0; v < NB; ++v) {
    best[v] = -3.0e38f;
    best_i[v] = 0x7fffffff;
  }

  const unsigned char* xfrag = xs + (m & (XR - 1)) * xrow_b + h * 16;   // activations on M: tile rows >= XR repeat, never stored
  const unsigned char* wfrag = patch + m * UPROW + h * 16;              // vocabulary rows on N
  int c_round = 0, c_tile = tile_of(0), c_step = 0;
  for (int g0 = 0; g0 < total; g0 += UD) {
#pragma unroll
    for (int d = 0; d < UD; ++d) {
      if (g0 + d < total) {                                   // uniform
        // step (c_tile, c_step) is in buf[d]: into the patch, then KS / 16 MFMAs
#pragma unroll
        for (int i = 0; i < LPS; ++i) {
          const int r = (i * 64 + lane) / CPS, kc = (i * 64 + lane) % CPS;
          if constexpr (W8) {
            typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;
            const u32x4 raw = __builtin_bit_cast(u32x4, buf[d][i]);                    // sixteen fp8
            *reinterpret_cast<bf16x8*>(patch + r * UPROW + kc * 32) = fp8x8_to_bf16x8(raw[0], raw[1]);
            *reinterpret_cast<bf16x8*>(patch + r * UPROW + kc * 32 + 16) = fp8x8_to_bf16x8(raw[2], raw[3]);
          } else {
            *reinterpret_cast<bf16x8*>(patch + r * UPROW + kc * 16) = buf[d][i];
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if constexpr (SR) {
          const int kb0 = c_step * KS;                        // the step's first byte inside the pair = K of the first row
          // One branch per step, not per MFMA: inside a case the sixteen fragment reads go out together.
          if (kb0 + KS <= a.hidden) {                         // uniform: the whole step belongs to the first row
#pragma unroll
            for (int t = 0; t < KS / 16; ++t) {
              const bf16x8 fa = *reinterpret_cast<const bf16x8*>(xfrag + (kb0 + 16 * t) * 2);
              const bf16x8 fb = *reinterpret_cast<const bf16x8*>(wfrag + t * 32);
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
            }
          } else if (kb0 >= a.hidden) {                       // ... to the second row
#pragma unroll
            for (int t = 0; t < KS / 16; ++t) {
              const bf16x8 fa = *reinterpret_cast<const bf16x8*>(xfrag + (kb0 - a.hidden + 16 * t) * 2);
              const bf16x8 fb = *reinterpret_cast<const bf16x8*>(wfrag + t * 32);
              acc2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc2, 0, 0, 0);
            }
          } else {                                            // the step in which the first row ends (hidden is a multiple of 16: no MFMA straddles)
#pragma unroll
            for (int t = 0; t < KS / 16; ++t) {
              const int kb = kb0 + 16 * t;
              const bf16x8 fb = *reinterpret_cast<const bf16x8*>(wfrag + t * 32);
              if (kb < a.hidden) {
                const bf16x8 fa = *reinterpret_cast<const bf16x8*>(xfrag + kb * 2);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
              } else {
                const bf16x8 fa = *reinterpret_cast<const bf16x8*>(xfrag + (kb - a.hidden) * 2);
                acc2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc2, 0, 0, 0);
              }
            }
          }
        } else {
#pragma unroll
          for (int t = 0; t < KS / 16; ++t) {
            const bf16x8 fa = *reinterpret_cast<const bf16x8*>(xfrag + c_step * (KS * 2) + t * 32);
            const bf16x8 fb = *reinterpret_cast<const bf16x8*>(wfrag + t * 32);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (SR && ++c_step == nsteps) {                       // tile finished: lane owns vocabulary rows 2 p and 2 p + 1, p = c_tile*32 + m
          const int v0 = 2 * (c_tile * 32 + m), v1 = v0 + 1;  // the vocabulary is even here: both are inside it, or neither
          const float sc0 = a.w_scale[v0 < a.vocab ? v0 : a.vocab - 2], sc1 = a.w_scale[v1 < a.vocab ? v1 : a.vocab - 1];
#pragma unroll
          for (int r = 0; r < NB; ++r) {
            const int brow = 8 * (r >> 2) + 4 * h + (r & 3);
            const float val0 = acc[r] * sc0, val1 = acc2[r] * sc1;
            if constexpr (ARGMAX) {
              if (v0 < a.vocab && val0 > best[r]) {           // ascending order: '>' keeps the lowest index
                best[r] = val0;
                best_i[r] = v0;
              }
              if (v0 < a.vocab && val1 > best[r]) {
                best[r] = val1;
                best_i[r] = v1;
              }
            } else if (v0 < a.vocab && brow < nvalid) {
              bf16* lrow = a.logits + (row0 + brow) * a.ld + v0;
              if (a.pair_stores) {
                bf16x2 pr;
                pr[0] = static_cast<bf16>(val0);
                pr[1] = static_cast<bf16>(val1);
                *reinterpret_cast<bf16x2*>(lrow) = pr;
              } else {
                lrow[0] = static_cast<bf16>(val0);
                lrow[1] = static_cast<bf16>(val1);
              }
            }
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = acc2[r] = 0.f;
          c_step = 0;
          c_tile = tile_of(++c_round);
        }
        if (!SR && ++c_step == nsteps) {                      // tile finished: lane owns vocabulary row c_tile*32 + m
          const int v = c_tile * 32 + m;
          float sc = 1.f;
          if constexpr (W8) sc = a.w_scale[v < a.vocab ? v : a.vocab - 1];
#pragma unroll
          for (int r = 0; r < NB; ++r) {
            const int brow = 8 * (r >> 2) + 4 * h + (r & 3);
            const float val = acc[r] * sc;
            if constexpr (ARGMAX) {
              if (v < a.vocab && val > best[r]) {             // tiles come in ascending order: '>' keeps the lowest index
                best[r] = val;
                best_i[r] = v;
              }
            } else {
              if (v < a.vocab && brow < nvalid) a.logits[(row0 + brow) * a.ld + v] = static_cast<bf16>(val);
            }
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = 0.f;
          c_step = 0;
          c_tile = tile_of(++c_round);
        }
      }
      // buf[d] is free again: the step UD ahead. Outside the branch above, so that every path through the loop
      // issues the same loads and the compiler's waits can count on all UD steps being in flight (with the request
      // inside the branch it has to assume that the steps before this one were skipped, and every UD-th step waited
      // for everything in flight).
      issue(d);
    }
  }

  if constexpr (ARGMAX) {
    // best of the wavefront per batch row: the 32 lanes of a half hold the same batch rows, different vocabulary rows
#pragma unroll
    for (int r = 0; r < NB; ++r) {
      float bv = best[r];
      int bi = best_i[r];
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ov > bv || (ov == bv && oi < bi)) {
          bv = ov;
          bi = oi;
        }
      }
      if (m == 0) {
        const int brow = 8 * (r >> 2) + 4 * h + (r & 3);
        const int64_t slot = (static_cast<int64_t>(blockIdx.y) * G + gw) * XR + brow;
        a.part_max[slot] = bv;
        a.part_idx[slot] = bi;
      }
    }
  }
}

// Thirty-two batch rows per workgroup (bf16 or fp8 weight): 32 activation rows of gpt-oss's width are 184 KB, more than the
// LDS holds, and chunks of sixteen stream the weight once per chunk. Here the workgroup keeps one K half of its 32
// rows in LDS at a time: every wavefront first walks the first half of K for ALL its tiles, the partial sums of a
// tile waiting in registers (a wavefront owns at most MT tiles: the host checks), then the workgroup swaps the other
// half of the rows in and the wavefronts walk their tiles again over the second half and store. The weight is still
// read exactly once -- a row as two contiguous, line-aligned pieces at different times -- and a tile's sum runs over
// K in the same order as in one pass. The rest is unembed_kernel: coalesced 1 KB loads, UD steps in flight, the
// wavefront-private patch into operand layout, v_mfma_f32_32x32x16_bf16 with all 32 M rows real, tiles dealt in pairs
// to neighbouring wavefronts. The accumulators of the waiting tiles sit in a queue of registers that is rotated at
// the end of each tile half, so every access is to a fixed register.
template <int UNW, int KS, int UD, bool W8, bool ARGMAX>
__global__ __launch_bounds__(UNW * 64) void unembed_rows32_kernel(UnembedArgs a) {
  constexpr int XR = 32, MT = 4;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  const int nsteps = a.hidden / KS;                           // K steps of a tile
  const int nA = nsteps >> 1, nB = nsteps - nA;               // ... of its two halves
  const int xrow_b = nB * (KS * 2) + 16;                      // activation row (the longer half) in LDS, bytes
  unsigned char* xs = smem;                                   // [XR][xrow_b]
  constexpr int UPROW = KS * 2 + 16, UPATCH = unembed_patch(KS);
  unsigned char* patch = smem + XR * xrow_b + wave * UPATCH;  // this wavefront's [32][UPROW]
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * XR;
  const int nvalid = static_cast<int>(a.rows - row0 < XR ? a.rows - row0 : XR);
  const int kvec = a.hidden >> 3;                             // 16-byte chunks per activation row

  // tiles: as in unembed_kernel (pairs of neighbouring tiles to neighbouring wavefronts of a workgroup, the last,
  // partly filled row of tiles dealt one per workgroup)
  const int G = gridDim.x * UNW;
  constexpr bool ADJ2 = !ARGMAX;
  const int nwg = static_cast<int>(gridDim.x), wg = static_cast<int>(blockIdx.x);
  const int ntiles = (a.vocab + 31) >> 5;
  auto tile_of = [&](int round) {
    const int base = round * G + (wave >> 1) * (2 * nwg);
    if (ADJ2 && ntiles - base >= 2 * nwg) return base + 2 * wg + (wave & 1);
    return base + (wave & 1) * nwg + wg;
  };
  const int full_rounds = ntiles / G;
  const int my_tiles = full_rounds + (tile_of(full_rounds) < ntiles ? 1 : 0);   // <= MT (checked on the host)
  const int gw = wave * nwg + wg;

  constexpr int CPS = (W8 ? KS : KS * 2) / 16;                // 16-byte chunks per row per step, as the weight lies in memory
  constexpr int LPS = 32 * CPS / 64;                          // load instructions per step
  const int64_t wrow_vec = W8 ? (a.hidden >> 4) : (a.hidden >> 3);   // 16-byte chunks per weight row
  const bf16x8* wv = reinterpret_cast<const bf16x8*>(a.W);
  auto row_base = [&](int tile, int i) -> const bf16x8* {
    const int c = i * 64 + lane;
    int v = tile * 32 + c / CPS;
    v = v < a.vocab ? v : a.vocab - 1;                        // ragged last tile: repeat the last row (never stored)
    return wv + static_cast<int64_t>(v) * wrow_vec + (c % CPS);
  };

  f32x16 acc, q0, q1, q2;                                     // the tile being multiplied, and the tiles that wait
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = q0[v] = q1[v] = q2[v] = 0.f;
  static_assert(MT == 4, "the queue below holds three waiting tiles");
  auto rotate = [&]() {                                       // the next tile's accumulator to the front, this one to the back
    if (my_tiles == 4) {
      const f32x16 t = acc; acc = q0; q0 = q1; q1 = q2; q2 = t;
    } else if (my_tiles == 3) {
      const f32x16 t = acc; acc = q0; q0 = q1; q1 = t;
    } else if (my_tiles == 2) {
      const f32x16 t = acc; acc = q0; q0 = t;
    }
  };
  float best[16];
  int best_i[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    best[v] = -3.0e38f;
    best_i[v] = 0x7fffffff;
  }
  const unsigned char* xfrag = xs + m * xrow_b + h * 16;      // activations on M
  const unsigned char* wfrag = patch + m * UPROW + h * 16;    // vocabulary rows on N

  for (int half = 0; half < 2; ++half) {
    const int s_lo = half ? nA : 0, s_n = half ? nB : nA;     // this half's steps of a tile: s_lo .. s_lo + s_n - 1
    const int total = my_tiles * s_n;                         // steps of this half's stream

    bf16x8 buf[UD][LPS];
    const bf16x8* lp[LPS];
    int l_round = 0, l_tile = tile_of(0), l_step = 0, l_count = 0;
#pragma unroll
    for (int i = 0; i < LPS; ++i) lp[i] = row_base(my_tiles > 0 ? l_tile : 0, i);
    auto issue = [&](int d) {                                 // unconditional: past the end the cursor stays on the last step
#pragma unroll
      for (int i = 0; i < LPS; ++i) {
        // (fp8 rows are 22.5 lines long, so a step's row pieces share lines with the next step's: read through the cache)
        if constexpr (W8) buf[d][i] = lp[i][(s_lo + l_step) * CPS];
        else buf[d][i] = __builtin_nontemporal_load(lp[i] + (s_lo + l_step) * CPS);
      }
      if (l_count + 1 < total) {
        ++l_count;
        if (++l_step == s_n) {
          l_step = 0;
          l_tile = tile_of(++l_round);
#pragma unroll
          for (int i = 0; i < LPS; ++i) lp[i] = row_base(l_tile < ntiles ? l_tile : ntiles - 1, i);
        }
      }
    };
#pragma unroll
    for (int d = 0; d < UD; ++d) issue(d);

    // ---- this half of the activation rows into LDS, behind the first weight requests (rows past the end repeat the
    // last one; never stored). The second time round every wavefront has left its first half behind it.
    if (half) __syncthreads();
    const int hvec = s_n * (KS / 8), hoff = s_lo * (KS / 8);  // 16-byte chunks of the half, its first chunk in the row
    for (int c = tid; c < XR * hvec; c += UNW * 64) {
      const int r = c / hvec, kc = c - r * hvec;
      const int rs = r < nvalid ? r : nvalid - 1;
      *reinterpret_cast<bf16x8*>(xs + r * xrow_b + kc * 16) = reinterpret_cast<const bf16x8*>(a.x)[(row0 + rs) * kvec + hoff + kc];
    }
    __syncthreads();

    int c_round = 0, c_tile = tile_of(0), c_step = 0;
    for (int g0 = 0; g0 < total; g0 += UD) {
#pragma unroll
      for (int d = 0; d < UD; ++d) {
        if (g0 + d < total) {                                 // uniform
#pragma unroll
          for (int i = 0; i < LPS; ++i) {
            const int r = (i * 64 + lane) / CPS, kc = (i * 64 + lane) % CPS;
            if constexpr (W8) {
              typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;
              const u32x4 raw = __builtin_bit_cast(u32x4, buf[d][i]);                  // sixteen fp8
              *reinterpret_cast<bf16x8*>(patch + r * UPROW + kc * 32) = fp8x8_to_bf16x8(raw[0], raw[1]);
              *reinterpret_cast<bf16x8*>(patch + r * UPROW + kc * 32 + 16) = fp8x8_to_bf16x8(raw[2], raw[3]);
            } else {
              *reinterpret_cast<bf16x8*>(patch + r * UPROW + kc * 16) = buf[d][i];
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int t = 0; t < KS / 16; ++t) {
            const bf16x8 fa = *reinterpret_cast<const bf16x8*>(xfrag + c_step * (KS * 2) + t * 32);
            const bf16x8 fb = *reinterpret_cast<const bf16x8*>(wfrag + t * 32);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          if (++c_step == s_n) {                              // this half of the tile is finished
            if (half) {                                       // ... and with it the tile: lane owns vocabulary row c_tile*32 + m
              const int v = c_tile * 32 + m;
              float sc = 1.f;
              if constexpr (W8) sc = a.w_scale[v < a.vocab ? v : a.vocab - 1];
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int brow = 8 * (r >> 2) + 4 * h + (r & 3);
                const float val = acc[r] * sc;
                if constexpr (ARGMAX) {
                  if (v < a.vocab && val > best[r]) {         // tiles come in ascending order: '>' keeps the lowest index
                    best[r] = val;
                    best_i[r] = v;
                  }
                } else {
                  if (v < a.vocab && brow < nvalid) a.logits[(row0 + brow) * a.ld + v] = static_cast<bf16>(val);
                }
              }
            }
            rotate();
            c_step = 0;
            c_tile = tile_of(++c_round);
          }
        }
        issue(d);
      }
    }
  }

  if constexpr (ARGMAX) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float bv = best[r];
      int bi = best_i[r];
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ov > bv || (ov == bv && oi < bi)) {
          bv = ov;
          bi = oi;
        }
      }
      if (m == 0) {
        const int brow = 8 * (r >> 2) + 4 * h + (r & 3);
        const int64_t slot = (static_cast<int64_t>(blockIdx.y) * G + gw) * XR + brow;
        a.part_max[slot] = bv;
        a.part_idx[slot] = bi;
      }
    }
  }
}

// One workgroup per batch row: the winner among the per-wavefront candidates (at most 4096). Lowest index wins a tie.
// A candidate becomes one 64-bit key -- the value's bits made monotonic in the upper word, the complement of its index
// in the lower -- so that the winner is a plain maximum. Every thread requests its (up to four) candidates before it
// looks at any; wavefront maximum through DPP operands and scalar lane reads, sixteen wavefront results through LDS.
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long k) {
  auto dpp = [](unsigned x, auto ctrl) {
    return static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), decltype(ctrl)::value, 0xf, 0xf, true));
  };
  auto step = [&](auto ctrl) {
    const unsigned long long o = (static_cast<unsigned long long>(dpp(static_cast<unsigned>(k >> 32), ctrl)) << 32) | dpp(static_cast<unsigned>(k), ctrl);
    k = o > k ? o : k;
  };
  step(std::integral_constant<int, 0xB1>{});               // quad_perm [1, 0, 3, 2]
  step(std::integral_constant<int, 0x4E>{});               // quad_perm [2, 3, 0, 1]
  step(std::integral_constant<int, 0x141>{});              // row_half_mirror
  step(std::integral_constant<int, 0x140>{});              // row_mirror: every lane of a row of 16 now holds the row's maximum
  unsigned long long best = 0;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(k >> 32), 16 * r));
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(k), 16 * r));
    const unsigned long long o = (static_cast<unsigned long long>(hi) << 32) | lo;
    best = o > best ? o : best;
  }
  return best;
}

constexpr int kArgmaxReduceThreads = 1024;

__global__ __launch_bounds__(kArgmaxReduceThreads) void unembed_argmax_reduce_kernel(const float* part_max, const int* part_idx, int* token_ids,
                                                                                     int n_part, int xr) {
  __shared__ unsigned long long s_k[kArgmaxReduceThreads / 64];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int chunk = row / xr, brow = row - chunk * xr;
  constexpr int PER = 4;                                    // n_part <= 4096
  float v[PER];
  int idx[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int p = tid + j * kArgmaxReduceThreads;
    const int64_t slot = (static_cast<int64_t>(chunk) * n_part + (p < n_part ? p : n_part - 1)) * xr + brow;
    v[j] = part_max[slot];
    idx[j] = part_idx[slot];
  }
  unsigned long long k = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const unsigned b = __float_as_uint(v[j] + 0.0f);        // -0 + 0 = +0: the two zeros compare equal, so they must make one key
    const unsigned mono = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    const unsigned long long o = (static_cast<unsigned long long>(mono) << 32) | static_cast<unsigned>(~idx[j]);
    k = (tid + j * kArgmaxReduceThreads < n_part && o > k) ? o : k;
  }
  k = wave_max_u64(k);
  if ((tid & 63) == 0) s_k[tid >> 6] = k;
  __syncthreads();
  if (tid < 64) {
    k = wave_max_u64(tid < kArgmaxReduceThreads / 64 ? s_k[tid] : 0ull);
    if (tid == 0) token_ids[row] = static_cast<int>(~static_cast<unsigned>(k));
  }
}

}  // namespace tllm

using namespace tllm;

namespace {
constexpr int kUnembedGrid = 256;      // one workgroup per CU

int unembed_xr_most(int64_t rows) { return rows <= 8 ? 8 : 16; }

// (wavefronts, K step, steps in flight), measured at B = 8 on the full vocabulary:
//   bf16, up to 8 rows : 10 wavefronts, K step 64 (whole 128-byte lines), 3 in flight   174.5 us (8 x 3: 175.1, 12 x 2: 175.4,
//                         16 x 4: 177.5, 10 x 2: 176.5, 8 x 192-element steps x 2: 182.8; the K step must divide hidden)
//   fp8,  up to 8 rows :  even vocabulary: pairs of rows, 8 wavefronts, 128 bytes per pair and step, 2 in flight   99 us
//                         odd vocabulary: 8 wavefronts, K step 192, 2 in flight           113 us (16 x 64 x 4: 124)
//   16 rows            :  8 wavefronts (LDS holds the 16 activation rows), K step 64, 3 in flight (bf16: 183.4 us; 4: 185.3, 2: 188.7)
//   fp8, 9-16 rows     :  even vocabulary: pairs of rows with the six wavefronts the LDS has room for, 2 in flight
//                         (9 / 16 rows: 116.7 / 120.8 us; K step 64 with eight wavefronts: 121.8 / 128.0)
// K steps that split 128-byte lines (96 elements of bf16, 32) cost 25-50 %.
int unembed_nw(int xr, bool w8) { return (xr == 8 && !w8) ? 10 : 8; }
int unembed_ks(int xr, bool w8, int64_t hidden) { return (xr == 8 && w8 && hidden % 192 == 0) ? 192 : 64; }
size_t unembed_smem(int xr, bool w8, int64_t hidden) {
  return static_cast<size_t>(xr) * unembed_xrow((int)hidden) + unembed_nw(xr, w8) * unembed_patch(unembed_ks(xr, w8, hidden));
}

// Batch rows per workgroup: sixteen above eight rows where the LDS holds them (gpt-oss: 2880 wide), else chunks of eight
// (each chunk streams the weight once more).
int unembed_xr(int64_t rows, bool w8, int64_t hidden) {
  return (rows > 8 && unembed_smem(16, w8, hidden) <= 160 * 1024) ? 16 : 8;
}
// More than sixteen rows (logits from a bf16 weight: more than eight): chunks of 32 rows whose K halves take turns in LDS (unembed_rows32_kernel), as
// long as no wavefront gets more tiles than it has accumulators for and a half of 32 rows fits the LDS. Full
// vocabulary: 32 rows 371 -> 187 us (two passes of the 16-row kernel -> one), 17 rows 180 us; at 9-16 rows it is 2 %
// faster than the 16-row kernel for logits (179.3 against 183.3 us at 16 rows, 174.9 against 177.2 at 9) and takes
// those too, and 3 % slower with the argmax (185.2 against 179.4), which stays with the 16-row kernel.
constexpr int kRows32Waves = 8, kRows32MaxTiles = 4;
size_t unembed_rows32_smem(int64_t hidden) {
  const int64_t nsteps = hidden / 64, nb = nsteps - nsteps / 2;
  return static_cast<size_t>(32) * (nb * 128 + 16) + kRows32Waves * unembed_patch(64);
}
bool unembed_rows32(int64_t rows, bool w8, int64_t hidden, int64_t vocab, bool argmax) {
  const int64_t ntiles = (vocab + 31) / 32;
  return rows > ((argmax || w8) ? 16 : 8) && hidden >= 128 && ntiles <= static_cast<int64_t>(kRows32MaxTiles) * kUnembedGrid * kRows32Waves &&
         unembed_rows32_smem(hidden) <= 160 * 1024;
}
// fp8 weight at 9-16 rows, even vocabulary: the pairs-of-rows stream with six wavefronts
bool unembed_pairs16(int64_t rows, bool w8, int64_t hidden, int64_t vocab) {
  return w8 && rows > 8 && rows <= 16 && vocab % 2 == 0 && unembed_xr(rows, w8, hidden) == 16 &&
         static_cast<size_t>(16) * unembed_xrow((int)hidden) + 6 * unembed_patch(128) <= 160 * 1024;
}
int unembed_check(const char* who, const void* x, const void* W, bool w8, int64_t rows, int64_t hidden, int64_t vocab) {
  TLLM_REQUIRE(rows >= 0 && hidden >= 1 && vocab >= 1 && vocab < (1ll << 31) && hidden < (1ll << 24), TLLM_E_SHAPE,
               "%s: rows %lld, hidden %lld, vocab %lld", who, (long long)rows, (long long)hidden, (long long)vocab);
  if (rows == 0) return TLLM_OK;
  TLLM_REQUIRE(x && W, TLLM_E_ARG, "%s: x and W must not be NULL", who);
  TLLM_REQUIRE(hidden % 64 == 0, TLLM_E_SHAPE, "%s: hidden %lld must be a multiple of 64", who, (long long)hidden);
  TLLM_REQUIRE(unembed_smem(unembed_xr(rows, w8, hidden), w8, hidden) <= 160 * 1024, TLLM_E_SHAPE, "%s: hidden %lld too large for the LDS-resident activations", who,
               (long long)hidden);
  TLLM_REQUIRE(aligned16(x) && aligned16(W), TLLM_E_ALIGN, "%s: x and W must be 16-byte aligned", who);
  TLLM_REQUIRE((rows + 15) / 16 <= 65535, TLLM_E_SHAPE, "%s: rows %lld too many", who, (long long)rows);
  return TLLM_OK;
}

template <bool ARGMAX>
int unembed_launch(const char* who, const UnembedArgs& a, bool w8, hipStream_t st) {
  if (unembed_rows32(a.rows, w8, a.hidden, a.vocab, ARGMAX)) {
    auto kern = w8 ? unembed_rows32_kernel<kRows32Waves, 64, 4, true, ARGMAX> : unembed_rows32_kernel<kRows32Waves, 64, 3, false, ARGMAX>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    TLLM_REQUIRE(e == hipSuccess, TLLM_E_LAUNCH, "%s: cannot raise LDS limit: %s", who, hipGetErrorString(e));
    hipLaunchKernelGGL(kern, dim3(kUnembedGrid, (unsigned)((a.rows + 31) / 32)), dim3(kRows32Waves * 64), unembed_rows32_smem(a.hidden), st, a);
    return check_launch(who);
  }
  const int xr = unembed_xr(a.rows, w8, a.hidden);
  // fp8 weight, up to 8 rows, even vocabulary: pairs of rows (whole cache lines), eight wavefronts, 128 bytes per pair and step
  const size_t smem_pairs = static_cast<size_t>(8) * unembed_xrow(a.hidden) + 8 * unembed_patch(128);
  const bool pairs = w8 && xr == 8 && a.vocab % 2 == 0 && smem_pairs <= 160 * 1024;
  // ... and at 9-16 rows with six wavefronts (what the LDS holds next to sixteen activation rows)
  const size_t smem_pairs16 = static_cast<size_t>(16) * unembed_xrow(a.hidden) + 6 * unembed_patch(128);
  const bool pairs16 = unembed_pairs16(a.rows, w8, a.hidden, a.vocab);
  const size_t smem = pairs ? smem_pairs : (pairs16 ? smem_pairs16 : unembed_smem(xr, w8, a.hidden));
  const dim3 grid(kUnembedGrid, (unsigned)((a.rows + xr - 1) / xr));
#define TLLM_UNEMBED(XR, NW, KS, UD, W8F, ...)                                                                              \
  do {                                                                                                                      \
    auto kern = unembed_kernel<XR, NW, KS, UD, W8F, ARGMAX, ##__VA_ARGS__>;                                                 \
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
    TLLM_REQUIRE(e == hipSuccess, TLLM_E_LAUNCH, "%s: cannot raise LDS limit: %s", who, hipGetErrorString(e));              \
    hipLaunchKernelGGL(kern, grid, dim3(NW * 64), smem, st, a);                                                             \
  } while (0)
  if (pairs16) TLLM_UNEMBED(16, 6, 128, 2, true, true);
  else if (pairs) TLLM_UNEMBED(8, 8, 128, 2, true, true);          // steps in flight 1 / 2 / 3 / 4: 122 / 99 / 105 / 107 us; 12 wavefronts x 3: 103, 10 x 2: 103, 6 x 2: 115
  else if (xr == 8 && !w8) TLLM_UNEMBED(8, 10, 64, 3, false);
  else if (xr == 8 && unembed_ks(8, true, a.hidden) == 192) TLLM_UNEMBED(8, 8, 192, 2, true);
  else if (xr == 8) TLLM_UNEMBED(8, 8, 64, 4, true);
  else if (w8) TLLM_UNEMBED(16, 8, 64, 4, true);
  else TLLM_UNEMBED(16, 8, 64, 3, false);
#undef TLLM_UNEMBED
  return check_launch(who);
}
}  // namespace

extern "C" int tllm_unembedding_decode_bf16(const void* x, const void* W, const float* w_scale, void* logits, int64_t logits_row_stride,
                                            int64_t rows, int64_t hidden, int64_t vocab, void* stream) {
  int rc = unembed_check("unembedding_decode", x, W, w_scale != nullptr, rows, hidden, vocab);
  if (rc != TLLM_OK || rows == 0) return rc;
  TLLM_REQUIRE(logits != nullptr && logits_row_stride >= vocab, TLLM_E_ARG, "unembedding_decode: logits NULL or row stride < vocab");
  UnembedArgs a{};
  a.x = (const bf16*)x;
  a.W = W;
  a.w_scale = w_scale;
  a.logits = (bf16*)logits;
  a.ld = logits_row_stride;
  a.rows = rows;
  a.hidden = (int)hidden;
  a.vocab = (int)vocab;
  a.pair_stores = reinterpret_cast<uintptr_t>(logits) % 4 == 0 && logits_row_stride % 2 == 0;
  return unembed_launch<false>("unembedding_decode", a, w_scale != nullptr, static_cast<hipStream_t>(stream));
}

extern "C" int64_t tllm_unembedding_argmax_workspace_bytes(int64_t rows) {
  if (rows <= 0) return 0;
  const int xr = unembed_xr_most(rows);
  const int64_t chunks = (rows + xr - 1) / xr;
  // one (float, int) pair per wavefront (at most 16 per workgroup) and batch-row slot; chunks of eight rows, which a
  // wide hidden size forces, never need more slots than chunks of sixteen
  return chunks * kUnembedGrid * 16 * xr * 8;
}

// Both argmax entry points: the stream kernel leaves one candidate per wavefront and batch row in `workspace`, the
// reduce kernel picks the winners. Every slot the reduce kernel reads is written by the stream kernel of the same
// call, so the workspace needs no clearing.
static int unembed_argmax_run(const char* who, const void* x, const void* W, const float* w_scale, void* workspace, int64_t need,
                              int32_t* token_ids, int64_t rows, int64_t hidden, int64_t vocab, void* stream) {
  const bool rows32 = unembed_rows32(rows, w_scale != nullptr, hidden, vocab, true);
  const int xr = rows32 ? 32 : unembed_xr(rows, w_scale != nullptr, hidden);
  UnembedArgs a{};
  a.x = (const bf16*)x;
  a.W = W;
  a.w_scale = w_scale;
  a.part_max = static_cast<float*>(workspace);
  a.part_idx = reinterpret_cast<int*>(static_cast<unsigned char*>(workspace) + need / 2);
  a.rows = rows;
  a.hidden = (int)hidden;
  a.vocab = (int)vocab;
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc = unembed_launch<true>(who, a, w_scale != nullptr, st);
  if (rc != TLLM_OK) return rc;
  static_assert(kUnembedGrid * 16 <= 4 * kArgmaxReduceThreads, "the reduce kernel takes up to four candidates per thread");
  hipLaunchKernelGGL(unembed_argmax_reduce_kernel, dim3((unsigned)rows), dim3(kArgmaxReduceThreads), 0, st, a.part_max, a.part_idx, token_ids,
                     kUnembedGrid * (rows32 ? kRows32Waves : (unembed_pairs16(rows, w_scale != nullptr, hidden, vocab) ? 6 : unembed_nw(xr, w_scale != nullptr))), xr);
  return check_launch(who);
}

extern "C" int tllm_unembedding_argmax_bf16(const void* x, const void* W, const float* w_scale, void* workspace, int64_t workspace_bytes,
                                            int32_t* token_ids, int64_t rows, int64_t hidden, int64_t vocab, void* stream) {
  int rc = unembed_check("unembedding_argmax", x, W, w_scale != nullptr, rows, hidden, vocab);
  if (rc != TLLM_OK || rows == 0) return rc;
  const int64_t need = tllm_unembedding_argmax_workspace_bytes(rows);
  TLLM_REQUIRE(token_ids != nullptr, TLLM_E_ARG, "unembedding_argmax: token_ids is NULL");
  TLLM_REQUIRE(workspace != nullptr && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 4 == 0, TLLM_E_ARG,
               "unembedding_argmax: workspace of %lld bytes needed (tllm_unembedding_argmax_workspace_bytes), got %lld", (long long)need,
               (long long)workspace_bytes);
  return unembed_argmax_run("unembedding_argmax", x, W, w_scale, workspace, need, token_ids, rows, hidden, vocab, stream);
}

// ---- the allocation-free form -----------------------------------------------------------------------------------
// The candidates travel through a buffer the library owns: a file-scope device array, present on every GPU the code
// object is loaded on from then until the process ends. In host code the array's name is only a handle for
// hipGetSymbolAddress; the kernels get the device address that call returns, looked up once per device.
namespace {
constexpr int kNoAllocMaxRows = 16;
constexpr int64_t kNoAllocScratchBytes = static_cast<int64_t>(kUnembedGrid) * 16 * kNoAllocMaxRows * 8;   // 512 KiB
constexpr int kMaxDevices = 64;
}  // namespace

static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device, looked up on the first call per device. The look-up is a runtime
// query (it may load the code object), which a capturing stream does not allow: `capturing_stream`, when not null, is
// the stream the caller is about to launch on, and an unresolved address under capture is refused instead of queried.
int noalloc_scratch(const char* who, void** out, hipStream_t capturing_stream, bool check_capture) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  TLLM_REQUIRE(e == hipSuccess && dev >= 0 && dev < kMaxDevices, TLLM_E_LAUNCH, "%s: hipGetDevice: %s (device %d)", who,
               hipGetErrorString(e), dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    if (check_capture) {
      hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
      e = hipStreamIsCapturing(capturing_stream, &cs);
      TLLM_REQUIRE(e == hipSuccess && cs == hipStreamCaptureStatusNone, TLLM_E_ARG,
                   "%s: first use on device %d inside a stream capture: call tllm_unembedding_argmax_noalloc_init() on this device "
                   "before capturing", who, dev);
    }
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    TLLM_REQUIRE(e == hipSuccess && p != nullptr, TLLM_E_LAUNCH, "%s: hipGetSymbolAddress(scratch): %s", who, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return TLLM_OK;
}
}  // namespace

extern "C" int tllm_unembedding_argmax_noalloc_init(void) {
  void* ws = nullptr;
  return noalloc_scratch("unembedding_argmax_noalloc_init", &ws, nullptr, false);
}

extern "C" int64_t tllm_unembedding_argmax_noalloc_max_rows(void) { return kNoAllocMaxRows; }

extern "C" int tllm_unembedding_argmax_noalloc_bf16(const void* x, const void* W, const float* w_scale, int32_t* token_ids, int64_t rows,
                                                    int64_t hidden, int64_t vocab, void* stream) {
  TLLM_REQUIRE(rows <= kNoAllocMaxRows, TLLM_E_SHAPE,
               "unembedding_argmax_noalloc: at most %d rows (got %lld): the library-owned scratch holds the candidates of %d batch rows; "
               "use tllm_unembedding_argmax_bf16 with a workspace for more",
               kNoAllocMaxRows, (long long)rows, kNoAllocMaxRows);
  int rc = unembed_check("unembedding_argmax_noalloc", x, W, w_scale != nullptr, rows, hidden, vocab);
  if (rc != TLLM_OK || rows == 0) return rc;
  TLLM_REQUIRE(token_ids != nullptr, TLLM_E_ARG, "unembedding_argmax_noalloc: token_ids is NULL");
  const int64_t need = tllm_unembedding_argmax_workspace_bytes(rows);
  TLLM_REQUIRE(need <= kNoAllocScratchBytes, TLLM_E_SHAPE, "unembedding_argmax_noalloc: %lld bytes of candidates exceed the scratch",
               (long long)need);
  void* ws = nullptr;
  rc = noalloc_scratch("unembedding_argmax_noalloc", &ws, static_cast<hipStream_t>(stream), true);
  if (rc != TLLM_OK) return rc;
  return unembed_argmax_run("unembedding_argmax_noalloc", x, W, w_scale, ws, need, token_ids, rows, hidden, vocab, stream);
}
