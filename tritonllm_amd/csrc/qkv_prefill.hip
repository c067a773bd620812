// Prefill-size fused QKV projection + bias + rotary: an LDS-staged bf16 MFMA GEMM.
//
//   D[T, 5120] = X[T, 2880] . W[5120, 2880]^T      (both operands K-contiguous)
//
// Tiling for 256 CUs: a workgroup computes a 128-token x 320-column tile (five whole heads),
// so T = 2048 is exactly 16 x 16 = 256 tiles -- one per CU, no tail wave -- and T = 8192 is
// exactly four per CU. Four wavefronts form a 2 x 2 grid; each owns 64 x 160 of the tile as
// 2 x 5 v_mfma_f32_32x32x16_bf16 blocks (160 fp32 accumulators per lane) and reads 7 operand
// fragments from LDS per 10 MFMAs. K is walked in slices of 64 through a double-buffered LDS
// stage: global -> registers (128-bit, coalesced along K) is issued one slice ahead of the
// MFMAs that consume the previous one. LDS rows are padded to 144 bytes so the 128-bit
// fragment reads of 16 consecutive rows fall in 16 different bank groups.
//
// The rotary pair (d, d+32) has to sit in one lane. A 32x32 block gives lane l column l%32,
// so for a whole head the pair is the same lane of two neighbouring blocks. 160 columns per
// wavefront are 2.5 heads; the tile's middle head is therefore split by *dims*: wavefront
// column 0 takes dims [0,16) u [32,48), column 1 takes [16,32) u [48,64), packed into one
// "mixed" block whose pair partner is lane l^16. The W rows are permuted accordingly when
// they are copied into LDS, which costs nothing.
//
// Epilogue: cos/sin of the tile's 128 positions x 32 frequencies are computed once per
// workgroup from the YaRN parameters into the (by then idle) LDS stage, then every lane adds
// the bias to its fp32 accumulators, rotates q/k pairs, rounds once to bf16 and stores
// straight into the separate q / k / v outputs (no split / contiguous copies afterwards).
#include "qkv_common.h"

namespace tllm {

namespace {
constexpr int BM = 128;            // tokens per tile
constexpr int HPT = 5;             // heads per tile
constexpr int BN = HPT * 64;       // 320 columns per tile
constexpr int BK = 64;             // K slice
constexpr int LROW = BK * 2 + 16;  // padded LDS row, bytes
constexpr int A_BYTES = BM * LROW;
constexpr int STAGE = (BM + BN) * LROW;   // 64 512 bytes
constexpr int SMEM = 2 * STAGE;           // 129 024 bytes
constexpr int A_SLABS = BM / 32;          // loader: 32 rows per slab of 256 threads x 16 B
constexpr int B_SLABS = BN / 32;
}  // namespace

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

__global__ __launch_bounds__(256) void qkv_prefill_kernel(QkvArgs a, RopeArgs ra, YarnFreqs fr, int tiles_m, int tiles_n, int swizzle) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  // ---- tile assignment: XCD-aware. Consecutive block ids go to different XCDs (8 of them, each
  // with its own L2), so give every XCD a compact 8 x 4 super-block of tiles to maximise L2 reuse.
  int tile_m, tile_n;
  {
    const int b = blockIdx.x;
    if (swizzle) {
      const int per = (tiles_m * tiles_n) >> 3;
      const int id = (b & 7) * per + (b >> 3);
      const int sb = id >> 5, in = id & 31;
      const int sbm = tiles_m >> 3;
      tile_m = (sb % sbm) * 8 + (in & 7);
      tile_n = (sb / sbm) * 4 + (in >> 3);
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

  // ---- loader setup: thread (lr, lc) copies 16-byte chunk lc of rows lr, lr+32, ... of the K slice
  const int lr = tid >> 3, lc = tid & 7;
  const bf16x8* xg = reinterpret_cast<const bf16x8*>(a.x);
  const bf16x8* wg = reinterpret_cast<const bf16x8*>(a.W);
  const bf16x8* a_src[A_SLABS];
  const bf16x8* b_src[B_SLABS];
#pragma unroll
  for (int s = 0; s < A_SLABS; ++s) {
    int64_t r = row0 + s * 32 + lr;
    if (r >= a.rows) r = a.rows - 1;            // clamp: valid memory, result rows are never stored
    a_src[s] = xg + r * kvec + lc;
  }
#pragma unroll
  for (int s = 0; s < B_SLABS; ++s) {
    int hl, dim;
    w_tile_row(s * 32 + lr, &hl, &dim);
    int h = head0 + hl;
    if (h >= total_heads) h = total_heads - 1;  // clamp for a ragged last tile
    b_src[s] = wg + (static_cast<int64_t>(h) * 64 + dim) * kvec + lc;
  }
  const int st_off = lr * LROW + lc * 16;       // where this thread's chunk lands inside a slab

  bf16x8 ra_[A_SLABS], rb_[B_SLABS];
  auto load_global = [&](int it) {
#pragma unroll
    for (int s = 0; s < A_SLABS; ++s) ra_[s] = a_src[s][it * 8];
#pragma unroll
    for (int s = 0; s < B_SLABS; ++s) rb_[s] = b_src[s][it * 8];
  };
  auto store_lds = [&](int stage) {
    unsigned char* base = smem + stage * STAGE + st_off;
#pragma unroll
    for (int s = 0; s < A_SLABS; ++s) *reinterpret_cast<bf16x8*>(base + s * 32 * LROW) = ra_[s];
#pragma unroll
    for (int s = 0; s < B_SLABS; ++s) *reinterpret_cast<bf16x8*>(base + A_BYTES + s * 32 * LROW) = rb_[s];
  };

  f32x16 acc[2][5];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < 5; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mb][nb][v] = 0.f;

  // fragment read offsets inside a stage (bytes)
  const int fa_off = (64 * wm + l32) * LROW + lh * 16;
  const int fb_off = A_BYTES + (160 * wn + l32) * LROW + lh * 16;

  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int it = 0; it < n_iter; ++it) {
    const int cur = it & 1;
    if (it + 1 < n_iter) load_global(it + 1);
    const unsigned char* sa = smem + cur * STAGE + fa_off;
    const unsigned char* sb = smem + cur * STAGE + fb_off;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 fa[2], fb[5];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) fa[mb] = *reinterpret_cast<const bf16x8*>(sa + mb * 32 * LROW + kk * 32);
#pragma unroll
      for (int nb = 0; nb < 5; ++nb) fb[nb] = *reinterpret_cast<const bf16x8*>(sb + nb * 32 * LROW + kk * 32);
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 5; ++nb) acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mb], fb[nb], acc[mb][nb], 0, 0, 0);
    }
    if (it + 1 < n_iter) store_lds(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue -------------------------------------------------------------------------------
  // cos/sin of (tile row, frequency) into LDS as float2 {cos, sin}; the stages are idle now.
  float2* cs_tab = reinterpret_cast<float2*>(smem);
  if (a.has_rope) {
    const int f = tid & 31;
#pragma unroll 1
    for (int j = 0; j < BM / 8; ++j) {
      const int r = (tid >> 5) + 8 * j;
      int64_t grow = row0 + r;
      if (grow >= a.rows) grow = a.rows - 1;
      const int64_t pos = rope_position(ra, grow);
      float c, s;
      rope_cos_sin(ra, fr, pos, f, &c, &s);
      cs_tab[r * 32 + f] = make_float2(c, s);
    }
    __syncthreads();
  }

  const int64_t slot_off = qkv_slot(a, ra) * a.kv_slot_stride;

  // The wavefront's three heads: two whole ones (blocks 0-1, 2-3) and its half of the middle head (block 4).
#pragma unroll
  for (int hp = 0; hp < 3; ++hp) {
    const int hl = (hp < 2) ? (3 * wn + hp) : 2;
    const int head = head0 + hl;
    if (head >= total_heads) continue;
    bf16* base;
    int64_t rs;
    if (head < a.n_q_heads) {
      base = a.q + static_cast<int64_t>(head) * 64;
      rs = a.q_rs;
    } else if (head < a.n_q_heads + a.n_kv_heads) {
      base = a.k + slot_off + static_cast<int64_t>(head - a.n_q_heads) * 64;
      rs = a.k_rs;
    } else {
      base = a.v + slot_off + static_cast<int64_t>(head - a.n_q_heads - a.n_kv_heads) * 64;
      rs = a.v_rs;
    }
    const bool rotate = a.has_rope && head < a.n_q_heads + a.n_kv_heads;

    if (hp < 2) {
      const int d = l32;                                     // frequency index == low dim
      const float b_lo = a.bias ? static_cast<float>(a.bias[head * 64 + d]) : 0.f;
      const float b_hi = a.bias ? static_cast<float>(a.bias[head * 64 + 32 + d]) : 0.f;
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int r = 64 * wm + 32 * mb + 8 * (v >> 2) + 4 * lh + (v & 3);
          const int64_t grow = row0 + r;
          float lo = acc[mb][2 * hp][v] + b_lo;
          float hi = acc[mb][2 * hp + 1][v] + b_hi;
          if (rotate) {
            const float2 cs = cs_tab[r * 32 + d];
            const float rl = lo * cs.x - hi * cs.y;
            const float rh = hi * cs.x + lo * cs.y;
            lo = rl;
            hi = rh;
          }
          if (grow < a.rows) {
            bf16* o = base + grow * rs;
            o[d] = static_cast<bf16>(lo);
            o[d + 32] = static_cast<bf16>(hi);
          }
        }
      }
    } else {
      const bool is_lo = l32 < 16;
      const int d = 16 * wn + (l32 & 15);                    // frequency index
      const int dim = is_lo ? d : d + 32;
      const float b_own = a.bias ? static_cast<float>(a.bias[head * 64 + dim]) : 0.f;
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int r = 64 * wm + 32 * mb + 8 * (v >> 2) + 4 * lh + (v & 3);
          const int64_t grow = row0 + r;
          float own = acc[mb][4][v] + b_own;
          const float partner = __shfl_xor(own, 16, 64);
          if (rotate) {
            const float2 cs = cs_tab[r * 32 + d];
            own = is_lo ? (own * cs.x - partner * cs.y) : (own * cs.x + partner * cs.y);
          }
          if (grow < a.rows) base[grow * rs + dim] = static_cast<bf16>(own);
        }
      }
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
  static bool attr_set = false;   // raising the dynamic-LDS limit is idempotent; a benign race at worst repeats it
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_prefill_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
    TLLM_REQUIRE(e == hipSuccess, TLLM_E_LAUNCH, "qkv_rope_prefill: cannot raise LDS limit: %s", hipGetErrorString(e));
    attr_set = true;
  }
  const int heads = n_q_heads + 2 * n_kv_heads;
  const int64_t tiles_m = (rows + BM - 1) / BM;
  const int tiles_n = (heads + HPT - 1) / HPT;
  const int64_t tiles = tiles_m * tiles_n;
  TLLM_REQUIRE(tiles < (1ll << 31), TLLM_E_SHAPE, "qkv_rope_prefill: too many tiles");
  const int swizzle = (tiles_m % 8 == 0 && tiles_n % 4 == 0) ? 1 : 0;
  hipLaunchKernelGGL(qkv_prefill_kernel, dim3((unsigned)tiles), dim3(256), SMEM, st, a, ra, fr, (int)tiles_m, tiles_n, swizzle);
  return check_launch("qkv_rope_prefill");
}
