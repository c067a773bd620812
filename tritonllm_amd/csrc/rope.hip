// Half-split (NeoX-style) rotary embedding applied in place to q and k, and the
// YaRN cos/sin table builder.
//
// A workgroup owns TOK consecutive tokens. The cos/sin of a (token, frequency) pair is
// needed by every head of that token, so the first TOK*n_freq lanes compute them once
// (in registers, from the YaRN parameters, or by reading the caller's table) into LDS;
// after one barrier all 256 lanes stream the heads: each work item is the pair of
// 128-bit vectors (dims d..d+7, dims d+hd/2..d+hd/2+7) of one head, rotated in fp32 and
// stored back with one round-to-nearest-even per output.
// Prompts take four tokens per workgroup (the cos/sin work is shared by more items). A decode
// batch is a handful of tokens: there a workgroup takes one token (the reference makes the same
// switch below 60 tokens, triton_kernels.py:94-107) and gridDim.y workgroups share its heads, so
// that every lane has one item and the launch is one load-rotate-store deep.
#include "common.h"

namespace tllm {

constexpr int kRopeTok = 4;
// up to here: one token per workgroup (us, four tokens per workgroup -> one: 128 tokens 4.27 -> 2.37, 512 4.74 -> 3.01,
// 1024 5.35 -> 4.27, 2048 6.97 -> 6.60; 4096 13.4 -> 14.7, 8192 24.4 -> 25.5: from there on four per workgroup)
constexpr int kRopeSmallRows = 2048;

template <int TOK>
__global__ __launch_bounds__(256) void rope_kernel(bf16x8* q, bf16x8* k, int64_t rows, int n_q_heads, int n_kv_heads, int head_dim,
                                                   RopeArgs ra, YarnFreqs fr) {
  __shared__ float s_cos[TOK * TLLM_MAX_ROPE_FREQS];
  __shared__ float s_sin[TOK * TLLM_MAX_ROPE_FREQS];
  const int tid = threadIdx.x;
  const int n_freq = head_dim >> 1;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * TOK;
  const int ntok = static_cast<int>(rows - row0 < TOK ? rows - row0 : TOK);

  for (int e = tid; e < ntok * n_freq; e += 256) {
    const int t = e / n_freq, i = e - t * n_freq;
    const int64_t pos = rope_position(ra, row0 + t);
    float c, s;
    rope_cos_sin(ra, fr, pos, i, &c, &s);
    s_cos[t * TLLM_MAX_ROPE_FREQS + i] = c;
    s_sin[t * TLLM_MAX_ROPE_FREQS + i] = s;
  }
  __syncthreads();

  const int vph = n_freq >> 3;                       // 128-bit vectors per half head
  const int heads = n_q_heads + n_kv_heads;
  const int items_per_tok = heads * vph;
  // the workgroups of one token group (gridDim.y of them) deal the items round-robin in runs of 256
  for (int it = blockIdx.y * 256 + tid; it < ntok * items_per_tok; it += 256 * gridDim.y) {
    const int t = it / items_per_tok;
    const int r = it - t * items_per_tok;
    const int h = r / vph, j = r - h * vph;
    bf16x8* base;
    if (h < n_q_heads)
      base = q + ((row0 + t) * n_q_heads + h) * (2 * vph);
    else
      base = k + ((row0 + t) * n_kv_heads + (h - n_q_heads)) * (2 * vph);
    const bf16x8 lo = base[j], hi = base[vph + j];
    const float* cs = s_cos + t * TLLM_MAX_ROPE_FREQS + 8 * j;
    const float* sn = s_sin + t * TLLM_MAX_ROPE_FREQS + 8 * j;
    bf16x8 olo, ohi;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float x1 = static_cast<float>(lo[e]), x2 = static_cast<float>(hi[e]);
      const float c = cs[e], s = sn[e];
      olo[e] = static_cast<bf16>(x1 * c - x2 * s);
      ohi[e] = static_cast<bf16>(x2 * c + x1 * s);
    }
    base[j] = olo;
    base[vph + j] = ohi;
  }
}

// A decode batch: one token per workgroup, gridDim.y workgroups sharing its heads, one item per lane. The item's two
// vectors are requested before anything else, so that the position load and the cos / sin arithmetic of the first n_freq
// lanes run while they are on their way; one barrier, then rotate and store.
__global__ __launch_bounds__(256) void rope_few_kernel(bf16x8* q, bf16x8* k, int n_q_heads, int n_kv_heads, int head_dim, RopeArgs ra,
                                                       YarnFreqs fr) {
  __shared__ float s_cos[TLLM_MAX_ROPE_FREQS];
  __shared__ float s_sin[TLLM_MAX_ROPE_FREQS];
  const int tid = threadIdx.x;
  const int n_freq = head_dim >> 1;
  const int64_t row = blockIdx.x;
  const int vph = n_freq >> 3;                       // 128-bit vectors per half head
  const int items = (n_q_heads + n_kv_heads) * vph;
  const int it = blockIdx.y * 256 + tid;
  const bool valid = it < items;
  const int itc = valid ? it : 0;
  const int h = itc / vph, j = itc - h * vph;
  bf16x8* base;
  if (h < n_q_heads)
    base = q + (row * n_q_heads + h) * (2 * vph);
  else
    base = k + (row * n_kv_heads + (h - n_q_heads)) * (2 * vph);
  const bf16x8 lo = base[j], hi = base[vph + j];     // lanes past the last item read item 0 and store nothing

  for (int i = tid; i < n_freq; i += 256) {
    const int64_t pos = rope_position(ra, row);
    float c, s;
    rope_cos_sin(ra, fr, pos, i, &c, &s);
    s_cos[i] = c;
    s_sin[i] = s;
  }
  __syncthreads();
  if (!valid) return;

  const float* cs = s_cos + 8 * j;
  const float* sn = s_sin + 8 * j;
  bf16x8 olo, ohi;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float x1 = static_cast<float>(lo[e]), x2 = static_cast<float>(hi[e]);
    const float c = cs[e], s = sn[e];
    olo[e] = static_cast<bf16>(x1 * c - x2 * s);
    ohi[e] = static_cast<bf16>(x2 * c + x1 * s);
  }
  base[j] = olo;
  base[vph + j] = ohi;
}

__global__ __launch_bounds__(256) void yarn_table_kernel(float* cos_out, float* sin_out, int64_t start, int64_t n_pos, int n_freq,
                                                         float concentration, YarnFreqs fr) {
  const int64_t total = n_pos * n_freq;
  const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += step) {
    const int64_t p = e / n_freq;
    const int i = static_cast<int>(e - p * n_freq);
    float c, s;
    yarn_cos_sin(start + p, fr.v[i], concentration, &c, &s);
    cos_out[e] = c;
    sin_out[e] = s;
  }
}

}  // namespace tllm

using namespace tllm;

extern "C" int tllm_rope_bf16(void* q, void* k, int64_t rows, int n_q_heads, int n_kv_heads, int head_dim, const TllmRope* rope,
                              void* stream) {
  TLLM_REQUIRE(rows >= 0 && n_q_heads >= 0, TLLM_E_ARG, "rope: rows %lld / n_q_heads %d invalid", (long long)rows, n_q_heads);
  if (k == nullptr) n_kv_heads = 0;
  TLLM_REQUIRE(n_kv_heads >= 0, TLLM_E_ARG, "rope: n_kv_heads %d invalid", n_kv_heads);
  RopeArgs ra;
  YarnFreqs fr;
  int rc = make_rope_args(rope, head_dim, &ra, &fr);
  if (rc != TLLM_OK) return rc;
  TLLM_REQUIRE(head_dim % 16 == 0, TLLM_E_SHAPE, "rope: head_dim %d must be a multiple of 16", head_dim);
  if (rows == 0 || n_q_heads + n_kv_heads == 0) return TLLM_OK;
  TLLM_REQUIRE(q != nullptr || n_q_heads == 0, TLLM_E_ARG, "rope: q is NULL");
  TLLM_REQUIRE(aligned16(q) && aligned16(k), TLLM_E_ALIGN, "rope: q/k must be 16-byte aligned");
  if (rows <= kRopeSmallRows) {
    const int items = (n_q_heads + n_kv_heads) * (head_dim >> 4);     // per token
    int parts = (items + 255) / 256;
    parts = parts < 1 ? 1 : (parts > 64 ? 64 : parts);
    if (items <= parts * 256)     // one item per lane
      hipLaunchKernelGGL(rope_few_kernel, dim3((unsigned)rows, (unsigned)parts), dim3(256), 0, static_cast<hipStream_t>(stream),
                         (bf16x8*)q, (bf16x8*)k, n_q_heads, n_kv_heads, head_dim, ra, fr);
    else
      hipLaunchKernelGGL(rope_kernel<1>, dim3((unsigned)rows, (unsigned)parts), dim3(256), 0, static_cast<hipStream_t>(stream), (bf16x8*)q,
                         (bf16x8*)k, rows, n_q_heads, n_kv_heads, head_dim, ra, fr);
    return check_launch("rope");
  }
  const int64_t blocks = (rows + kRopeTok - 1) / kRopeTok;
  TLLM_REQUIRE(blocks < (1ll << 31), TLLM_E_SHAPE, "rope: rows %lld too large", (long long)rows);
  hipLaunchKernelGGL(rope_kernel<kRopeTok>, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), (bf16x8*)q, (bf16x8*)k,
                     rows, n_q_heads, n_kv_heads, head_dim, ra, fr);
  return check_launch("rope");
}

extern "C" int tllm_yarn_table_f32(float* cos, float* sin, int64_t start, int64_t n_pos, const TllmYarn* yarn, void* stream) {
  TLLM_REQUIRE(n_pos >= 0 && start >= 0, TLLM_E_ARG, "yarn_table: start %lld / n_pos %lld invalid", (long long)start, (long long)n_pos);
  TLLM_REQUIRE(yarn != nullptr, TLLM_E_ARG, "yarn_table: yarn is NULL");
  TLLM_REQUIRE(yarn->n_freq > 0 && yarn->n_freq <= TLLM_MAX_ROPE_FREQS, TLLM_E_SHAPE, "yarn_table: n_freq %d out of range", yarn->n_freq);
  if (n_pos == 0) return TLLM_OK;
  TLLM_REQUIRE(cos && sin, TLLM_E_ARG, "yarn_table: null pointer");
  YarnFreqs fr = {};
  for (int i = 0; i < yarn->n_freq; ++i) fr.v[i] = yarn->inv_freq[i];
  const int64_t total = n_pos * yarn->n_freq;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(yarn_table_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), cos, sin, start, n_pos,
                     yarn->n_freq, yarn->concentration, fr);
  return check_launch("yarn_table");
}
