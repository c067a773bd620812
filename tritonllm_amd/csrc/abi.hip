// ABI bookkeeping: version, thread-local error text, launch checks, rotary argument validation.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "common.h"

namespace tllm {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return TLLM_E_LAUNCH;
  }
  return TLLM_OK;
}

int make_rope_args(const TllmRope* rope, int head_dim, RopeArgs* out, YarnFreqs* freqs) {
  memset(out, 0, sizeof(*out));
  memset(freqs, 0, sizeof(*freqs));
  TLLM_REQUIRE(rope != nullptr, TLLM_E_ARG, "rope: descriptor is NULL");
  TLLM_REQUIRE(head_dim > 0 && head_dim % 2 == 0, TLLM_E_SHAPE, "rope: head_dim %d must be even and positive", head_dim);
  const int n_freq = head_dim / 2;
  TLLM_REQUIRE(n_freq <= TLLM_MAX_ROPE_FREQS, TLLM_E_SHAPE, "rope: head_dim %d exceeds %d", head_dim, 2 * TLLM_MAX_ROPE_FREQS);
  TLLM_REQUIRE(rope->max_ctx >= 1, TLLM_E_ARG, "rope: max_ctx %lld must be >= 1", (long long)rope->max_ctx);
  TLLM_REQUIRE(rope->positions != nullptr || rope->tokens_per_batch >= 1, TLLM_E_ARG,
               "rope: tokens_per_batch %lld must be >= 1 when positions is NULL", (long long)rope->tokens_per_batch);
  if (rope->yarn) {
    TLLM_REQUIRE(rope->yarn->n_freq == n_freq, TLLM_E_SHAPE, "rope: yarn.n_freq %d != head_dim/2 = %d", rope->yarn->n_freq, n_freq);
    TLLM_REQUIRE(rope->max_ctx <= (1ll << 24), TLLM_E_SHAPE,
                 "rope: in-register cos/sin supports max_ctx <= 2^24 (got %lld); pass cos/sin tables instead", (long long)rope->max_ctx);
    memcpy(freqs->v, rope->yarn->inv_freq, sizeof(float) * n_freq);
    out->concentration = rope->yarn->concentration;
    out->use_yarn = 1;
  } else {
    TLLM_REQUIRE(rope->cos_table && rope->sin_table, TLLM_E_ARG, "rope: neither yarn parameters nor cos/sin tables given");
    TLLM_REQUIRE(rope->table_row_stride >= n_freq, TLLM_E_ARG, "rope: table_row_stride %lld < head_dim/2", (long long)rope->table_row_stride);
    out->cos_table = rope->cos_table;
    out->sin_table = rope->sin_table;
    out->table_row_stride = rope->table_row_stride;
    out->use_yarn = 0;
  }
  out->positions = rope->positions;
  out->offset = rope->offset;
  out->tokens_per_batch = rope->tokens_per_batch >= 1 ? rope->tokens_per_batch : 1;
  out->max_ctx = rope->max_ctx;
  out->n_freq = n_freq;
  return TLLM_OK;
}

}  // namespace tllm

extern "C" int tllm_abi_version(void) { return TLLM_ABI_VERSION; }
extern "C" const char* tllm_last_error(void) { return tllm::g_err; }
