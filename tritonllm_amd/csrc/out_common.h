// Argument block shared by the decode out-projection kernels (out_decode.hip, out_decode_r8.hip, out_decode_r32.hip).
#pragma once
#include "common.h"

namespace tllm {

struct OutArgs {
  const bf16* x;          // [rows, in_dim]
  const void* W;          // [out_dim, in_dim] bf16, or fp8 bytes when w_scale != null
  const float* w_scale;   // [out_dim] or null
  const bf16* bias;       // [out_dim] or null
  const bf16* res;        // [rows, out_dim] with row stride res_rs, or null
  bf16* out;              // [rows, out_dim] with row stride out_rs
  int64_t res_rs, out_rs;
  int64_t rows;
  int in_dim, out_dim;
};

// in_dim 4096, out_dim % 12 == 0, rows <= 8, bf16 weight or (a.w_scale != null) fp8; grid = (out_dim / 12)
void launch_out_decode_r8(dim3 grid, hipStream_t st, const OutArgs& a);

// in_dim 4096, out_dim % 12 == 0, bf16 or fp8 weight, any number of rows in chunks of 32; grid = (out_dim / 12, ceil(rows / 32)) as
// the caller counts chunks -- the launch itself gives a workgroup up to four of them
void launch_out_decode_r32(dim3 grid, hipStream_t st, const OutArgs& a);

}  // namespace tllm
