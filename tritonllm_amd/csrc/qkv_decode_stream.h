// What the streaming decode QKV kernels (qkv_decode_r8.hip, qkv_decode_r32.hip, qkv_decode_rows.hip) share: the epilogue lane that
// finishes four adjacent outputs of one activation row.
#pragma once

#include "qkv_common.h"

namespace tllm {

// One lane of an epilogue wavefront. A workgroup owns ten rotation pairs in two 16-row MFMA tiles (tile 0 = pairs
// 0..5, tile 1 = pairs 6..9), two adjacent pairs (2i, 2i+1) occupying the four tile rows [lo(2i), lo(2i+1), hi(2i),
// hi(2i+1)] of quad i; the accumulator registers of lane (activation row n, quad eg) are exactly those four values of
// row n. prepare() issues every global load the lane needs (position, bias, row scales) and computes cos / sin and the
// output address while the weight streams; finish() takes the reduced sums to the stored bf16 values. prepare() is
// prepare_lane() + request_row() + prepare_row(), for the kernel that finishes one block of rows after the other.
template <bool W8>
struct StreamEpilogueLane {
  float cs0, sn0, cs1, sn1;       // rotation of pair epair and epair + 1
  float bl0, bl1, bh0, bh1;       // bias of [lo(d), lo(d+1), hi(d), hi(d+1)]
  float ws_l0, ws_l1, ws_h0, ws_h1;   // W8: row scales of the same four weight rows
  bf16* out;                      // &row[head * 64 + d]; the hi half sits 32 elements further
  bool evalid, erot;
  // what prepare_lane() leaves for prepare_row()
  float freq0, freq1;
  int64_t off_ld;
  int ehead, ed;
  bool lane_ok;

  // The part that depends on the lane's place in the tile only: bias, row scales, frequencies, the offset. A kernel
  // that finishes several row blocks per lane does this once.
  __device__ __forceinline__ void prepare_lane(const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr, int pair0, int tile, int eg) {
    const int total_pairs = (a.n_q_heads + 2 * a.n_kv_heads) * 32;
    const int epair = pair0 + (tile ? 6 : 0) + 2 * eg;      // even; its neighbour epair + 1 shares head and quad
    lane_ok = eg < (tile ? 2 : 3) && epair < total_pairs;
    const int egp = lane_ok ? epair : 0;
    ehead = egp >> 5;
    ed = egp & 31;
    erot = a.has_rope && ehead < a.n_q_heads + a.n_kv_heads;
    // absent operands read a valid dummy address instead of being predicated (a load under a branch makes the compiler
    // wait for everything in flight where the paths join)
    const int64_t* off_ptr = ra.offset ? ra.offset : reinterpret_cast<const int64_t*>(a.W);
    const unsigned* bias_ptr = reinterpret_cast<const unsigned*>(a.bias ? a.bias : a.W);   // two bf16 per load; ed is even
    off_ld = *off_ptr;
    const unsigned b_lo = bias_ptr[(ehead * 64 + ed) >> 1];
    const unsigned b_hi = bias_ptr[(ehead * 64 + 32 + ed) >> 1];
    freq0 = fr.v[ed];
    freq1 = fr.v[ed + 1];
    ws_l0 = ws_l1 = ws_h0 = ws_h1 = 1.f;
    if constexpr (W8) {
      const float* sp = a.w_scale + ehead * 64 + ed;        // 4-byte aligned is all the interface asks for
      ws_l0 = sp[0];
      ws_l1 = sp[1];
      ws_h0 = sp[32];
      ws_h1 = sp[33];
    }
    bl0 = bl1 = bh0 = bh1 = 0.f;
    if (a.bias) {
      bl0 = __uint_as_float(b_lo << 16);
      bl1 = __uint_as_float(b_lo & 0xffff0000u);
      bh0 = __uint_as_float(b_hi << 16);
      bh1 = __uint_as_float(b_hi & 0xffff0000u);
    }
  }

  // The position of activation row `en` of the block at row0, as loaded (the load is on its way when this returns; rows
  // past the block's last one read the block's first).
  __device__ __forceinline__ int64_t request_row(const QkvArgs& a, const RopeArgs& ra, int en, int64_t row0, int nvalid) const {
    const int64_t erow = row0 + (en < nvalid ? en : 0);
    const int64_t* pos_ptr = ra.positions ? ra.positions + erow : reinterpret_cast<const int64_t*>(a.W);
    return *pos_ptr;
  }

  // The part that depends on the activation row: cos / sin at its position, the output address.
  __device__ __forceinline__ void prepare_row(const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr, int64_t pos_ld, int en, int64_t row0,
                                              int nvalid) {
    evalid = lane_ok && en < nvalid;
    const int64_t erow = row0 + (en < nvalid ? en : 0);
    cs0 = cs1 = 1.f;
    sn0 = sn1 = 0.f;
    const int64_t slot = (a.kv_slot_stride != 0 && ra.offset != nullptr) ? off_ld : 0;
    if (erot) {
      int64_t pos = ra.positions ? pos_ld : (erow % ra.tokens_per_batch) + (ra.offset ? off_ld : 0);
      pos = rope_wrap(pos, ra.max_ctx);
      if (ra.use_yarn) {
        yarn_cos_sin(pos, freq0, ra.concentration, &cs0, &sn0);
        yarn_cos_sin(pos, freq1, ra.concentration, &cs1, &sn1);
      } else {
        rope_cos_sin(ra, fr, pos, ed, &cs0, &sn0);
        rope_cos_sin(ra, fr, pos, ed + 1, &cs1, &sn1);
      }
    }
    out = qkv_out_ptr(a, slot, erow, ehead) + ed;
    // One wavefront runs alone from the last barrier to the stores, so every instruction after that barrier is
    // latency: all of the above is forced to exist here (left to itself the compiler moves it to its first use,
    // behind the barrier).
    asm volatile("" : "+v"(cs0), "+v"(sn0), "+v"(cs1), "+v"(sn1), "+v"(bl0), "+v"(bl1), "+v"(bh0), "+v"(bh1), "+v"(out));
    if constexpr (W8) asm volatile("" : "+v"(ws_l0), "+v"(ws_l1), "+v"(ws_h0), "+v"(ws_h1));
  }

  // Everything for one block: lane (quad eg of tile `tile`, activation row en of the nvalid rows at row0).
  __device__ __forceinline__ void prepare(const QkvArgs& a, const RopeArgs& ra, const YarnFreqs& fr, int pair0, int tile, int eg, int en,
                                          int64_t row0, int nvalid) {
    const int64_t pos_ld = request_row(a, ra, en, row0, nvalid);   // first: the longest chain hangs on it
    prepare_lane(a, ra, fr, pair0, tile, eg);
    prepare_row(a, ra, fr, pos_ld, en, row0, nvalid);
  }

  // acc = the reduced [lo(d), lo(d+1), hi(d), hi(d+1)] of the lane's activation row: row scale, bias, rotation, one
  // rounding; 4-byte stores when `out4` says the outputs allow them.
  __device__ __forceinline__ void finish(f32x4 acc, int out4) const {
    if (!evalid) return;
    if constexpr (W8) {
      acc[0] *= ws_l0;
      acc[1] *= ws_l1;
      acc[2] *= ws_h0;
      acc[3] *= ws_h1;
    }
    float lo0 = acc[0] + bl0, lo1 = acc[1] + bl1, hi0 = acc[2] + bh0, hi1 = acc[3] + bh1;
    if (erot) {
      const float r0 = lo0 * cs0 - hi0 * sn0, r2 = hi0 * cs0 + lo0 * sn0;
      const float r1 = lo1 * cs1 - hi1 * sn1, r3 = hi1 * cs1 + lo1 * sn1;
      lo0 = r0;
      lo1 = r1;
      hi0 = r2;
      hi1 = r3;
    }
    bf16x2 plo, phi;
    plo[0] = static_cast<bf16>(lo0);
    plo[1] = static_cast<bf16>(lo1);
    phi[0] = static_cast<bf16>(hi0);
    phi[1] = static_cast<bf16>(hi1);
    if (out4) {
      *reinterpret_cast<bf16x2*>(out) = plo;
      *reinterpret_cast<bf16x2*>(out + 32) = phi;
    } else {
      out[0] = plo[0];
      out[1] = plo[1];
      out[32] = phi[0];
      out[33] = phi[1];
    }
  }
};

// Whether q / k / v (and the KV slot stride) allow the epilogue's 4-byte stores.
inline int qkv_outputs_allow_4_byte_stores(const QkvArgs& a) {
  auto even = [](int64_t v) { return (v & 1) == 0; };
  return (reinterpret_cast<uintptr_t>(a.q) % 4 == 0) && (reinterpret_cast<uintptr_t>(a.k) % 4 == 0) && (reinterpret_cast<uintptr_t>(a.v) % 4 == 0) &&
         even(a.q_rs) && even(a.k_rs) && even(a.v_rs) && even(a.kv_slot_stride);
}

}  // namespace tllm
