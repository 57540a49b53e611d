// A single-channel 3x3 convolution tile on the 16x16x4 MFMA, shared by k_conv_rows1.hip (the
// convolution as a command of its own) and k_conv_rows.hip (the same convolution, Rectify and 2x2
// pooling computed in front of the next convolution, in LDS).  Both call the functions below, so
// both sum every result in the same order and store the same bits.
//
// K = 9 taps in the reference's (kr, kc) order (op_nn.go:418-437), padded to 12: three MFMA steps,
// step s covering taps 4 s + lk for the lane's k group lk = lane / 16.  The pixels are the MFMA's
// rows and the filters its columns; the N order is the rows kernel's: the 2x2 windows of a
// stride-2 pooling row by row, four positions each, so a lane's four accumulator registers are
// one pooling window of one filter.
//
// The padded image lives in LDS as rows of RW floats with a zero halo, behind a run of at least
// 2 RW + 4 zero floats starting at offset 0: a lane whose pixel or tap does not exist reads from
// there (its filter operand is zero too, but 0 * inf would still be NaN).
#pragma once
#include <hip/hip_runtime.h>

namespace rows1 {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// offsets of a lane's three taps from the top-left cell of a pixel's 3x3 patch
struct LaneTaps {
  int t0, t1, t2;
  bool has2;   // tap 8 + lk exists (lk == 0)
};

__device__ __forceinline__ LaneTaps lane_taps(int lk, int RW) {
  LaneTaps L;
  const int a = lk, b = 4 + lk;   // both below 9
  L.t0 = (a / 3) * RW + a % 3;
  L.t1 = (b / 3) * RW + b % 3;
  L.t2 = 2 * RW + 2;              // tap 8
  L.has2 = lk == 0;
  return L;
}

// A lane's filter operand: column `col` of the tile (a filter, or nothing when col >= F), taps 4 s + lk.
// r: buffer descriptor over the F * 9 filter floats (a read past it gives zero).
__device__ __forceinline__ void filter_operand(__amdgpu_buffer_rsrc_t r, int col, int lk, float (&b)[3]) {
  const int v = col * 36 + lk * 4;   // bytes
  b[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, v, 0, 0));
  b[1] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, v, 16, 0));
  b[2] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, lk == 0 ? v : 0x7ffffff0, 32, 0));
}

// The pixel operand of a lane: `base` = offset of the patch's top-left cell in the padded image, or 0 for a
// pixel that does not exist.
__device__ __forceinline__ void pixel_operand(const float* raw, int base, const LaneTaps& L, float (&a)[3]) {
  a[0] = raw[base + L.t0];
  a[1] = raw[base + L.t1];
  a[2] = raw[L.has2 ? base + L.t2 : 0];
}

// One tile: 16 pixels x 16 filters, one accumulator chain per result.
__device__ __forceinline__ f32x4 tile(const float (&a)[3], const float (&b)[3]) {
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], acc, 0, 0, 0);
  return acc;
}

// The 2x2 / stride-2 max-pool of a lane's window: the pooling kernel's scan from -FLT_MAX with a
// strict compare, positions in scan order (op_nn.go:860-907).
__device__ __forceinline__ float pool_window(const f32x4& v) {
  float best = -3.402823466e+38f;
#pragma unroll
  for (int r = 0; r < 4; r++)
    if (v[r] > best) best = v[r];
  return best;
}

}  // namespace rows1
