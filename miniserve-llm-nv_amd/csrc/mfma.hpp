// Matrix-core helpers for gfx950 (CDNA4), wave64.
//
// v_mfma_f32_16x16x32_bf16 computes C[16x16] += A[16x32] * B[32x16].  With lane
// l = 16*g + r (g = 0..3, r = 0..15):
//   A: lane holds row r,    k = 8*g + 0..7   (8 bf16, one 128-bit register group)
//   B: lane holds column r, k = 8*g + 0..7
//   C: lane holds column r, rows 4*g + 0..3  (4 floats)
// The k index is a contraction index: any assignment of real indices to the 32
// k-slots is valid as long as A and B use the same one.
//
// v_mfma_f32_32x32x16_bf16 computes C[32x32] += A[32x16] * B[16x32].  With lane
// l = 32*h + i (h = 0..1, i = 0..31):
//   A: lane holds row i,    k = 8*h + 0..7
//   B: lane holds column i, k = 8*h + 0..7
//   C: lane holds column i, register v (0..15) = row 8*(v/4) + 4*h + v%4
#pragma once

#include "common.hpp"

namespace ms {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ floatx4 mfma_16x16x32(bf16x8 a, bf16x8 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ floatx16 mfma_32x32x16(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 load_bf16x8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x4 load_bf16x4(const bf16* p) { return *reinterpret_cast<const bf16x4*>(p); }

__device__ __forceinline__ bf16x8 zero_bf16x8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = static_cast<__bf16>(0.0f);
  return z;
}

__device__ __forceinline__ bf16x4 zero_bf16x4() {
  bf16x4 z;
#pragma unroll
  for (int i = 0; i < 4; ++i) z[i] = static_cast<__bf16>(0.0f);
  return z;
}

__device__ __forceinline__ bf16x8 concat(bf16x4 lo, bf16x4 hi) {
  bf16x8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[i] = lo[i];
    r[i + 4] = hi[i];
  }
  return r;
}

}  // namespace ms
