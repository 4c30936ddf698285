// True 32-bit matrix product for the float32 path: C[M,N] (+)= A[M,K] * W[N,K]^T
// with plain FMA (no matrix-core mode, no reduced precision anywhere).
//
// Every output element is accumulated by one thread over k = 0..K-1 in order,
// so the value of C[m,n] depends on row m of A and row n of W alone: it is
// bit-identical for any M, for any position of the row in the batch.
#include "common.hpp"

namespace {

constexpr int kTileM = 64, kTileN = 64, kTileK = 16;

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                       float* __restrict__ c, int m, int n, int k,
                                                       int accumulate) {
  __shared__ float a_s[kTileK][kTileM + 4];
  __shared__ float w_s[kTileK][kTileN + 4];

  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * kTileM, n0 = blockIdx.x * kTileN;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // Each thread stages 4 elements of A and 4 of W per k-tile: element e of the
  // 64x16 tile has row e / 16 and column e % 16.
  for (int k0 = 0; k0 < k; k0 += kTileK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int index = tid + e * 256;
      const int r = index / kTileK, col = index % kTileK;
      const int gk = k0 + col;
      const int gm = m0 + r, gn = n0 + r;
      a_s[col][r] = (gm < m && gk < k) ? a[static_cast<int64_t>(gm) * k + gk] : 0.f;
      w_s[col][r] = (gn < n && gk < k) ? w[static_cast<int64_t>(gn) * k + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTileK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = a_s[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = w_s[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= n) continue;
      float* dst = c + static_cast<int64_t>(gm) * n + gn;
      *dst = accumulate ? *dst + acc[i][j] : acc[i][j];
    }
  }
}

}  // namespace

// a: [m, k], w: [n, k], c: [m, n], all float, row-major and dense.
extern "C" int ms_gemm_f32(const void* a, const void* w, void* c, int m, int n, int k, int accumulate,
                           hipStream_t stream) {
  MS_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_f32: empty shape %d x %d x %d", m, n, k);
  const dim3 grid((n + kTileN - 1) / kTileN, (m + kTileM - 1) / kTileM);
  MS_REQUIRE(grid.y <= 65535, "gemm_f32: %d rows exceed the grid limit", m);
  hipLaunchKernelGGL(gemm_f32_kernel, dim3(grid), dim3(256), 0, stream, static_cast<const float*>(a), static_cast<const float*>(w),
                                            static_cast<float*>(c), m, n, k, accumulate);
  MS_CHECK_LAUNCH("gemm_f32");
  return 0;
}
