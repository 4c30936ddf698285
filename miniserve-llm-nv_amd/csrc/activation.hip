// Gated activation of the feed-forward: out = silu(gate) * up, silu(z) = z * sigmoid(z)
// (reference: miniserve/model/layers.py:86-87).  The gate and up projections
// arrive packed in one row, gate columns first.  Computed in 32-bit, rounded once.
#include "common.hpp"

namespace {

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int64_t rows, int inter) {
  const int64_t total = rows * inter;
  for (int64_t index = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = index / inter;
    const int64_t col = index - r * inter;
    const float g = ms::to_float(gate_up[r * 2 * inter + col]);
    const float u = ms::to_float(gate_up[r * 2 * inter + inter + col]);
    const float silu = g / (1.0f + expf(-g));
    out[index] = ms::from_float<T>(silu * u);
  }
}

// The same, 8 elements a thread (16-byte loads and stores of bfloat16); the width
// must be a multiple of 8.
__global__ void silu_mul_bf16x8_kernel(const uint4* __restrict__ gate_up, uint4* __restrict__ out, int64_t rows,
                                       int inter8) {
  const int64_t total = rows * inter8;
  for (int64_t index = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = index / inter8;
    const int64_t col = index - r * inter8;
    const uint4 g4 = gate_up[r * 2 * inter8 + col];
    const uint4 u4 = gate_up[r * 2 * inter8 + inter8 + col];
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w};
    const uint32_t uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t ow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float m[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float g = ms::bf16_bits_to_float(static_cast<uint16_t>(gw[i] >> (16 * h)));
        const float u = ms::bf16_bits_to_float(static_cast<uint16_t>(uw[i] >> (16 * h)));
        m[h] = g / (1.0f + expf(-g)) * u;
      }
      ow[i] = static_cast<uint32_t>(ms::float_to_bf16_bits(m[0])) |
              (static_cast<uint32_t>(ms::float_to_bf16_bits(m[1])) << 16);
    }
    out[index] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

}  // namespace

// gate_up: [rows, 2*inter]; out: [rows, inter].
extern "C" int ms_silu_mul(const void* gate_up, void* out, int rows, int inter, int dtype, hipStream_t stream) {
  MS_REQUIRE(rows > 0 && inter > 0, "silu_mul: empty shape");
  const int64_t total = static_cast<int64_t>(rows) * inter;
  const int threads = 256;
  int64_t blocks = (total + threads - 1) / threads;
  if (blocks > 65536) blocks = 65536;
  if (dtype == MS_F32) {
    hipLaunchKernelGGL((silu_mul_kernel<float>), dim3(blocks), dim3(threads), 0, stream, static_cast<const float*>(gate_up),
                                                                 static_cast<float*>(out), rows, inter);
  } else if (dtype == MS_BF16 && inter % 8 == 0) {
    int64_t wide_blocks = (total / 8 + threads - 1) / threads;
    if (wide_blocks > 65536) wide_blocks = 65536;
    hipLaunchKernelGGL(silu_mul_bf16x8_kernel, dim3(wide_blocks), dim3(threads), 0, stream,
                       static_cast<const uint4*>(gate_up), static_cast<uint4*>(out), static_cast<int64_t>(rows),
                       inter / 8);
  } else if (dtype == MS_BF16) {
    hipLaunchKernelGGL((silu_mul_kernel<ms::bf16>), dim3(blocks), dim3(threads), 0, stream, static_cast<const ms::bf16*>(gate_up),
                                                                    static_cast<ms::bf16*>(out), rows, inter);
  } else {
    return ms_fail("silu_mul: unknown dtype code %d", dtype);
  }
  MS_CHECK_LAUNCH("silu_mul");
  return 0;
}

namespace {

template <typename T>
__global__ void residual_add_kernel(float* __restrict__ h, const T* __restrict__ delta, int64_t total) {
  for (int64_t index = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    h[index] += ms::to_float(delta[index]);
  }
}

}  // namespace

// Residual update in 32-bit: h[rows, dim] (float) += delta[rows, dim] (storage type).
extern "C" int ms_residual_add(void* h, const void* delta, int rows, int dim, int dtype, hipStream_t stream) {
  MS_REQUIRE(rows > 0 && dim > 0, "residual_add: empty shape");
  const int64_t total = static_cast<int64_t>(rows) * dim;
  const int threads = 256;
  int64_t blocks = (total + threads - 1) / threads;
  if (blocks > 65536) blocks = 65536;
  if (dtype == MS_F32) {
    hipLaunchKernelGGL((residual_add_kernel<float>), dim3(blocks), dim3(threads), 0, stream, static_cast<float*>(h),
                                                                     static_cast<const float*>(delta), total);
  } else if (dtype == MS_BF16) {
    hipLaunchKernelGGL((residual_add_kernel<ms::bf16>), dim3(blocks), dim3(threads), 0, stream, 
        static_cast<float*>(h), static_cast<const ms::bf16*>(delta), total);
  } else {
    return ms_fail("residual_add: unknown dtype code %d", dtype);
  }
  MS_CHECK_LAUNCH("residual_add");
  return 0;
}
