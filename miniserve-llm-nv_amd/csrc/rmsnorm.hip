// RMSNorm with 32-bit statistics.
//   v = x (+ delta);  var = mean(v^2);  n = v * (1 / sqrt(var + eps));
//   y = w * round_to_storage(n)
// The normalised value is rounded to the storage type before the multiply by
// the weight, the order of the reference (miniserve/model/layers.py:30-34,
// csrc/rmsnorm.cu:92-105).  In 32-bit storage the rounding is the identity.
//
// One workgroup per output row.  The number of threads and the kernel variant
// depend on the row length and the input type only, so a row's result never depends
// on the rest of the batch nor on where its operands lie.  (The variant for the 32-bit
// residual stream in rows of a multiple of four reads 16 bytes at a time; operands
// that are not 16-byte aligned are refused there rather than served by another variant
// whose sums have another order.)
#include <type_traits>

#include "common.hpp"

namespace {

// Input of type TIn (float for the residual stream, or the storage type),
// optional delta of the storage type that is added first; when `write_back` the
// sum is stored to x (the residual update h <- h + delta, in 32-bit).
template <typename TIn, typename T>
__global__ void rmsnorm_kernel(TIn* __restrict__ x, const T* __restrict__ delta, const T* __restrict__ weight,
                               T* __restrict__ out, const int32_t* __restrict__ rows, int dim, float eps,
                               int write_back) {
  __shared__ float scratch[16];
  const int64_t out_row = blockIdx.x;
  const int64_t in_row = rows ? static_cast<int64_t>(rows[out_row]) : out_row;
  TIn* xr = x + in_row * dim;
  const T* dr = delta ? delta + in_row * dim : nullptr;
  T* yr = out + out_row * dim;

  float partial = 0.f;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    float v = ms::to_float(xr[i]);
    if (dr) {
      v += ms::to_float(dr[i]);
      if (write_back) xr[i] = ms::from_float<TIn>(v);
    }
    partial = fmaf(v, v, partial);
  }
  const float total = ms::block_sum(partial, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    float v = ms::to_float(xr[i]);
    if (dr && !write_back) v += ms::to_float(dr[i]);
    const float n = ms::round_to<T>(v * inv);
    yr[i] = ms::from_float<T>(ms::to_float(weight[i]) * n);
  }
}

// The same with the row kept in registers between the two passes: one read of the
// row instead of two.  EPT values per thread; the row has at most EPT * blockDim.x.
template <typename TIn, typename T, int EPT>
__global__ void rmsnorm_registers_kernel(TIn* __restrict__ x, const T* __restrict__ delta,
                                         const T* __restrict__ weight, T* __restrict__ out,
                                         const int32_t* __restrict__ rows, int dim, float eps, int write_back) {
  __shared__ float scratch[16];
  const int64_t out_row = blockIdx.x;
  const int64_t in_row = rows ? static_cast<int64_t>(rows[out_row]) : out_row;
  TIn* xr = x + in_row * dim;
  const T* dr = delta ? delta + in_row * dim : nullptr;
  T* yr = out + out_row * dim;

  float v[EPT];
  float partial = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = threadIdx.x + e * blockDim.x;
    v[e] = 0.f;
    if (i < dim) {
      v[e] = ms::to_float(xr[i]);
      if (dr) {
        v[e] += ms::to_float(dr[i]);
        if (write_back) {
          xr[i] = ms::from_float<TIn>(v[e]);
          v[e] = ms::round_to<TIn>(v[e]);     // what a second read of x would see
        }
      }
      partial = fmaf(v[e], v[e], partial);
    }
  }
  const float total = ms::block_sum(partial, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = threadIdx.x + e * blockDim.x;
    if (i < dim) yr[i] = ms::from_float<T>(ms::to_float(weight[i]) * ms::round_to<T>(v[e] * inv));
  }
}

// Four values of the storage type to and from floats, as one 8- or 16-byte access.
__device__ __forceinline__ void load4(const float* p, float (&f)[4]) {
  const float4 raw = *reinterpret_cast<const float4*>(p);
  f[0] = raw.x, f[1] = raw.y, f[2] = raw.z, f[3] = raw.w;
}
__device__ __forceinline__ void load4(const ms::bf16* p, float (&f)[4]) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  f[0] = __uint_as_float(raw.x << 16), f[1] = __uint_as_float(raw.x & 0xffff0000u);
  f[2] = __uint_as_float(raw.y << 16), f[3] = __uint_as_float(raw.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float (&f)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
}
__device__ __forceinline__ void store4(ms::bf16* p, const float (&f)[4]) {
  uint2 raw;
  raw.x = ms::float_to_bf16_bits(f[0]) | (static_cast<uint32_t>(ms::float_to_bf16_bits(f[1])) << 16);
  raw.y = ms::float_to_bf16_bits(f[2]) | (static_cast<uint32_t>(ms::float_to_bf16_bits(f[3])) << 16);
  *reinterpret_cast<uint2*>(p) = raw;
}

// The residual stream's norm for rows of a multiple of four values, every operand aligned
// to 16 bytes: the row in registers as above, four consecutive values a thread and access
// (one 16-byte read of the 32-bit row, one 8-byte write of the bfloat16 output), 256 threads
// for any row up to 16,384.  VPT such groups per thread.
template <typename T, int VPT>
__global__ void rmsnorm_by_fours_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                        const T* __restrict__ weight, T* __restrict__ out,
                                        const int32_t* __restrict__ rows, int dim, float eps, int write_back) {
  __shared__ float scratch[16];
  const int64_t out_row = blockIdx.x;
  const int64_t in_row = rows ? static_cast<int64_t>(rows[out_row]) : out_row;
  float* xr = x + in_row * dim;
  const T* dr = delta ? delta + in_row * dim : nullptr;
  T* yr = out + out_row * dim;
  const int groups = dim / 4;

  float v[VPT][4];
  float partial = 0.f;
#pragma unroll
  for (int e = 0; e < VPT; ++e) {
    const int i = threadIdx.x + e * blockDim.x;
    if (i < groups) {
      load4(xr + 4 * i, v[e]);
      if (dr) {
        float d[4];
        load4(dr + 4 * i, d);
#pragma unroll
        for (int c = 0; c < 4; ++c) v[e][c] += d[c];
        if (write_back) store4(xr + 4 * i, v[e]);
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) partial = fmaf(v[e][c], v[e][c], partial);
    }
  }
  const float total = ms::block_sum(partial, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
#pragma unroll
  for (int e = 0; e < VPT; ++e) {
    const int i = threadIdx.x + e * blockDim.x;
    if (i < groups) {
      float w[4], y[4];
      load4(weight + 4 * i, w);
#pragma unroll
      for (int c = 0; c < 4; ++c) y[c] = w[c] * ms::round_to<T>(v[e][c] * inv);
      store4(yr + 4 * i, y);
    }
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Whether a row of `dim` 32-bit values goes four values a thread and access.
bool by_fours(int dim) { return dim % 4 == 0 && dim >= 256 && dim <= 16384; }

template <typename TIn, typename T>
void launch_rmsnorm(void* x, const void* delta, const void* weight, void* out, const void* rows, int n_out, int dim,
                    float eps, int write_back, hipStream_t stream) {
  const dim3 grid(n_out);
  TIn* xp = static_cast<TIn*>(x);
  const T* dp = static_cast<const T*>(delta);
  const T* wp = static_cast<const T*>(weight);
  T* op = static_cast<T*>(out);
  const int32_t* rp = static_cast<const int32_t*>(rows);
  if constexpr (std::is_same<TIn, float>::value) {
    // (the choice goes by the row's length, never by the number of rows; the entry point has checked the alignment)
    if (by_fours(dim)) {
      const dim3 block(256);
#define MS_NORM_BY_FOURS(VPT)                                                                                     \
  hipLaunchKernelGGL((rmsnorm_by_fours_kernel<T, VPT>), grid, block, 0, stream, xp, dp, wp, op, rp, dim, eps, write_back)
      if (dim <= 1024) MS_NORM_BY_FOURS(1);
      else if (dim <= 2048) MS_NORM_BY_FOURS(2);
      else if (dim <= 4096) MS_NORM_BY_FOURS(4);
      else if (dim <= 8192) MS_NORM_BY_FOURS(8);
      else MS_NORM_BY_FOURS(16);
#undef MS_NORM_BY_FOURS
      return;
    }
  }
  if (dim <= 64) {
    hipLaunchKernelGGL((rmsnorm_registers_kernel<TIn, T, 1>), grid, dim3(64), 0, stream, xp, dp, wp, op, rp, dim, eps, write_back);
  } else if (dim <= 256) {
    hipLaunchKernelGGL((rmsnorm_registers_kernel<TIn, T, 4>), grid, dim3(64), 0, stream, xp, dp, wp, op, rp, dim, eps, write_back);
  } else if (dim <= 1024) {
    hipLaunchKernelGGL((rmsnorm_registers_kernel<TIn, T, 4>), grid, dim3(256), 0, stream, xp, dp, wp, op, rp, dim, eps, write_back);
  } else if (dim <= 4096) {
    hipLaunchKernelGGL((rmsnorm_registers_kernel<TIn, T, 8>), grid, dim3(512), 0, stream, xp, dp, wp, op, rp, dim, eps, write_back);
  } else if (dim <= 16384) {
    hipLaunchKernelGGL((rmsnorm_registers_kernel<TIn, T, 16>), grid, dim3(1024), 0, stream, xp, dp, wp, op, rp, dim, eps, write_back);
  } else {
    hipLaunchKernelGGL((rmsnorm_kernel<TIn, T>), grid, dim3(1024), 0, stream, xp, dp, wp, op, rp, dim, eps, write_back);
  }
}

}  // namespace

// x: [n_in, dim] (float when x_is_f32, else the storage type); delta: null or
// [n_in, dim]; rows: null (out row r reads in row r) or int32 [n_out];
// out: [n_out, dim] of the storage type.
extern "C" int ms_rmsnorm(void* x, const void* delta, const void* weight, void* out, const void* rows,
                          int n_out, int dim, float eps, int x_is_f32, int write_back, int dtype,
                          hipStream_t stream) {
  MS_REQUIRE(n_out > 0 && dim > 0, "rmsnorm: empty shape");
  MS_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive");
  MS_REQUIRE(!(write_back && rows), "rmsnorm: write_back with gathered rows is not defined");
  MS_REQUIRE(!(write_back && !delta), "rmsnorm: write_back needs a delta");
  if (x_is_f32 || dtype == MS_F32) {
    MS_REQUIRE(!by_fours(dim) || (aligned16(x) && aligned16(delta) && aligned16(weight) && aligned16(out)),
               "rmsnorm: 32-bit rows of %d values are read 16 bytes at a time; x, delta, weight and out must be "
               "16-byte aligned (a view that starts inside a row is not)", dim);
  }
  if (dtype == MS_F32) {
    launch_rmsnorm<float, float>(x, delta, weight, out, rows, n_out, dim, eps, write_back, stream);
  } else if (dtype == MS_BF16) {
    if (x_is_f32) {
      launch_rmsnorm<float, ms::bf16>(x, delta, weight, out, rows, n_out, dim, eps, write_back, stream);
    } else {
      launch_rmsnorm<ms::bf16, ms::bf16>(x, delta, weight, out, rows, n_out, dim, eps, write_back, stream);
    }
  } else {
    return ms_fail("rmsnorm: unknown dtype code %d", dtype);
  }
  MS_CHECK_LAUNCH("rmsnorm");
  return 0;
}
