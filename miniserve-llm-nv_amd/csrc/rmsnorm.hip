// RMSNorm with 32-bit statistics.
//   v = x (+ delta);  var = mean(v^2);  n = v * (1 / sqrt(var + eps));
//   y = w * round_to_storage(n)
// The normalised value is rounded to the storage type before the multiply by
// the weight, the order of the reference (miniserve/model/layers.py:30-34,
// csrc/rmsnorm.cu:92-105).  In 32-bit storage the rounding is the identity.
//
// One workgroup per output row.  The number of threads depends on the row
// length only, so a row's result never depends on the rest of the batch.
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
  const int threads = dim >= 2048 ? 512 : (dim >= 512 ? 256 : (dim >= 128 ? 128 : 64));
  const dim3 grid(n_out);
  const int32_t* r = static_cast<const int32_t*>(rows);
  if (dtype == MS_F32) {
    hipLaunchKernelGGL((rmsnorm_kernel<float, float>), dim3(grid), dim3(threads), 0, stream, 
        static_cast<float*>(x), static_cast<const float*>(delta), static_cast<const float*>(weight),
        static_cast<float*>(out), r, dim, eps, write_back);
  } else if (dtype == MS_BF16) {
    if (x_is_f32) {
      hipLaunchKernelGGL((rmsnorm_kernel<float, ms::bf16>), dim3(grid), dim3(threads), 0, stream, 
          static_cast<float*>(x), static_cast<const ms::bf16*>(delta), static_cast<const ms::bf16*>(weight),
          static_cast<ms::bf16*>(out), r, dim, eps, write_back);
    } else {
      hipLaunchKernelGGL((rmsnorm_kernel<ms::bf16, ms::bf16>), dim3(grid), dim3(threads), 0, stream, 
          static_cast<ms::bf16*>(x), static_cast<const ms::bf16*>(delta), static_cast<const ms::bf16*>(weight),
          static_cast<ms::bf16*>(out), r, dim, eps, write_back);
    }
  } else {
    return ms_fail("rmsnorm: unknown dtype code %d", dtype);
  }
  MS_CHECK_LAUNCH("rmsnorm");
  return 0;
}
