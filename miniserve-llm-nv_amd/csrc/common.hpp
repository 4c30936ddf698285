// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of this library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Occupancy hint for a kernel: the register budget is set for `lo`..`hi` waves per SIMD.
#define MS_WAVES_PER_EU(lo, hi) __attribute__((amdgpu_waves_per_eu(lo, hi)))

namespace ms {

constexpr int kWave = 64;

// Storage types.  bfloat16 is kept as its 16 raw bits; all arithmetic is float.
struct bf16 {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t bits) {
  return __uint_as_float(static_cast<uint32_t>(bits) << 16);
}

// Round to nearest even; NaN stays NaN.  The conversion is one instruction of gfx950
// (two values at a time where the compiler finds two).
__device__ __forceinline__ uint16_t float_to_bf16_bits(float value) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(value));
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return bf16_bits_to_float(v.bits); }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16 from_float<bf16>(float v) {
  bf16 r;
  r.bits = float_to_bf16_bits(v);
  return r;
}

// Value after a round trip through the storage type (identity for float).
template <typename T>
__device__ __forceinline__ float round_to(float v) {
  return to_float(from_float<T>(v));
}

// max of a value with that of the lane 32 further (or back): one swap of the wave's
// halves on gfx950 instead of a trip through the LDS crossbar.
__device__ __forceinline__ float max_swap32(float v) {
  const auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
}

// 2^x by the hardware instruction alone (no handling of results below the smallest
// normal number, which are zero weights anyway).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// A value that is the same in every lane of the wave, moved to a scalar register so
// that what is computed from it is scalar work and branches on it are scalar branches.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Butterfly reductions over the 64 lanes of a wave; every lane gets the result
// and the order of additions is fixed, so a row's result never depends on what
// else is in the launch.
__device__ __forceinline__ float max_xor32(float v) { return max_swap32(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, kWave));
  return v;
}

__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
  return v;
}

// Sum over a workgroup of up to 1024 threads (a multiple of 64).  `scratch`
// holds one float per wave.  All threads must call it; all get the result.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();  // scratch may still be read from an earlier call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

}  // namespace ms

// ---- host side ------------------------------------------------------------

// dtype codes shared with the Python wrappers.
enum MsDtype : int { MS_F32 = 0, MS_BF16 = 1 };

// Records a message for ms_last_error() and returns a non-zero code.
int ms_fail(const char* format, ...);

// Compute units of the current device (256 on MI355X), asked once.
int ms_compute_units();

#define MS_REQUIRE(cond, ...)                \
  do {                                       \
    if (!(cond)) return ms_fail(__VA_ARGS__); \
  } while (0)

// Checks the launch itself (bad configuration); asynchronous faults are not
// visible here.
#define MS_CHECK_LAUNCH(name)                                                      \
  do {                                                                             \
    hipError_t ms_err_ = hipGetLastError();                                        \
    if (ms_err_ != hipSuccess) return ms_fail("%s: %s", name, hipGetErrorString(ms_err_)); \
  } while (0)
