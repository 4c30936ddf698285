// Next-token choice on the device: greedy argmax, or temperature -> top-k ->
// top-p -> softmax -> one draw, the order of the reference
// (miniserve/model/sampling.py:61-79).  The draw is the inverse CDF, in token
// order, of a uniform number that the host supplies per row, so a host
// implementation with the same number picks the same token.
//
// One workgroup of 1024 threads per row of 32-bit logits; any vocabulary size.
//   temperature == 0      : argmax, lowest index among equals
//   x = logit / temperature
//   top-k (0 = off)       : keep the k largest x; among values equal to the
//                           k-th largest the lowest indices, so exactly k stay
//   top-p (1 = off)       : in descending order of x, keep a token iff the
//                           probability mass strictly ahead of it is <= top_p
//                           (the token that crosses the threshold stays, the
//                           first token always stays); tokens with equal x are
//                           kept or dropped together
//   draw                  : first index whose running sum of exp(x - max) over
//                           the kept tokens exceeds uniform * total
// A row with a NaN or infinite logit yields -1.
#include "common.hpp"

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / ms::kWave;

// Monotone map from float to unsigned: a < b  <=>  ordered(a) < ordered(b).
__device__ __forceinline__ uint32_t ordered(float value) {
  const uint32_t u = __float_as_uint(value);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
  v = ms::wave_sum_int(v);
  __syncthreads();
  if ((threadIdx.x & (ms::kWave - 1)) == 0) scratch[threadIdx.x / ms::kWave] = v;
  __syncthreads();
  int total = 0;
  for (int w = 0; w < kWaves; ++w) total += scratch[w];
  return total;
}

struct Keep {
  uint32_t k_threshold;  // ordered value of the k-th largest (0: top-k off)
  int tie_limit;         // values equal to k_threshold are kept up to this index
  uint32_t p_threshold;  // keep ordered(x) >= this (0: top-p off)
  __device__ __forceinline__ bool operator()(uint32_t o, int index) const {
    if (o < p_threshold) return false;
    if (o > k_threshold) return true;
    return o == k_threshold && index <= tie_limit;
  }
};

__global__ __launch_bounds__(kThreads) void sample_rows_kernel(const float* __restrict__ logits,
                                                               const float* __restrict__ temperature,
                                                               const int32_t* __restrict__ top_k,
                                                               const float* __restrict__ top_p,
                                                               const float* __restrict__ uniform,
                                                               int32_t* __restrict__ out, int vocab) {
  __shared__ float f_scratch[kWaves];
  __shared__ int i_scratch[kWaves];
  __shared__ float seg_sum[kThreads];
  __shared__ int seg_count[kThreads];
  __shared__ int shared_index;
  __shared__ float shared_total;

  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  const float temp = temperature ? temperature[row] : 0.f;

  // Contiguous segment of this thread, for everything that needs token order.
  const int seg = (vocab + kThreads - 1) / kThreads;
  const int seg_begin = min(tid * seg, vocab);
  const int seg_end = min(seg_begin + seg, vocab);

  // ---- finiteness, maximum and its lowest index ---------------------------
  float best = -INFINITY;
  int best_index = vocab;
  int bad = 0;
  for (int i = tid; i < vocab; i += kThreads) {
    const float v = x[i];
    if (!(fabsf(v) <= 3.402823466e38f)) bad = 1;  // NaN or infinite
    if (v > best) {
      best = v;
      best_index = i;
    }
  }
  bad = block_sum_int(bad, i_scratch);
  const float row_max = ms::block_max(best, f_scratch);
  if (bad) {
    if (tid == 0) out[row] = -1;
    return;
  }
  if (temp == 0.f) {
    if (tid == 0) shared_index = vocab;
    __syncthreads();
    if (best == row_max) atomicMin(&shared_index, best_index);
    __syncthreads();
    if (tid == 0) out[row] = shared_index;
    return;
  }

  Keep keep;
  keep.k_threshold = 0u;
  keep.tie_limit = vocab;
  keep.p_threshold = 0u;
  const float scaled_max = row_max / temp;

  // ---- top-k ----------------------------------------------------------------
  const int k = top_k ? top_k[row] : 0;
  if (k > 0 && k < vocab) {
    uint32_t threshold = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t candidate = threshold | (1u << bit);
      int count = 0;
      for (int i = tid; i < vocab; i += kThreads) count += ordered(x[i] / temp) >= candidate;
      if (block_sum_int(count, i_scratch) >= k) threshold = candidate;
    }
    int greater = 0, equal = 0;
    for (int i = seg_begin; i < seg_end; ++i) {
      const uint32_t o = ordered(x[i] / temp);
      greater += o > threshold;
      equal += o == threshold;
    }
    const int total_greater = block_sum_int(greater, i_scratch);
    const int wanted = k - total_greater;  // >= 1 equal values to keep, lowest indices first
    seg_count[tid] = equal;
    __syncthreads();
    if (tid == 0) {
      int running = 0;
      for (int t = 0; t < kThreads; ++t) {
        const int c = seg_count[t];
        seg_count[t] = running;  // exclusive prefix
        running += c;
      }
      shared_index = vocab;
    }
    __syncthreads();
    int seen = seg_count[tid];
    for (int i = seg_begin; i < seg_end; ++i) {
      if (ordered(x[i] / temp) == threshold) {
        ++seen;
        if (seen == wanted) shared_index = i;  // exactly one thread reaches `wanted`
      }
    }
    __syncthreads();
    keep.k_threshold = threshold;
    keep.tie_limit = shared_index;
    __syncthreads();
  }

  // ---- top-p ----------------------------------------------------------------
  const float p = top_p ? top_p[row] : 1.f;
  if (p < 1.f) {
    float mass = 0.f;
    for (int i = seg_begin; i < seg_end; ++i) {
      const float v = x[i] / temp;
      if (keep(ordered(v), i)) mass += expf(v - scaled_max);
    }
    const float limit = p * ms::block_sum(mass, f_scratch);
    // Largest t with mass{ordered >= t} > limit; tokens at or above it stay.
    uint32_t threshold = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t candidate = threshold | (1u << bit);
      float part = 0.f;
      for (int i = seg_begin; i < seg_end; ++i) {
        const float v = x[i] / temp;
        const uint32_t o = ordered(v);
        if (o >= candidate && keep(o, i)) part += expf(v - scaled_max);
      }
      if (ms::block_sum(part, f_scratch) > limit) threshold = candidate;
    }
    keep.p_threshold = threshold;
  }

  // ---- draw -----------------------------------------------------------------
  float mine = 0.f;
  int last_kept = -1;
  for (int i = seg_begin; i < seg_end; ++i) {
    const float v = x[i] / temp;
    if (keep(ordered(v), i)) {
      mine += expf(v - scaled_max);
      last_kept = i;
    }
  }
  seg_sum[tid] = mine;
  seg_count[tid] = last_kept;
  __syncthreads();
  if (tid == 0) {
    float running = 0.f;
    int last = -1;
    for (int t = 0; t < kThreads; ++t) {
      const float s = seg_sum[t];
      seg_sum[t] = running;  // exclusive prefix, in token order
      running += s;
      if (seg_count[t] > last) last = seg_count[t];
    }
    shared_total = running;
    shared_index = last;  // fallback: the last kept token
  }
  __syncthreads();
  const float target = uniform[row] * shared_total;
  __syncthreads();
  float running = seg_sum[tid];
  for (int i = seg_begin; i < seg_end; ++i) {
    const float v = x[i] / temp;
    if (keep(ordered(v), i)) {
      running += expf(v - scaled_max);
      if (running > target) {
        atomicMin(&shared_index, i);
        break;
      }
    }
  }
  __syncthreads();
  if (tid == 0) out[row] = shared_index;
}

// Greedy choice for large vocabularies in two stages, so that a row is read by many
// workgroups: stage 1 finds (maximum, its lowest index, any non-finite value) per
// chunk of the row, stage 2 per row.
constexpr int kArgmaxThreads = 256;

__global__ __launch_bounds__(kArgmaxThreads) void argmax_chunks_kernel(const float* __restrict__ logits,
                                                                       float* __restrict__ chunk_max,
                                                                       int32_t* __restrict__ chunk_index, int vocab,
                                                                       int chunks) {
  __shared__ float f_scratch[kArgmaxThreads / ms::kWave];
  __shared__ int i_scratch[kArgmaxThreads / ms::kWave];
  __shared__ int shared_index;
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int per_chunk = (vocab + chunks - 1) / chunks;
  const int begin = chunk * per_chunk, end = min(begin + per_chunk, vocab);
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  float best = -INFINITY;
  int best_index = vocab, bad = 0;
  for (int i = begin + threadIdx.x; i < end; i += kArgmaxThreads) {
    const float v = x[i];
    if (!(fabsf(v) <= 3.402823466e38f)) bad = 1;
    if (v > best) {
      best = v;
      best_index = i;
    }
  }
  bad = ms::wave_sum_int(bad);
  if ((threadIdx.x & (ms::kWave - 1)) == 0) i_scratch[threadIdx.x / ms::kWave] = bad;
  if (threadIdx.x == 0) shared_index = vocab;
  const float chunk_best = ms::block_max(best, f_scratch);    // has barriers: i_scratch and shared_index are visible
  if (best == chunk_best) atomicMin(&shared_index, best_index);
  __syncthreads();
  if (threadIdx.x == 0) {
    int any_bad = 0;
    for (int w = 0; w < kArgmaxThreads / ms::kWave; ++w) any_bad += i_scratch[w];
    chunk_max[row * chunks + chunk] = chunk_best;
    chunk_index[row * chunks + chunk] = any_bad ? -1 : shared_index;
  }
}

// One wave per row over at most 64 chunks.
__global__ void argmax_rows_kernel(const float* __restrict__ chunk_max, const int32_t* __restrict__ chunk_index,
                                   int32_t* __restrict__ out, int chunks) {
  const int row = blockIdx.x, lane = threadIdx.x;
  const bool live = lane < chunks;
  const float value = live ? chunk_max[row * chunks + lane] : -INFINITY;
  const int index = live ? chunk_index[row * chunks + lane] : 0x7fffffff;
  const int bad = ms::wave_sum_int(live && index < 0);
  const float best = ms::wave_max(value);
  int candidate = (live && value == best && index >= 0) ? index : 0x7fffffff;
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) candidate = min(candidate, __shfl_xor(candidate, offset, ms::kWave));
  if (lane == 0) out[row] = bad ? -1 : candidate;
}

}  // namespace

// Greedy tokens of float logits [rows, vocab] through `chunks` (1..64) partial
// results per row: chunk_max float [rows, chunks], chunk_index int32 [rows, chunks].
extern "C" int ms_argmax_rows(const void* logits, void* chunk_max, void* chunk_index, void* out, int rows,
                              int vocab, int chunks, hipStream_t stream) {
  MS_REQUIRE(rows > 0 && rows <= 65535 && vocab > 0, "argmax_rows: bad shape %d x %d", rows, vocab);
  MS_REQUIRE(chunks >= 1 && chunks <= ms::kWave && chunks <= vocab, "argmax_rows: %d chunks", chunks);
  hipLaunchKernelGGL(argmax_chunks_kernel, dim3(chunks, rows), dim3(kArgmaxThreads), 0, stream,
                     static_cast<const float*>(logits), static_cast<float*>(chunk_max),
                     static_cast<int32_t*>(chunk_index), vocab, chunks);
  MS_CHECK_LAUNCH("argmax_chunks");
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(ms::kWave), 0, stream,
                     static_cast<const float*>(chunk_max), static_cast<const int32_t*>(chunk_index),
                     static_cast<int32_t*>(out), chunks);
  MS_CHECK_LAUNCH("argmax_rows");
  return 0;
}

// logits: float [rows, vocab]; temperature, top_p, uniform: float [rows] (null
// temperature = all rows greedy); top_k: int32 [rows]; out: int32 [rows].
extern "C" int ms_sample_rows(const void* logits, const void* temperature, const void* top_k, const void* top_p,
                              const void* uniform, void* out, int rows, int vocab, hipStream_t stream) {
  MS_REQUIRE(rows > 0 && vocab > 0, "sample_rows: empty shape");
  MS_REQUIRE(!temperature || uniform, "sample_rows: sampling rows need uniform numbers");
  hipLaunchKernelGGL(sample_rows_kernel, dim3(rows), dim3(kThreads), 0, stream, 
      static_cast<const float*>(logits), static_cast<const float*>(temperature),
      static_cast<const int32_t*>(top_k), static_cast<const float*>(top_p), static_cast<const float*>(uniform),
      static_cast<int32_t*>(out), vocab);
  MS_CHECK_LAUNCH("sample_rows");
  return 0;
}
