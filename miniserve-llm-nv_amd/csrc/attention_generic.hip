// Paged causal attention for any head size, page size, head count and group
// size, in 32-bit arithmetic from 32-bit or bfloat16 storage.  It is the kernel
// of the 32-bit path and the fallback of the bfloat16 path for shapes that the
// MFMA kernels refuse.
//
// For the query at absolute position p of sequence s, head h (kv head h / G):
//   s_j = (sum_d q_d k_{j,d}) * scale   for lo <= j <= p
//   o_d = sum_j softmax(s)_j v_{j,d}
// with lo = 0, or p - window + 1 when a window is set
// (reference: miniserve/model/qwen3.py:243-249 for the chunk form,
//  csrc/paged_decode_attention.cu:44-94 for the one-token form; in 32-bit the
//  two are the same function).
//
// One wave per (token, head).  Keys are walked in tiles of 64 that start at
// absolute multiples of 64; lane i of a tile scores key 64*t + i, the wave does
// the online-softmax bookkeeping, then every lane accumulates its own output
// columns over the tile's keys in key order.  The order of every addition is
// fixed by (p, window, head size) alone, so the result for a position is
// bit-identical however the tokens are cut into steps, whatever else is in the
// batch and wherever the pages lie.
#include "common.hpp"

namespace {

constexpr int kMaxHeadDim = 512;
constexpr int kColumnsPerLane = kMaxHeadDim / ms::kWave;

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ q, const T* __restrict__ k, int head_dim) {
  float dot = 0.f;
  for (int d = 0; d < head_dim; ++d) dot = fmaf(q[d], ms::to_float(k[d]), dot);
  return dot;
}

template <typename T>
__global__ void attention_generic_kernel(const T* __restrict__ q, const T* __restrict__ key_pool,
                                         const T* __restrict__ value_pool, const int32_t* __restrict__ block_table,
                                         const int32_t* __restrict__ seq_of_token,
                                         const int32_t* __restrict__ positions, T* __restrict__ out,
                                         int num_q_heads, int num_kv_heads, int head_dim, int block_size,
                                         int max_blocks, float scale, int window) {
  __shared__ float q_s[kMaxHeadDim];
  __shared__ float p_s[ms::kWave];
  __shared__ int64_t value_s[ms::kWave];   // where each key's value column starts

  const int64_t token = blockIdx.x;
  const int head = blockIdx.y;
  const int lane = threadIdx.x;
  const int group = num_q_heads / num_kv_heads;
  const int kv_head = head / group;
  const int seq = seq_of_token[token];
  const int pos = positions[token];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* table = block_table + static_cast<int64_t>(seq) * max_blocks;

  const T* q_row = q + (token * num_q_heads + head) * head_dim;
  for (int d = lane; d < head_dim; d += ms::kWave) q_s[d] = ms::to_float(q_row[d]);
  __syncthreads();

  float running_max = -INFINITY;
  float running_sum = 0.f;
  float acc[kColumnsPerLane];
#pragma unroll
  for (int c = 0; c < kColumnsPerLane; ++c) acc[c] = 0.f;

  for (int tile = lo / ms::kWave; tile <= pos / ms::kWave; ++tile) {
    const int j = tile * ms::kWave + lane;
    const bool valid = j >= lo && j <= pos;
    float score = -INFINITY;
    int64_t value_start = 0;
    if (valid) {
      const int logical = j / block_size;
      const int offset = j - logical * block_size;
      const int64_t page = table[logical];
      const int64_t row = ((page * num_kv_heads + kv_head) * block_size + offset) * head_dim;
      value_start = (page * num_kv_heads + kv_head) * head_dim * block_size + offset;
      score = dot_row(q_s, key_pool + row, head_dim) * scale;
    }
    const float new_max = fmaxf(running_max, ms::wave_max(score));
    const float p = valid ? expf(score - new_max) : 0.f;
    const float alpha = (running_max == -INFINITY) ? 0.f : expf(running_max - new_max);
    running_sum = running_sum * alpha + ms::wave_sum(p);
    running_max = new_max;

    __syncthreads();  // the previous tile's readers are done
    p_s[lane] = p;
    value_s[lane] = value_start;
    __syncthreads();

    const int first = lo > tile * ms::kWave ? lo - tile * ms::kWave : 0;
    const int last = pos - tile * ms::kWave < ms::kWave - 1 ? pos - tile * ms::kWave : ms::kWave - 1;
#pragma unroll
    for (int c = 0; c < kColumnsPerLane; ++c) {
      const int d = lane + c * ms::kWave;
      if (d < head_dim) {
        float a = acc[c] * alpha;
        for (int jj = first; jj <= last; ++jj)
          a = fmaf(p_s[jj], ms::to_float(value_pool[value_s[jj] + static_cast<int64_t>(d) * block_size]), a);
        acc[c] = a;
      }
    }
  }

  T* out_row = out + (token * num_q_heads + head) * head_dim;
  const float inv_sum = 1.0f / running_sum;
#pragma unroll
  for (int c = 0; c < kColumnsPerLane; ++c) {
    const int d = lane + c * ms::kWave;
    if (d < head_dim) out_row[d] = ms::from_float<T>(acc[c] * inv_sum);
  }
}

}  // namespace

// q, out: [num_tokens, num_q_heads, head_dim]; key_pool: [num_blocks, num_kv_heads,
// block_size, head_dim]; value_pool: [num_blocks, num_kv_heads, head_dim,
// block_size]; block_table: int32 [num_seqs, max_blocks];
// seq_of_token, positions: int32 [num_tokens]; window: 0 = all keys.
extern "C" int ms_attention_generic(const void* q, const void* key_pool, const void* value_pool,
                                    const void* block_table, const void* seq_of_token, const void* positions,
                                    void* out, int num_tokens, int num_q_heads, int num_kv_heads, int head_dim,
                                    int block_size, int max_blocks, float scale, int window, int dtype,
                                    hipStream_t stream) {
  MS_REQUIRE(num_tokens > 0, "attention_generic: no tokens");
  MS_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0,
             "attention_generic: %d query heads are not a multiple of %d kv heads", num_q_heads, num_kv_heads);
  MS_REQUIRE(head_dim > 0 && head_dim <= kMaxHeadDim, "attention_generic: head_dim %d is outside 1..%d", head_dim,
             kMaxHeadDim);
  MS_REQUIRE(block_size > 0 && max_blocks > 0, "attention_generic: bad page geometry");
  MS_REQUIRE(window >= 0, "attention_generic: negative window");
  MS_REQUIRE(num_q_heads <= 65535, "attention_generic: too many heads");
  const dim3 grid(num_tokens, num_q_heads);
  if (dtype == MS_F32) {
    hipLaunchKernelGGL((attention_generic_kernel<float>), dim3(grid), dim3(ms::kWave), 0, stream, 
        static_cast<const float*>(q), static_cast<const float*>(key_pool), static_cast<const float*>(value_pool),
        static_cast<const int32_t*>(block_table), static_cast<const int32_t*>(seq_of_token),
        static_cast<const int32_t*>(positions), static_cast<float*>(out), num_q_heads, num_kv_heads, head_dim,
        block_size, max_blocks, scale, window);
  } else if (dtype == MS_BF16) {
    hipLaunchKernelGGL((attention_generic_kernel<ms::bf16>), dim3(grid), dim3(ms::kWave), 0, stream, 
        static_cast<const ms::bf16*>(q), static_cast<const ms::bf16*>(key_pool),
        static_cast<const ms::bf16*>(value_pool), static_cast<const int32_t*>(block_table),
        static_cast<const int32_t*>(seq_of_token), static_cast<const int32_t*>(positions),
        static_cast<ms::bf16*>(out), num_q_heads, num_kv_heads, head_dim, block_size, max_blocks, scale, window);
  } else {
    return ms_fail("attention_generic: unknown dtype code %d", dtype);
  }
  MS_CHECK_LAUNCH("attention_generic");
  return 0;
}
