// Per-head RMSNorm of q and k, half-split rotary embedding, and the write of
// K and V into their pages, in one pass over the packed projection output.
//
//   q,k: n = x * (1/sqrt(mean(x^2)+eps)); y = w * round(n)      (per head, over D)
//        reference: miniserve/model/qwen3.py:177-178, layers.py:30-34
//   rotary (half-split pairs i, i+D/2), cos and sin of angle = float(pos) * inv_freq[i]
//   from a table that is made once per step for all layers:
//        y'[i]     = y[i]*cos - y[i+D/2]*sin
//        y'[i+D/2] = y[i+D/2]*cos + y[i]*sin
//        reference: miniserve/model/rope.py:24-52
//   cache write: slot = page*block_size + offset; keys to key_pool[page, kv_head,
//        offset, :], values transposed to value_pool[page, kv_head, :, offset]
//        (the layout the matrix-core attention kernels read without a shuffle)
//        reference: csrc/paged_kv_append.cu:28-43
//
// The rotation is done in 32-bit on the storage-rounded norm output and rounded
// once.  Each (token, head) is one wave; nothing depends on the batch.
#include "common.hpp"

namespace {

constexpr int kMaxPairsPerLane = 4;  // head_dim <= 512

template <typename T>
__global__ void qk_norm_rope_append_kernel(const T* __restrict__ packed, const T* __restrict__ q_weight,
                                           const T* __restrict__ k_weight, const float* __restrict__ cos_table,
                                           const float* __restrict__ sin_table,
                                           const int32_t* __restrict__ slot_mapping, T* __restrict__ q_out,
                                           T* __restrict__ key_pool, T* __restrict__ value_pool, int num_q_heads,
                                           int num_kv_heads, int head_dim, int block_size, float eps) {
  const int64_t token = blockIdx.x;
  const int head = blockIdx.y;
  const int lane = threadIdx.x;
  const int half = head_dim / 2;
  const int packed_heads = num_q_heads + 2 * num_kv_heads;
  const T* row = packed + (token * packed_heads + head) * head_dim;

  const bool is_q = head < num_q_heads;
  const bool is_k = !is_q && head < num_q_heads + num_kv_heads;
  const int kv_head = is_q ? 0 : (is_k ? head - num_q_heads : head - num_q_heads - num_kv_heads);

  T* dst;
  int64_t dst_stride = 1;   // distance between consecutive d
  if (is_q) {
    dst = q_out + (token * num_q_heads + head) * head_dim;
  } else {
    const int64_t slot = slot_mapping[token];
    const int64_t page = slot / block_size;
    const int64_t offset = slot - page * block_size;
    if (is_k) {
      dst = key_pool + ((page * num_kv_heads + kv_head) * block_size + offset) * head_dim;
    } else {
      dst = value_pool + (page * num_kv_heads + kv_head) * head_dim * block_size + offset;
      dst_stride = block_size;
    }
  }

  float lo[kMaxPairsPerLane], hi[kMaxPairsPerLane];
  float partial = 0.f;
#pragma unroll
  for (int c = 0; c < kMaxPairsPerLane; ++c) {
    const int i = lane + c * ms::kWave;
    lo[c] = hi[c] = 0.f;
    if (i < half) {
      lo[c] = ms::to_float(row[i]);
      hi[c] = ms::to_float(row[i + half]);
      partial = fmaf(lo[c], lo[c], partial);
      partial = fmaf(hi[c], hi[c], partial);
    }
  }

  const T* weight = is_q ? q_weight : (is_k ? k_weight : nullptr);
  if (weight) {
    const float total = ms::wave_sum(partial);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(head_dim) + eps);
#pragma unroll
    for (int c = 0; c < kMaxPairsPerLane; ++c) {
      const int i = lane + c * ms::kWave;
      if (i < half) {
        lo[c] = ms::round_to<T>(ms::to_float(weight[i]) * ms::round_to<T>(lo[c] * inv));
        hi[c] = ms::round_to<T>(ms::to_float(weight[i + half]) * ms::round_to<T>(hi[c] * inv));
      }
    }
  }

  const bool rotate = cos_table != nullptr && (is_q || is_k);
#pragma unroll
  for (int c = 0; c < kMaxPairsPerLane; ++c) {
    const int i = lane + c * ms::kWave;
    if (i < half) {
      float a = lo[c], b = hi[c];
      if (rotate) {
        const float cs = cos_table[token * half + i];
        const float sn = sin_table[token * half + i];
        const float ra = a * cs - b * sn;
        const float rb = b * cs + a * sn;
        a = ra;
        b = rb;
      }
      dst[i * dst_stride] = ms::from_float<T>(a);
      dst[(i + half) * dst_stride] = ms::from_float<T>(b);
    }
  }
}

template <typename T>
int launch(const void* packed, const void* q_weight, const void* k_weight, const void* cos_table,
           const void* sin_table, const void* slot_mapping, void* q_out, void* key_pool, void* value_pool,
           int num_tokens, int num_q_heads, int num_kv_heads, int head_dim, int block_size, float eps,
           hipStream_t stream) {
  const dim3 grid(num_tokens, num_q_heads + 2 * num_kv_heads);
  hipLaunchKernelGGL((qk_norm_rope_append_kernel<T>), dim3(grid), dim3(ms::kWave), 0, stream, 
      static_cast<const T*>(packed), static_cast<const T*>(q_weight), static_cast<const T*>(k_weight),
      static_cast<const float*>(cos_table), static_cast<const float*>(sin_table),
      static_cast<const int32_t*>(slot_mapping), static_cast<T*>(q_out), static_cast<T*>(key_pool),
      static_cast<T*>(value_pool), num_q_heads, num_kv_heads, head_dim, block_size, eps);
  return 0;
}

// cos and sin of float(position) * inv_freq[i], in 32-bit, for every token of the step.
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float* __restrict__ cos_table, float* __restrict__ sin_table, int64_t total, int half) {
  const int64_t index = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (index >= total) return;
  const int64_t token = index / half;
  const int i = static_cast<int>(index - token * half);
  const float angle = static_cast<float>(positions[token]) * inv_freq[i];
  float sn, cs;
  sincosf(angle, &sn, &cs);
  cos_table[index] = cs;
  sin_table[index] = sn;
}

}  // namespace

// positions: int32 [num_tokens]; inv_freq: float [half]; cos_table, sin_table: float [num_tokens, half].
extern "C" int ms_rope_table(const void* positions, const void* inv_freq, void* cos_table, void* sin_table,
                             int num_tokens, int half, hipStream_t stream) {
  MS_REQUIRE(num_tokens > 0 && half > 0, "rope_table: empty shape");
  const int64_t total = static_cast<int64_t>(num_tokens) * half;
  hipLaunchKernelGGL(rope_table_kernel, dim3((total + 255) / 256), dim3(256), 0, stream,
                     static_cast<const int32_t*>(positions), static_cast<const float*>(inv_freq),
                     static_cast<float*>(cos_table), static_cast<float*>(sin_table), total, half);
  MS_CHECK_LAUNCH("rope_table");
  return 0;
}

// packed: [num_tokens, (num_q_heads + 2*num_kv_heads) * head_dim], heads in the
// order q..., k..., v....  q_weight/k_weight: [head_dim] or null (no norm).
// cos_table, sin_table: float [num_tokens, head_dim/2] (from ms_rope_table) or both
// null (no rotation).  With num_kv_heads == 0
// nothing is written to a cache and slot_mapping/pools may be null.
extern "C" int ms_qk_norm_rope_append(const void* packed, const void* q_weight, const void* k_weight,
                                      const void* cos_table, const void* sin_table, const void* slot_mapping,
                                      void* q_out, void* key_pool, void* value_pool, int num_tokens,
                                      int num_q_heads, int num_kv_heads, int head_dim, int block_size, float eps,
                                      int dtype, hipStream_t stream) {
  MS_REQUIRE(num_tokens > 0 && head_dim > 0, "qk_norm_rope_append: empty shape");
  MS_REQUIRE(num_q_heads >= 0 && num_kv_heads >= 0 && num_q_heads + num_kv_heads > 0,
             "qk_norm_rope_append: no heads");
  MS_REQUIRE(head_dim % 2 == 0, "qk_norm_rope_append: head_dim %d must be even", head_dim);
  MS_REQUIRE(head_dim <= 2 * ms::kWave * kMaxPairsPerLane, "qk_norm_rope_append: head_dim %d exceeds %d",
             head_dim, 2 * ms::kWave * kMaxPairsPerLane);
  MS_REQUIRE(num_q_heads == 0 || q_out != nullptr, "qk_norm_rope_append: q_out is null");
  if (num_kv_heads > 0) {
    MS_REQUIRE(slot_mapping && key_pool && value_pool && block_size > 0,
               "qk_norm_rope_append: cache write needs slot_mapping, pools and block_size");
  }
  MS_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "qk_norm_rope_append: rotation needs both tables");
  MS_REQUIRE(num_q_heads + 2 * num_kv_heads <= 65535, "qk_norm_rope_append: too many heads");
  int rc;
  if (dtype == MS_F32) {
    rc = launch<float>(packed, q_weight, k_weight, cos_table, sin_table, slot_mapping, q_out, key_pool, value_pool,
                       num_tokens, num_q_heads, num_kv_heads, head_dim, block_size, eps, stream);
  } else if (dtype == MS_BF16) {
    rc = launch<ms::bf16>(packed, q_weight, k_weight, cos_table, sin_table, slot_mapping, q_out, key_pool,
                          value_pool, num_tokens, num_q_heads, num_kv_heads, head_dim, block_size, eps, stream);
  } else {
    return ms_fail("qk_norm_rope_append: unknown dtype code %d", dtype);
  }
  MS_CHECK_LAUNCH("qk_norm_rope_append");
  return rc;
}
