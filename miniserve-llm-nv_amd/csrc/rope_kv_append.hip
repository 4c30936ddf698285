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

  // Everything the row needs is asked for at once (the row, the norm's weight, the
  // angles): one round trip to memory, not three behind one another.
  const T* weight = is_q ? q_weight : (is_k ? k_weight : nullptr);
  const bool rotate = cos_table != nullptr && (is_q || is_k);
  // The loads leave their values untouched (a value that is used behind a branch is
  // waited for behind that branch, before the next load goes out); they are turned
  // into floats when all are on their way.
  T raw_lo[kMaxPairsPerLane], raw_hi[kMaxPairsPerLane], raw_w_lo[kMaxPairsPerLane], raw_w_hi[kMaxPairsPerLane];
  float cs[kMaxPairsPerLane], sn[kMaxPairsPerLane];
#pragma unroll
  for (int c = 0; c < kMaxPairsPerLane; ++c) {
    const int i = min(lane + c * ms::kWave, half - 1);      // lanes past the end read the last pair and store nothing
    if (c * ms::kWave < half) {
      raw_lo[c] = row[i];
      raw_hi[c] = row[i + half];
      if (weight) {
        raw_w_lo[c] = weight[i];
        raw_w_hi[c] = weight[i + half];
      }
      if (rotate) {
        cs[c] = cos_table[token * half + i];
        sn[c] = sin_table[token * half + i];
      }
    }
  }
  const int slot = is_q ? 0 : slot_mapping[token];      // asked for behind the row's loads, not ahead of them
  float lo[kMaxPairsPerLane], hi[kMaxPairsPerLane], w_lo[kMaxPairsPerLane], w_hi[kMaxPairsPerLane];
#pragma unroll
  for (int c = 0; c < kMaxPairsPerLane; ++c) {
    const bool live = lane + c * ms::kWave < half;
    const bool loaded = c * ms::kWave < half;
    lo[c] = live ? ms::to_float(raw_lo[c]) : 0.f;
    hi[c] = live ? ms::to_float(raw_hi[c]) : 0.f;
    w_lo[c] = (loaded && weight) ? ms::to_float(raw_w_lo[c]) : 1.f;
    w_hi[c] = (loaded && weight) ? ms::to_float(raw_w_hi[c]) : 1.f;
    if (!(loaded && rotate)) {
      cs[c] = 1.f;
      sn[c] = 0.f;
    }
  }

  // Where the row goes.  The slot is asked for with the row; the address is made from
  // it only here, so that the wait for it is the wait for the row.
  T* dst;
  int64_t dst_stride = 1;   // distance between consecutive d
  if (is_q) {
    dst = q_out + (token * num_q_heads + head) * head_dim;
  } else {
    const int page = slot / block_size;           // 32-bit: a slot number is below 2^31
    const int offset = slot - page * block_size;
    if (is_k) {
      dst = key_pool + ((static_cast<int64_t>(page) * num_kv_heads + kv_head) * block_size + offset) * head_dim;
    } else {
      dst = value_pool + (static_cast<int64_t>(page) * num_kv_heads + kv_head) * head_dim * block_size + offset;
      dst_stride = block_size;
    }
  }

  if (weight) {
    float partial = 0.f;
#pragma unroll
    for (int c = 0; c < kMaxPairsPerLane; ++c) {
      partial = fmaf(lo[c], lo[c], partial);
      partial = fmaf(hi[c], hi[c], partial);
    }
    const float total = ms::wave_sum(partial);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(head_dim) + eps);
#pragma unroll
    for (int c = 0; c < kMaxPairsPerLane; ++c) {
      lo[c] = ms::round_to<T>(w_lo[c] * ms::round_to<T>(lo[c] * inv));
      hi[c] = ms::round_to<T>(w_hi[c] * ms::round_to<T>(hi[c] * inv));
    }
  }

#pragma unroll
  for (int c = 0; c < kMaxPairsPerLane; ++c) {
    const int i = lane + c * ms::kWave;
    if (i < half) {
      float a = lo[c], b = hi[c];
      if (rotate) {
        const float ra = a * cs[c] - b * sn[c];
        const float rb = b * cs[c] + a * sn[c];
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

// ---- the same for head sizes in steps of 16, 16 bytes a lane ----------------
//
// A workgroup takes one head of a tile of consecutive tokens; a (token, head) row is
// held by head_dim / 16 lanes, each with 8 elements of the lower and the matching 8
// of the upper half.  The squares are summed through LDS in a fixed order.  Values
// go through LDS to be written transposed: runs of tokens in consecutive slots that
// fill an aligned 16 bytes of a page's row are written by one store.

constexpr int kTiledThreads = 256;
constexpr int kTiledMaxElements = kTiledThreads * 16;   // elements of one head of a tile
constexpr int kTiledHeads = 4;                          // query and key heads that one workgroup rotates

__device__ __forceinline__ void unpack8(const uint4& raw, float out[8]) {
  const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[2 * i] = ms::bf16_bits_to_float(static_cast<uint16_t>(words[i]));
    out[2 * i + 1] = ms::bf16_bits_to_float(static_cast<uint16_t>(words[i] >> 16));
  }
}

__device__ __forceinline__ void load8(const float* src, float out[8]) {
  const float4 a = *reinterpret_cast<const float4*>(src);
  const float4 b = *reinterpret_cast<const float4*>(src + 4);
  out[0] = a.x, out[1] = a.y, out[2] = a.z, out[3] = a.w;
  out[4] = b.x, out[5] = b.y, out[6] = b.z, out[7] = b.w;
}

__device__ __forceinline__ void store8(ms::bf16* dst, const float in[8]) {
  uint32_t words[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    words[i] = static_cast<uint32_t>(ms::float_to_bf16_bits(in[2 * i])) |
               (static_cast<uint32_t>(ms::float_to_bf16_bits(in[2 * i + 1])) << 16);
  *reinterpret_cast<uint4*>(dst) = make_uint4(words[0], words[1], words[2], words[3]);
}

template <typename T>
__global__ __launch_bounds__(kTiledThreads) void qk_norm_rope_append_tiled_kernel(
    const T* __restrict__ packed, const T* __restrict__ q_weight, const T* __restrict__ k_weight,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table,
    const int32_t* __restrict__ slot_mapping, T* __restrict__ q_out, T* __restrict__ key_pool,
    T* __restrict__ value_pool, int num_tokens, int num_q_heads, int num_kv_heads, int head_dim, int block_size,
    float eps) {
  constexpr int kGroup = 16 / static_cast<int>(sizeof(T));   // values of one 16-byte store
  __shared__ float square_s[kTiledHeads][kTiledThreads];
  __shared__ int32_t slot_s[kTiledThreads];
  __shared__ bool whole_s[kTiledThreads];
  __shared__ __align__(16) T tile_s[kTiledMaxElements];

  // blockIdx.y: first the groups of kTiledHeads query and key heads (one workgroup reads
  // the tile's cos and sin once for all of them), then one block per value head
  const int half = head_dim / 2;
  const int lanes_per_row = half / 8;
  const int tile_tokens = kTiledThreads / lanes_per_row;
  const int rotated_heads = num_q_heads + num_kv_heads;
  const int rotated_groups = (rotated_heads + kTiledHeads - 1) / kTiledHeads;
  const int64_t first_token = static_cast<int64_t>(blockIdx.x) * tile_tokens;
  const int live_tokens = static_cast<int>(min(static_cast<int64_t>(tile_tokens), num_tokens - first_token));
  const int item = threadIdx.x / lanes_per_row;
  const int part = threadIdx.x - item * lanes_per_row;
  const bool live = item < live_tokens;
  const int64_t token = first_token + (live ? item : 0);
  const int packed_heads = num_q_heads + 2 * num_kv_heads;

  if (static_cast<int>(blockIdx.y) >= rotated_groups) {
    // values: through LDS, written along the page's offset axis
    const int kv_head = static_cast<int>(blockIdx.y) - rotated_groups;
    const T* row = packed + (token * packed_heads + rotated_heads + kv_head) * head_dim;
    if (live) {      // 16 bytes as they are
      const uint4 lo = *reinterpret_cast<const uint4*>(row + 8 * part);
      const uint4 hi = *reinterpret_cast<const uint4*>(row + half + 8 * part);
      *reinterpret_cast<uint4*>(tile_s + item * head_dim + 8 * part) = lo;
      *reinterpret_cast<uint4*>(tile_s + item * head_dim + half + 8 * part) = hi;
    }
    if (threadIdx.x < live_tokens) slot_s[threadIdx.x] = slot_mapping[first_token + threadIdx.x];
    __syncthreads();
    // A group of kGroup consecutive tokens whose slots are consecutive and begin a
    // 16-byte group of a page's row is written with one store for every d (a prompt's
    // tokens are, but for the first and the last group of a portion); the tokens of any
    // other group go one by one.
    const int groups = (live_tokens + kGroup - 1) / kGroup;
    if (threadIdx.x < groups) {
      const int j0 = threadIdx.x * kGroup;
      bool whole = block_size % kGroup == 0 && j0 + kGroup <= live_tokens && slot_s[j0] % kGroup == 0;
      for (int i = 1; whole && i < kGroup; ++i) whole = slot_s[j0 + i] == slot_s[j0] + i;
      whole_s[threadIdx.x] = whole;
    }
    __syncthreads();
    for (int task = threadIdx.x; task < groups * head_dim; task += kTiledThreads) {
      const int group = task / head_dim;
      const int d = task - group * head_dim;
      const int j0 = group * kGroup;
      if (whole_s[group]) {
        const int32_t slot = slot_s[j0];
        const int page = slot / block_size;
        const int offset = slot - page * block_size;
        __align__(16) T gathered[kGroup];
#pragma unroll
        for (int i = 0; i < kGroup; ++i) gathered[i] = tile_s[(j0 + i) * head_dim + d];
        T* dst = value_pool + ((static_cast<int64_t>(page) * num_kv_heads + kv_head) * head_dim + d) * block_size + offset;
        *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(gathered);
      } else {
        for (int i = 0; i < kGroup && j0 + i < live_tokens; ++i) {
          const int32_t slot = slot_s[j0 + i];
          const int page = slot / block_size;
          const int offset = slot - page * block_size;
          value_pool[((static_cast<int64_t>(page) * num_kv_heads + kv_head) * head_dim + d) * block_size + offset] =
              tile_s[(j0 + i) * head_dim + d];
        }
      }
    }
    return;
  }

  // query and key heads first_head .. first_head + heads_here - 1: all their loads go
  // out together, with the tile's cos and sin
  const int first_head = static_cast<int>(blockIdx.y) * kTiledHeads;
  const int heads_here = min(kTiledHeads, rotated_heads - first_head);
  // No branch that differs between lanes stands around a load (a dead lane reads the
  // tile's first token, a missing head the last one, and stores nothing): a value that is
  // used behind such a branch is waited for behind it, head after head, and the kernel
  // would take as many trips to memory as it has heads.  The values are turned into
  // floats when all loads are on their way.
  static_assert(sizeof(T) == 2, "16 bytes are 8 elements");
  uint4 raw_lo[kTiledHeads], raw_hi[kTiledHeads];
#pragma unroll
  for (int i = 0; i < kTiledHeads; ++i) {
    const T* row = packed + (token * packed_heads + first_head + min(i, heads_here - 1)) * head_dim;
    raw_lo[i] = *reinterpret_cast<const uint4*>(row + 8 * part);
    raw_hi[i] = *reinterpret_cast<const uint4*>(row + half + 8 * part);
  }
  float cs[8], sn[8];
  if (cos_table != nullptr) {
    load8(cos_table + token * half + 8 * part, cs);
    load8(sin_table + token * half + 8 * part, sn);
  }
  int slot = 0;      // a slot number is below 2^31
  if (first_head + heads_here > num_q_heads) slot = slot_mapping[token];
  // the norms' weights go out with the rows: asked for where they are used, behind the
  // barrier, each head would wait for memory once more
  uint4 raw_wq[2], raw_wk[2];
  const bool has_q = q_weight != nullptr && first_head < num_q_heads;
  const bool has_k = k_weight != nullptr && first_head + heads_here > num_q_heads;
  if (has_q) {
    raw_wq[0] = *reinterpret_cast<const uint4*>(q_weight + 8 * part);
    raw_wq[1] = *reinterpret_cast<const uint4*>(q_weight + half + 8 * part);
  }
  if (has_k) {
    raw_wk[0] = *reinterpret_cast<const uint4*>(k_weight + 8 * part);
    raw_wk[1] = *reinterpret_cast<const uint4*>(k_weight + half + 8 * part);
  }
  float lo[kTiledHeads][8], hi[kTiledHeads][8];
#pragma unroll
  for (int i = 0; i < kTiledHeads; ++i) {
    unpack8(raw_lo[i], lo[i]);
    unpack8(raw_hi[i], hi[i]);
  }

  if (q_weight != nullptr || k_weight != nullptr) {
#pragma unroll
    for (int i = 0; i < kTiledHeads; ++i) {
      float partial = 0.f;
      if (live && i < heads_here) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          partial = fmaf(lo[i][e], lo[i][e], partial);
          partial = fmaf(hi[i][e], hi[i][e], partial);
        }
      }
      square_s[i][threadIdx.x] = partial;
    }
    __syncthreads();
  }
  if (!live) return;

#pragma unroll
  for (int i = 0; i < kTiledHeads; ++i) {
    if (i >= heads_here) break;
    const int head = first_head + i;
    const bool is_q = head < num_q_heads;
    const T* weight = is_q ? q_weight : k_weight;
    if (weight) {
      float total = 0.f;
      for (int p = 0; p < lanes_per_row; ++p) total += square_s[i][item * lanes_per_row + p];
      const float inv = 1.0f / sqrtf(total / static_cast<float>(head_dim) + eps);
      float w_lo[8], w_hi[8];
      unpack8(is_q ? raw_wq[0] : raw_wk[0], w_lo);
      unpack8(is_q ? raw_wq[1] : raw_wk[1], w_hi);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        lo[i][e] = ms::round_to<T>(w_lo[e] * ms::round_to<T>(lo[i][e] * inv));
        hi[i][e] = ms::round_to<T>(w_hi[e] * ms::round_to<T>(hi[i][e] * inv));
      }
    }
    if (cos_table != nullptr) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float a = lo[i][e], b = hi[i][e];
        lo[i][e] = a * cs[e] - b * sn[e];
        hi[i][e] = b * cs[e] + a * sn[e];
      }
    }
    T* dst;
    if (is_q) {
      dst = q_out + (token * num_q_heads + head) * head_dim;
    } else {
      const int kv_head = head - num_q_heads;
      const int page = slot / block_size;
      const int offset = slot - page * block_size;
      dst = key_pool + ((static_cast<int64_t>(page) * num_kv_heads + kv_head) * block_size + offset) * head_dim;
    }
    store8(dst + 8 * part, lo[i]);
    store8(dst + half + 8 * part, hi[i]);
  }
}

template <typename T>
void launch_tiled(const void* packed, const void* q_weight, const void* k_weight, const void* cos_table,
                  const void* sin_table, const void* slot_mapping, void* q_out, void* key_pool, void* value_pool,
                  int num_tokens, int num_q_heads, int num_kv_heads, int head_dim, int block_size, float eps,
                  hipStream_t stream) {
  const int tile_tokens = kTiledThreads / (head_dim / 16);
  const int rotated_groups = (num_q_heads + num_kv_heads + kTiledHeads - 1) / kTiledHeads;
  const dim3 grid((num_tokens + tile_tokens - 1) / tile_tokens, rotated_groups + num_kv_heads);
  hipLaunchKernelGGL((qk_norm_rope_append_tiled_kernel<T>), grid, dim3(kTiledThreads), 0, stream,
      static_cast<const T*>(packed), static_cast<const T*>(q_weight), static_cast<const T*>(k_weight),
      static_cast<const float*>(cos_table), static_cast<const float*>(sin_table),
      static_cast<const int32_t*>(slot_mapping), static_cast<T*>(q_out), static_cast<T*>(key_pool),
      static_cast<T*>(value_pool), num_tokens, num_q_heads, num_kv_heads, head_dim, block_size, eps);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

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
  // bfloat16, 16 bytes a lane, where the head size is a multiple of 16 and every operand
  // is aligned to 16 bytes (null operands are), for more tokens than four tiles; few
  // tokens are quicker with a wave to each row.  32-bit storage always takes the wave
  // to each row: the order of its sums never depends on the number of tokens, so a
  // position's result is the same to the bit however the tokens are cut into steps.
  const bool tiled = dtype == MS_BF16 && head_dim % 16 == 0 && head_dim <= 16 * kTiledThreads &&
                     num_tokens > 4 * (kTiledThreads / (head_dim / 16)) && aligned16(packed) &&
                     aligned16(q_weight) && aligned16(k_weight) && aligned16(cos_table) && aligned16(sin_table) &&
                     aligned16(q_out) && aligned16(key_pool) && aligned16(value_pool);
  if (tiled) {
    launch_tiled<ms::bf16>(packed, q_weight, k_weight, cos_table, sin_table, slot_mapping, q_out, key_pool,
                           value_pool, num_tokens, num_q_heads, num_kv_heads, head_dim, block_size, eps, stream);
    MS_CHECK_LAUNCH("qk_norm_rope_append");
    return 0;
  }
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
