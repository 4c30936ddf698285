// Paged attention for rows that each bring ONE query token (decoding), bfloat16
// storage, matrix cores, split over the keys.
//
// Work is cut as (split of the keys, kv head x group of 16 query heads, token).
// All query heads that share a kv head are the 16 columns of one MFMA tile, so
// every key and value is read once for all of them.  A workgroup of 4 waves walks
// its share of the keys in tiles of 16 keys, two tiles (32 keys) per MFMA; each
// wave keeps an online softmax (running max m, sum l) in 32-bit and an
// unnormalised output tile in 32-bit; the waves are merged through LDS; a split
// writes its (m, l, O) and a second kernel merges the splits.  (Merging in the
// split that finishes last would need a device-wide fence per workgroup, which
// on this chip writes back the whole L2 of its die: measured 3x slower.)
//
//   S^T[key, head] = K[key, :] . Q[head, :]      A = K tile (16 keys x 32 d), B = Q^T
//   P = exp(S * scale - m)                        (scale after the product, as the
//                                                  reference does: qwen3.py:243)
//   O[head, d]   += P[head, keys] . V[keys, d]    A = P (the S^T accumulator, as it
//                                                  lies in the registers), B = V
// The cache layout serves the operands directly: keys as [page, kv_head, offset, d]
// (8 consecutive d per lane, 16 bytes), values as [page, kv_head, d, offset]
// (4 consecutive keys per lane, 8 bytes).
//
// Formula of the one-token form: reference csrc/paged_decode_attention.cu:44-94.
// Unlike there, no shared memory grows with the context.
#include "attention_tiles.hpp"

namespace {

using ms::bf16;
using ms::bf16x4;
using ms::bf16x8;
using ms::floatx4;

using ms::kTileKeys;
using ms::load_pair;
using ms::TilePair;

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * ms::kWave;

// Online-softmax state of one wave: head r's running max and sum (the same in all
// four lane groups) and the unnormalised output tile.
template <int D>
struct WaveState {
  floatx4 o[D / 16];
  float run_max, run_sum;
};

template <int D>
__device__ __forceinline__ void consume_pair(WaveState<D>& st, TilePair<D>& pair, const bf16x8* q_reg, int tile,
                                             int lo, int pos, float scale, int g) {
  constexpr int KS = TilePair<D>::KS, CS = TilePair<D>::CS;
  const int key_a = tile * kTileKeys, key_b = key_a + kTileKeys;
  // ---- S^T = K . Q^T ---------------------------------------------------------
  floatx4 s_a = {0.f, 0.f, 0.f, 0.f}, s_b = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    s_a = ms::mfma_16x16x32(pair.k_a[s], q_reg[s], s_a);
    s_b = ms::mfma_16x16x32(pair.k_b[s], q_reg[s], s_b);
  }
  // this lane: head r, keys key_a + 4 g + e and key_b + 4 g + e
  bool ok_a[4], ok_b[4];
  float tile_max = -INFINITY;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int ka = key_a + 4 * g + e, kb = key_b + 4 * g + e;
    ok_a[e] = ka >= lo && ka <= pos;
    ok_b[e] = pair.has_b && kb >= lo && kb <= pos;
    s_a[e] = ok_a[e] ? s_a[e] * scale : -INFINITY;
    s_b[e] = ok_b[e] ? s_b[e] * scale : -INFINITY;
    tile_max = fmaxf(tile_max, fmaxf(s_a[e], s_b[e]));
  }
  tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, ms::kWave));
  tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, ms::kWave));
  const float new_max = fmaxf(st.run_max, tile_max);   // finite: every tile of the range holds a visible key
  const float alpha = __expf(st.run_max - new_max);
  float tile_sum = 0.f;
  bf16x8 p;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float pa = __expf(s_a[e] - new_max);
    const float pb = __expf(s_b[e] - new_max);
    tile_sum += pa + pb;
    p[e] = static_cast<__bf16>(pa);
    p[e + 4] = static_cast<__bf16>(pb);
  }
  tile_sum += __shfl_xor(tile_sum, 16, ms::kWave);
  tile_sum += __shfl_xor(tile_sum, 32, ms::kWave);
  st.run_sum = st.run_sum * alpha + tile_sum;
  st.run_max = new_max;

  // ---- O = alpha O + P . V ---------------------------------------------------
  // O's rows in this lane are the heads 4 g + e; their alpha lives in lane 4 g + e.
  float alpha_row[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) alpha_row[e] = __shfl(alpha, 4 * g + e, ms::kWave);
  const bool partial = !(ok_a[0] && ok_a[3] && ok_b[0] && ok_b[3]);
#pragma unroll
  for (int c = 0; c < CS; ++c) {
    bf16x4 va = pair.v_a[c], vb = pair.v_b[c];
    if (partial) {   // a stale value times a zero weight must not become NaN
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (!ok_a[e]) va[e] = static_cast<__bf16>(0.0f);
        if (!ok_b[e]) vb[e] = static_cast<__bf16>(0.0f);
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) st.o[c][e] *= alpha_row[e];
    st.o[c] = ms::mfma_16x16x32(p, ms::concat(va, vb), st.o[c]);
  }
}

template <int D>
__global__ __launch_bounds__(kThreads) MS_WAVES_PER_EU(D <= 128 ? 2 : 1, 2) void attention_decode_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ key_pool, const bf16* __restrict__ value_pool,
    const int32_t* __restrict__ block_table, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, bf16* __restrict__ out, float* __restrict__ partial_o,
    float* __restrict__ partial_ml, int num_q_heads, int num_kv_heads, int block_size, int max_blocks, float scale,
    int window, int num_splits) {
  constexpr int KS = TilePair<D>::KS, CS = TilePair<D>::CS;

  __shared__ float o_s[kWaves - 1][16][D];
  __shared__ float m_s[kWaves][16];
  __shared__ float l_s[kWaves][16];

  const int lane = threadIdx.x & 63;
  const int wave = ms::uniform(threadIdx.x >> 6);   // the same in all lanes: tile numbers and table entries are scalar work
  const int g = lane >> 4;
  const int r = lane & 15;

  const int split = blockIdx.x;
  const int group = num_q_heads / num_kv_heads;
  const int head_groups = (group + 15) / 16;
  const int kv_head = blockIdx.y / head_groups;
  const int head_group = blockIdx.y - kv_head * head_groups;
  const int64_t token = blockIdx.z;
  const int head0 = kv_head * group + head_group * 16;
  const int heads_here = min(16, group - head_group * 16);

  const int pos = positions[token];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* table = block_table + static_cast<int64_t>(seq_of_token[token]) * max_blocks;

  const int first_tile = lo / kTileKeys;
  const int last_tile = pos / kTileKeys;
  const int tiles_per_split = (last_tile - first_tile + num_splits) / num_splits;
  const int t0 = first_tile + split * tiles_per_split;
  const int t1 = min(t0 + tiles_per_split, last_tile + 1);

  // Q^T operand: column r = head, k-slots d = 32 s + 8 g + 0..7
  bf16x8 q_reg[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int d0 = 32 * s + 8 * g;
    q_reg[s] = (r < heads_here && d0 < D) ? ms::load_bf16x8(q + (token * num_q_heads + head0 + r) * D + d0)
                                          : ms::zero_bf16x8();
  }

  WaveState<D> st;
#pragma unroll
  for (int c = 0; c < CS; ++c) st.o[c] = floatx4{0.f, 0.f, 0.f, 0.f};
  st.run_max = -INFINITY;
  st.run_sum = 0.f;

  // The wave's pairs of tiles, the loads of the next pair in flight while the
  // current one is consumed.
  constexpr int kStep = 2 * kWaves;
  constexpr bool kPrefetch = D <= 128;      // larger heads would spill registers
  int t = t0 + 2 * wave;
  if (!kPrefetch) {
    for (; t < t1; t += kStep) {
      TilePair<D> pair;
      load_pair<D>(pair, ms::find_pair(t, t1, table, block_size), key_pool, value_pool, num_kv_heads, kv_head,
                   block_size, g, r);
      consume_pair<D>(st, pair, q_reg, t, lo, pos, scale, g);
    }
  } else if (t < t1) {
    // the pages of a pair are looked up while the pair before it is on its way
    TilePair<D> ping, pong;
    load_pair<D>(ping, ms::find_pair(t, t1, table, block_size), key_pool, value_pool, num_kv_heads, kv_head, block_size,
                 g, r);
    ms::PairPlace ahead = ms::find_pair(t + kStep, t1, table, block_size);
    while (true) {
      int next = t + kStep;
      if (next < t1) {
        load_pair<D>(pong, ahead, key_pool, value_pool, num_kv_heads, kv_head, block_size, g, r);
        ahead = ms::find_pair(next + kStep, t1, table, block_size);
      }
      consume_pair<D>(st, ping, q_reg, t, lo, pos, scale, g);
      t = next;
      if (t >= t1) break;
      next = t + kStep;
      if (next < t1) {
        load_pair<D>(ping, ahead, key_pool, value_pool, num_kv_heads, kv_head, block_size, g, r);
        ahead = ms::find_pair(next + kStep, t1, table, block_size);
      }
      consume_pair<D>(st, pong, q_reg, t, lo, pos, scale, g);
      t = next;
      if (t >= t1) break;
    }
  }

  // ---- merge the waves through LDS, into wave 0 -------------------------------
  if (g == 0) {
    m_s[wave][r] = st.run_max;
    l_s[wave][r] = st.run_sum;
  }
  if (wave > 0) {
#pragma unroll
    for (int c = 0; c < CS; ++c)
#pragma unroll
      for (int e = 0; e < 4; ++e) o_s[wave - 1][4 * g + e][16 * c + r] = st.o[c][e];
  }
  __syncthreads();

  if (wave != 0) return;

  float total_max[4], total_sum[4], factor[kWaves][4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int row = 4 * g + e;
    float mx = m_s[0][row];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mx = fmaxf(mx, m_s[w][row]);
    total_max[e] = mx;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      factor[w][e] = (mx == -INFINITY) ? 0.f : __expf(m_s[w][row] - mx);
      sum += factor[w][e] * l_s[w][row];
    }
    total_sum[e] = sum;
  }
#pragma unroll
  for (int c = 0; c < CS; ++c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float acc = st.o[c][e] * factor[0][e];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) acc += o_s[w - 1][4 * g + e][16 * c + r] * factor[w][e];
      st.o[c][e] = acc;
    }
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int row = 4 * g + e;
    if (row >= heads_here) continue;
    const int64_t head = head0 + row;
    if (num_splits == 1) {
      const float inv = 1.0f / total_sum[e];
      bf16* dst = out + (token * num_q_heads + head) * D;
#pragma unroll
      for (int c = 0; c < CS; ++c) dst[16 * c + r] = ms::from_float<bf16>(st.o[c][e] * inv);
    } else {
      const int64_t slot = (token * num_q_heads + head) * num_splits + split;
      float* dst = partial_o + slot * D;
#pragma unroll
      for (int c = 0; c < CS; ++c) dst[16 * c + r] = st.o[c][e];
      if (r == 0) {
        partial_ml[2 * slot] = total_max[e];
        partial_ml[2 * slot + 1] = total_sum[e];
      }
    }
  }
}

// Merge of the splits, one workgroup per (token, head):
//   out = sum_s e^{m_s - M} O_s / sum_s e^{m_s - M} l_s,  M = max_s m_s.
// The first wave turns the (m_s, l_s) into weights, then every thread owns one
// column of the head.  At most 64 splits.
__global__ void attention_merge_splits_kernel(const float* __restrict__ partial_o,
                                              const float* __restrict__ partial_ml, bf16* __restrict__ out,
                                              int head_dim, int num_splits) {
  __shared__ float weight_s[ms::kWave];
  const int64_t row = blockIdx.x;
  // the first partial outputs of this thread's column are on their way while the first
  // wave makes the weights
  constexpr int kAhead = 16;
  const int d0 = threadIdx.x;
  float ahead[kAhead];
  if (d0 < head_dim) {
    const float* column = partial_o + row * num_splits * head_dim + d0;
#pragma unroll
    for (int s = 0; s < kAhead; ++s) ahead[s] = s < num_splits ? column[static_cast<int64_t>(s) * head_dim] : 0.f;
  }
  if (threadIdx.x < ms::kWave) {
    const int s = threadIdx.x;
    const bool live = s < num_splits;
    const float m = live ? partial_ml[2 * (row * num_splits + s)] : -INFINITY;
    const float l = live ? partial_ml[2 * (row * num_splits + s) + 1] : 0.f;
    const float mx = ms::wave_max(m);
    const float f = live ? __expf(m - mx) : 0.f;
    const float total = ms::wave_sum(f * l);
    weight_s[s] = f / total;
  }
  __syncthreads();
  for (int d = d0; d < head_dim; d += blockDim.x) {
    const float* column = partial_o + row * num_splits * head_dim + d;
    float acc = 0.f;
    if (d == d0) {
#pragma unroll
      for (int s = 0; s < kAhead; ++s) acc = fmaf(s < num_splits ? weight_s[s] : 0.f, ahead[s], acc);
      for (int s = kAhead; s < num_splits; ++s) acc = fmaf(weight_s[s], column[static_cast<int64_t>(s) * head_dim], acc);
    } else {
#pragma unroll 8
      for (int s = 0; s < num_splits; ++s) acc = fmaf(weight_s[s], column[static_cast<int64_t>(s) * head_dim], acc);
    }
    out[row * head_dim + d] = ms::from_float<bf16>(acc);
  }
}

template <int D>
void launch_decode(const void* q, const void* key_pool, const void* value_pool, const void* block_table,
                   const void* seq_of_token, const void* positions, void* out, void* partial_o, void* partial_ml,
                   int num_tokens, int num_q_heads, int num_kv_heads, int block_size, int max_blocks, float scale,
                   int window, int num_splits, hipStream_t stream) {
  const int head_groups = (num_q_heads / num_kv_heads + 15) / 16;
  const dim3 grid(num_splits, num_kv_heads * head_groups, num_tokens);
  hipLaunchKernelGGL((attention_decode_kernel<D>), grid, dim3(kThreads), 0, stream, static_cast<const bf16*>(q),
                     static_cast<const bf16*>(key_pool), static_cast<const bf16*>(value_pool),
                     static_cast<const int32_t*>(block_table), static_cast<const int32_t*>(seq_of_token),
                     static_cast<const int32_t*>(positions), static_cast<bf16*>(out), static_cast<float*>(partial_o),
                     static_cast<float*>(partial_ml), num_q_heads, num_kv_heads, block_size, max_blocks, scale,
                     window, num_splits);
}

}  // namespace

// Whether ms_attention_decode takes this geometry (else the caller uses the
// generic kernel): head size a multiple of 16 up to 256, pages of a multiple of
// 16 keys.
extern "C" int ms_attention_decode_supported(int head_dim, int block_size) {
  return head_dim >= 16 && head_dim <= 256 && head_dim % 16 == 0 && block_size % kTileKeys == 0;
}

// q, out: bfloat16 [num_tokens, num_q_heads, head_dim]; key_pool: [pages, kv_heads,
// block_size, head_dim]; value_pool: [pages, kv_heads, head_dim, block_size];
// partial_o: float [num_tokens, num_q_heads, num_splits, head_dim] and partial_ml:
// float [num_tokens, num_q_heads, num_splits, 2], both unused when num_splits == 1
// (at most 64 splits).
extern "C" int ms_attention_decode(const void* q, const void* key_pool, const void* value_pool,
                                   const void* block_table, const void* seq_of_token, const void* positions,
                                   void* out, void* partial_o, void* partial_ml, int num_tokens, int num_q_heads,
                                   int num_kv_heads, int head_dim, int block_size, int max_blocks, float scale,
                                   int window, int num_splits, hipStream_t stream) {
  MS_REQUIRE(num_tokens > 0 && num_tokens <= 65535, "attention_decode: %d tokens are outside 1..65535", num_tokens);
  MS_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0,
             "attention_decode: %d query heads are not a multiple of %d kv heads", num_q_heads, num_kv_heads);
  MS_REQUIRE(ms_attention_decode_supported(head_dim, block_size),
             "attention_decode: head_dim %d (multiples of 16 up to 256) or block_size %d (multiples of 16) "
             "is not supported",
             head_dim, block_size);
  MS_REQUIRE(num_splits >= 1 && num_splits <= ms::kWave, "attention_decode: %d splits are outside 1..64", num_splits);
  MS_REQUIRE(num_splits == 1 || (partial_o && partial_ml), "attention_decode: splits need partial buffers");
  MS_REQUIRE(max_blocks > 0 && window >= 0, "attention_decode: bad table width or window");
  MS_REQUIRE(num_kv_heads * ((num_q_heads / num_kv_heads + 15) / 16) <= 65535, "attention_decode: too many heads");
#define MS_DECODE_CASE(DIM)                                                                                     \
  case DIM:                                                                                                     \
    launch_decode<DIM>(q, key_pool, value_pool, block_table, seq_of_token, positions, out, partial_o, partial_ml, \
                       num_tokens, num_q_heads, num_kv_heads, block_size, max_blocks, scale, window, num_splits,  \
                       stream);                                                                                 \
    break;
  switch (head_dim) {
    MS_DECODE_CASE(16) MS_DECODE_CASE(32) MS_DECODE_CASE(48) MS_DECODE_CASE(64) MS_DECODE_CASE(80)
    MS_DECODE_CASE(96) MS_DECODE_CASE(112) MS_DECODE_CASE(128) MS_DECODE_CASE(144) MS_DECODE_CASE(160)
    MS_DECODE_CASE(176) MS_DECODE_CASE(192) MS_DECODE_CASE(208) MS_DECODE_CASE(224) MS_DECODE_CASE(240)
    MS_DECODE_CASE(256)
    default:
      return ms_fail("attention_decode: head_dim %d", head_dim);
  }
#undef MS_DECODE_CASE
  MS_CHECK_LAUNCH("attention_decode");
  if (num_splits > 1) {
    const int threads = head_dim <= 64 ? 64 : (head_dim <= 128 ? 128 : 256);
    hipLaunchKernelGGL(attention_merge_splits_kernel, dim3(num_tokens * num_q_heads), dim3(threads), 0, stream,
                       static_cast<const float*>(partial_o), static_cast<const float*>(partial_ml),
                       static_cast<bf16*>(out), head_dim, num_splits);
    MS_CHECK_LAUNCH("attention_merge_splits");
  }
  return 0;
}
