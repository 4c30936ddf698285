// Paged causal attention for rows that bring runs of query tokens (prompts and
// their portions), bfloat16 storage, matrix cores.
//
// One wave owns a tile of 16 consecutive query tokens of one sequence and HB query
// heads that share a kv head: 16 * HB columns.  It walks the keys 0 .. (its last
// token's position) in tiles of 16, two tiles per MFMA, with the loads of the next
// pair in flight while the current one is consumed, and keeps for every column an
// online softmax in 32-bit:
//
//   S^T[key, query] = K[key, :] . Q[query, :]     A = K tile, B = Q^T (16 queries of one head)
//   P = exp(S * scale - m), masked to lo <= key <= position of the query
//   O[query, d]    += P[query, keys] . V[keys, d]
//
// Every key and value tile read serves all 16 * HB columns.  The mask is by
// absolute position, so a portion of a prompt sees the history in the cache and
// itself (reference: miniserve/model/qwen3.py:237-249, where the scores of a chunk
// are a dense product over the gathered history).
#include "attention_tiles.hpp"

namespace {

using ms::bf16;
using ms::bf16x4;
using ms::bf16x8;
using ms::floatx4;
using ms::kTileKeys;
using ms::load_pair;
using ms::TilePair;

constexpr int kQueryTile = 16;

template <int D, int HB>
struct PrefillState {
  floatx4 o[HB][D / 16];
  float run_max[HB], run_sum[HB];   // of query column r (the same in all four lane groups)
};

template <int D, int HB>
__device__ __forceinline__ void consume_pair(PrefillState<D, HB>& st, TilePair<D>& pair,
                                             const bf16x8 (&q_reg)[HB][TilePair<D>::KS], int tile, int lo, int pos,
                                             int last_key, float scale, int g) {
  constexpr int KS = TilePair<D>::KS, CS = TilePair<D>::CS;
  const int key_a = tile * kTileKeys, key_b = key_a + kTileKeys;
  // this lane: query column r (position pos, window start lo), keys key_a + 4 g + e and key_b + 4 g + e
  bool ok_a[4], ok_b[4], stale_a[4], stale_b[4];
  bool any_stale = false;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int ka = key_a + 4 * g + e, kb = key_b + 4 * g + e;
    ok_a[e] = ka >= lo && ka <= pos;
    ok_b[e] = pair.has_b && kb >= lo && kb <= pos;
    stale_a[e] = ka > last_key;                     // beyond what the sequence has written
    stale_b[e] = kb > last_key;
    any_stale = any_stale || stale_a[e] || stale_b[e];
  }
  float alpha[HB];
  bf16x8 p[HB];
#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
    floatx4 s_a = {0.f, 0.f, 0.f, 0.f}, s_b = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      s_a = ms::mfma_16x16x32(pair.k_a[s], q_reg[hb][s], s_a);
      s_b = ms::mfma_16x16x32(pair.k_b[s], q_reg[hb][s], s_b);
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s_a[e] = ok_a[e] ? s_a[e] * scale : -INFINITY;
      s_b[e] = ok_b[e] ? s_b[e] * scale : -INFINITY;
      tile_max = fmaxf(tile_max, fmaxf(s_a[e], s_b[e]));
    }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, ms::kWave));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, ms::kWave));
    const float new_max = fmaxf(st.run_max[hb], tile_max);
    // a column may see no key of this pair (and none before): keep everything at zero
    const float safe_max = new_max == -INFINITY ? 0.f : new_max;
    alpha[hb] = __expf(st.run_max[hb] - safe_max);
    float tile_sum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float pa = __expf(s_a[e] - safe_max);
      const float pb = __expf(s_b[e] - safe_max);
      tile_sum += pa + pb;
      p[hb][e] = static_cast<__bf16>(pa);
      p[hb][e + 4] = static_cast<__bf16>(pb);
    }
    tile_sum += __shfl_xor(tile_sum, 16, ms::kWave);
    tile_sum += __shfl_xor(tile_sum, 32, ms::kWave);
    st.run_sum[hb] = st.run_sum[hb] * alpha[hb] + tile_sum;
    st.run_max[hb] = new_max;
  }

  // O's rows in this lane are the queries 4 g + e; their alpha lives in lane 4 g + e.
  float alpha_row[HB][4];
#pragma unroll
  for (int hb = 0; hb < HB; ++hb)
#pragma unroll
    for (int e = 0; e < 4; ++e) alpha_row[hb][e] = __shfl(alpha[hb], 4 * g + e, ms::kWave);
#pragma unroll
  for (int c = 0; c < CS; ++c) {
    bf16x4 va = pair.v_a[c], vb = pair.v_b[c];
    if (any_stale) {   // a stale value times a zero weight must not become NaN
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (stale_a[e]) va[e] = static_cast<__bf16>(0.0f);
        if (stale_b[e]) vb[e] = static_cast<__bf16>(0.0f);
      }
    }
    const bf16x8 v = ms::concat(va, vb);
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
#pragma unroll
      for (int e = 0; e < 4; ++e) st.o[hb][c][e] *= alpha_row[hb][e];
      st.o[hb][c] = ms::mfma_16x16x32(p[hb], v, st.o[hb][c]);
    }
  }
}

template <int D, int HB>
__global__ __launch_bounds__(ms::kWave) void attention_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ key_pool, const bf16* __restrict__ value_pool,
    const int32_t* __restrict__ block_table, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_token, const int32_t* __restrict__ tile_count,
    bf16* __restrict__ out, int num_q_heads, int num_kv_heads, int block_size, int max_blocks, float scale,
    int window) {
  constexpr int KS = TilePair<D>::KS, CS = TilePair<D>::CS;
  const int lane = threadIdx.x;
  const int g = lane >> 4;
  const int r = lane & 15;

  const int tile_index = blockIdx.x;
  const int group = num_q_heads / num_kv_heads;
  const int head_blocks = (group + HB - 1) / HB;
  const int kv_head = blockIdx.y / head_blocks;
  const int head0 = kv_head * group + (blockIdx.y - kv_head * head_blocks) * HB;
  const int heads_here = min(HB, kv_head * group + group - head0);

  const int token0 = tile_token[tile_index];
  const int count = tile_count[tile_index];           // 1..16 tokens of one sequence, consecutive positions
  const int32_t* table = block_table + static_cast<int64_t>(tile_seq[tile_index]) * max_blocks;

  // query column r of this lane; a column past the tile's tokens repeats the last one and is not stored
  const int64_t my_token = token0 + min(r, count - 1);
  const int pos = positions[my_token];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int first_pos = positions[token0];
  const int last_key = first_pos + count - 1;         // the tile's last position: all keys up to it are written
  const int first_lo = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  const int t0 = first_lo / kTileKeys;
  const int t1 = last_key / kTileKeys + 1;

  bf16x8 q_reg[HB][KS];
#pragma unroll
  for (int hb = 0; hb < HB; ++hb)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int d0 = 32 * s + 8 * g;
      q_reg[hb][s] = (hb < heads_here && d0 < D) ? ms::load_bf16x8(q + (my_token * num_q_heads + head0 + hb) * D + d0)
                                                  : ms::zero_bf16x8();
    }

  PrefillState<D, HB> st;
#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
#pragma unroll
    for (int c = 0; c < CS; ++c) st.o[hb][c] = floatx4{0.f, 0.f, 0.f, 0.f};
    st.run_max[hb] = -INFINITY;
    st.run_sum[hb] = 0.f;
  }

  int t = t0;
  TilePair<D> ping, pong;
  load_pair<D>(ping, t, t1, table, key_pool, value_pool, num_kv_heads, kv_head, block_size, g, r);
  while (true) {
    int next = t + 2;
    if (next < t1) load_pair<D>(pong, next, t1, table, key_pool, value_pool, num_kv_heads, kv_head, block_size, g, r);
    consume_pair<D, HB>(st, ping, q_reg, t, lo, pos, last_key, scale, g);
    t = next;
    if (t >= t1) break;
    next = t + 2;
    if (next < t1) load_pair<D>(ping, next, t1, table, key_pool, value_pool, num_kv_heads, kv_head, block_size, g, r);
    consume_pair<D, HB>(st, pong, q_reg, t, lo, pos, last_key, scale, g);
    t = next;
    if (t >= t1) break;
  }

  // this lane: output rows = queries 4 g + e, column d = 16 c + r; the row's sum lives in lane 4 g + e
#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
    float inv_row[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) inv_row[e] = 1.0f / __shfl(st.run_sum[hb], 4 * g + e, ms::kWave);
    if (hb >= heads_here) continue;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int row = 4 * g + e;
      if (row >= count) continue;
      bf16* dst = out + ((static_cast<int64_t>(token0) + row) * num_q_heads + head0 + hb) * D;
#pragma unroll
      for (int c = 0; c < CS; ++c) dst[16 * c + r] = ms::from_float<bf16>(st.o[hb][c][e] * inv_row[e]);
    }
  }
}

template <int D, int HB>
void launch_prefill(const void* q, const void* key_pool, const void* value_pool, const void* block_table,
                    const void* positions, const void* tile_seq, const void* tile_token, const void* tile_count,
                    void* out, int num_tiles, int num_q_heads, int num_kv_heads, int block_size, int max_blocks,
                    float scale, int window, hipStream_t stream) {
  const int head_blocks = (num_q_heads / num_kv_heads + HB - 1) / HB;
  const dim3 grid(num_tiles, num_kv_heads * head_blocks);
  hipLaunchKernelGGL((attention_prefill_kernel<D, HB>), grid, dim3(ms::kWave), 0, stream, static_cast<const bf16*>(q),
                     static_cast<const bf16*>(key_pool), static_cast<const bf16*>(value_pool),
                     static_cast<const int32_t*>(block_table), static_cast<const int32_t*>(positions),
                     static_cast<const int32_t*>(tile_seq), static_cast<const int32_t*>(tile_token),
                     static_cast<const int32_t*>(tile_count), static_cast<bf16*>(out), num_q_heads, num_kv_heads,
                     block_size, max_blocks, scale, window);
}

template <int D>
void launch_prefill_heads(int hb, const void* q, const void* key_pool, const void* value_pool,
                          const void* block_table, const void* positions, const void* tile_seq,
                          const void* tile_token, const void* tile_count, void* out, int num_tiles, int num_q_heads,
                          int num_kv_heads, int block_size, int max_blocks, float scale, int window,
                          hipStream_t stream) {
  if (hb == 1) {
    launch_prefill<D, 1>(q, key_pool, value_pool, block_table, positions, tile_seq, tile_token, tile_count, out,
                         num_tiles, num_q_heads, num_kv_heads, block_size, max_blocks, scale, window, stream);
  } else if (hb == 2) {
    launch_prefill<D, 2>(q, key_pool, value_pool, block_table, positions, tile_seq, tile_token, tile_count, out,
                         num_tiles, num_q_heads, num_kv_heads, block_size, max_blocks, scale, window, stream);
  } else {
    launch_prefill<D, 4>(q, key_pool, value_pool, block_table, positions, tile_seq, tile_token, tile_count, out,
                         num_tiles, num_q_heads, num_kv_heads, block_size, max_blocks, scale, window, stream);
  }
}

}  // namespace

// Whether ms_attention_prefill takes this geometry: head size a multiple of 16 up to
// 128, pages of a multiple of 16 keys.
extern "C" int ms_attention_prefill_supported(int head_dim, int block_size) {
  return head_dim >= 16 && head_dim <= 128 && head_dim % 16 == 0 && block_size % kTileKeys == 0;
}

// q, out: bfloat16 [num_tokens, num_q_heads, head_dim]; key_pool: [pages, kv_heads,
// block_size, head_dim]; value_pool: [pages, kv_heads, head_dim, block_size];
// positions: int32 [num_tokens].  The query tokens are cut into num_tiles tiles of
// at most 16 consecutive tokens of one sequence: tile_seq (row of block_table),
// tile_token (index of its first token), tile_count (1..16), all int32 [num_tiles].
extern "C" int ms_attention_prefill(const void* q, const void* key_pool, const void* value_pool,
                                    const void* block_table, const void* positions, const void* tile_seq,
                                    const void* tile_token, const void* tile_count, void* out, int num_tiles,
                                    int num_q_heads, int num_kv_heads, int head_dim, int block_size, int max_blocks,
                                    float scale, int window, hipStream_t stream) {
  MS_REQUIRE(num_tiles > 0, "attention_prefill: no tiles");
  MS_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0,
             "attention_prefill: %d query heads are not a multiple of %d kv heads", num_q_heads, num_kv_heads);
  MS_REQUIRE(ms_attention_prefill_supported(head_dim, block_size),
             "attention_prefill: head_dim %d (multiples of 16 up to 128) or block_size %d (multiples of 16) "
             "is not supported",
             head_dim, block_size);
  MS_REQUIRE(max_blocks > 0 && window >= 0, "attention_prefill: bad table width or window");
  const int group = num_q_heads / num_kv_heads;
  // four heads a wave only where the registers hold them
  const int hb = (group >= 4 && head_dim <= 64) ? 4 : (group >= 2 ? 2 : 1);
  MS_REQUIRE(num_kv_heads * ((group + hb - 1) / hb) <= 65535, "attention_prefill: too many heads");
#define MS_PREFILL_CASE(DIM)                                                                                       \
  case DIM:                                                                                                        \
    launch_prefill_heads<DIM>(hb, q, key_pool, value_pool, block_table, positions, tile_seq, tile_token, tile_count, \
                              out, num_tiles, num_q_heads, num_kv_heads, block_size, max_blocks, scale, window,     \
                              stream);                                                                             \
    break;
  switch (head_dim) {
    MS_PREFILL_CASE(16) MS_PREFILL_CASE(32) MS_PREFILL_CASE(48) MS_PREFILL_CASE(64) MS_PREFILL_CASE(80)
    MS_PREFILL_CASE(96) MS_PREFILL_CASE(112) MS_PREFILL_CASE(128)
    default:
      return ms_fail("attention_prefill: head_dim %d", head_dim);
  }
#undef MS_PREFILL_CASE
  MS_CHECK_LAUNCH("attention_prefill");
  return 0;
}
