// Paged causal attention for rows that bring runs of query tokens (prompts and
// their portions), bfloat16 storage, matrix cores.
//
// A workgroup of 4 waves owns a tile of up to 64 consecutive query tokens of one
// sequence and HB query heads that share a kv head; each wave owns 16 of the tokens:
// 16 * HB columns.  The workgroup walks the keys 0 .. (its last token's position)
// in pairs of tiles of 16; all threads load a pair together (16 bytes a thread,
// three pairs in flight in registers) into one of two LDS buffers, and every wave
// reads its matrix-core operands from there.  Each wave keeps for every column an
// online softmax in 32-bit:
//
//   S^T[key, query] = K[key, :] . Q[query, :]     A = K tile, B = Q^T (16 queries of one head)
//   P = exp(S * scale - m), masked to lo <= key <= position of the query
//   O[query, d]    += P[query, keys] . V[keys, d]
//
// Every key and value read from memory serves all 64 * HB columns.  The mask is by
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

constexpr int kQueryTile = 16;        // query tokens of one wave
constexpr int kBlockWaves = 4;        // waves of a workgroup: 64 query tokens share the keys and values in LDS
constexpr int kBlockThreads = kBlockWaves * ms::kWave;

template <int D, int HB>
struct PrefillState {
  floatx4 o[HB][D / 16];
  float run_max[HB], run_sum[HB];   // of query column r (the same in all four lane groups)
};

// Softmax arithmetic runs in base 2: scores are multiplied by scale * log2(e) once
// and exp2 is one instruction.  The running maximum of a column moves only when a
// tile exceeds it by more than kMaxSlack (in base-2 units): weights may then be as
// large as 2^kMaxSlack instead of 1, which 32-bit sums and bfloat16 weights hold
// without loss, and the rescaling of the output tile - the most expensive vector
// work of a step - is skipped for the steps in which no column's maximum moved.
constexpr float kMaxSlack = 6.0f;

template <int D, int HB>
__device__ __forceinline__ void consume_pair(PrefillState<D, HB>& st, TilePair<D>& pair,
                                             const bf16x8 (&q_reg)[HB][TilePair<D>::KS], int tile, int lo, int pos,
                                             int last_key, float scale_log2, int g, bool all_visible) {
  constexpr int KS = TilePair<D>::KS, CS = TilePair<D>::CS;
  const int key_a = tile * kTileKeys, key_b = key_a + kTileKeys;
  // this lane: query column r (position pos, window start lo), keys key_a + 4 g + e and key_b + 4 g + e
  bool ok_a[4], ok_b[4];
  if (!all_visible) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int ka = key_a + 4 * g + e, kb = key_b + 4 * g + e;
      ok_a[e] = ka >= lo && ka <= pos;
      ok_b[e] = pair.has_b && kb >= lo && kb <= pos;
    }
  }
  float alpha[HB];
  bf16x8 p[HB];
  bool moved = false;
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
      s_a[e] *= scale_log2;
      s_b[e] *= scale_log2;
      if (!all_visible) {
        s_a[e] = ok_a[e] ? s_a[e] : -INFINITY;
        s_b[e] = ok_b[e] ? s_b[e] : -INFINITY;
      }
      tile_max = fmaxf(tile_max, fmaxf(s_a[e], s_b[e]));
    }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, ms::kWave));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, ms::kWave));
    // the maximum moves only when it is exceeded by more than the slack (or is still unset)
    const bool move = tile_max > st.run_max[hb] + kMaxSlack;
    const float new_max = move ? tile_max : st.run_max[hb];
    // a column may have seen no key yet: keep everything at zero
    const float safe_max = new_max == -INFINITY ? 0.f : new_max;
    alpha[hb] = move ? ms::fast_exp2(st.run_max[hb] - safe_max) : 1.0f;
    moved = moved || move;
    float tile_sum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float pa = ms::fast_exp2(s_a[e] - safe_max);
      const float pb = ms::fast_exp2(s_b[e] - safe_max);
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
  if (__any(moved)) {
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      float alpha_row[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) alpha_row[e] = __shfl(alpha[hb], 4 * g + e, ms::kWave);
#pragma unroll
      for (int c = 0; c < CS; ++c)
#pragma unroll
        for (int e = 0; e < 4; ++e) st.o[hb][c][e] *= alpha_row[e];
    }
  }
  // A stale value (a slot beyond what the sequence has written) times a zero weight
  // must not become NaN: such slots exist only in the pair that holds the last key.
  const bool has_stale = key_b + kTileKeys - 1 > last_key;
#pragma unroll
  for (int c = 0; c < CS; ++c) {
    bf16x4 va = pair.v_a[c], vb = pair.v_b[c];
    if (has_stale) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (key_a + 4 * g + e > last_key) va[e] = static_cast<__bf16>(0.0f);
        if (key_b + 4 * g + e > last_key) vb[e] = static_cast<__bf16>(0.0f);
      }
    }
    const bf16x8 v = ms::concat(va, vb);
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) st.o[hb][c] = ms::mfma_16x16x32(p[hb], v, st.o[hb][c]);
  }
}

// Keys and values of one pair of tiles in LDS.  Rows are padded so that the 16 lanes
// that read 16 different rows spread over the banks.
template <int D>
struct alignas(16) PairBuffer {
  static constexpr int kKeyRow = D + 8;      // elements; 16-byte aligned rows
  static constexpr int kValueRow = 24;       // 16 keys of one value column + padding
  bf16 k[2 * kTileKeys][kKeyRow];
  bf16 v[2][D][kValueRow];
};

// The share of one thread in the cooperative load of a pair: 16-byte chunks, the
// same number for keys and for values.
template <int D>
struct StagedPair {
  static constexpr int kChunks = 4 * D;                        // of keys; as many of values
  static constexpr int kPerThread = (kChunks + kBlockThreads - 1) / kBlockThreads;
  bf16x8 k[kPerThread], v[kPerThread];
};

template <int D>
__device__ __forceinline__ void stage_load(StagedPair<D>& staged, int tile, int end_tile,
                                           const int32_t* __restrict__ table, const bf16* __restrict__ key_pool,
                                           const bf16* __restrict__ value_pool, int num_kv_heads, int kv_head,
                                           int block_size) {
  // No branch stands around a load: the counters that order the loads of the three
  // register sets stay exact.  A pair past the end repeats the last one and a missing
  // second tile repeats the first; what they hold lies beyond the last key and is masked.
  tile = min(tile, end_tile - 1);
  const bool has_b = tile + 1 < end_tile;
  const int key_a = tile * kTileKeys, key_b = key_a + kTileKeys;
  const int second_key = has_b ? key_b : key_a;
  const int64_t page_a = table[key_a / block_size];
  const int off_a = key_a % block_size;
  const int64_t page_b = table[second_key / block_size];
  const int off_b = second_key % block_size;
#pragma unroll
  for (int j = 0; j < StagedPair<D>::kPerThread; ++j) {
    // small heads have fewer chunks than threads: the surplus threads repeat the last chunk
    const int chunk = min(static_cast<int>(threadIdx.x) + j * kBlockThreads, StagedPair<D>::kChunks - 1);
    {   // keys: chunk -> (key 0..31, 8 consecutive d)
      const int key = chunk / (D / 8), part = chunk - key * (D / 8);
      const bool second = key >= kTileKeys;
      const int64_t page = second ? page_b : page_a;
      const int offset = (second ? off_b : off_a) + (key & (kTileKeys - 1));
      staged.k[j] = ms::load_bf16x8(key_pool + ((page * num_kv_heads + kv_head) * block_size + offset) * D + 8 * part);
    }
    {   // values: chunk -> (tile, column d, 8 consecutive keys)
      const int tile_index = chunk / (2 * D), rest = chunk - tile_index * 2 * D;
      const int d = rest >> 1, half = rest & 1;
      const int64_t page = tile_index ? page_b : page_a;
      const int offset = (tile_index ? off_b : off_a) + 8 * half;
      staged.v[j] = ms::load_bf16x8(value_pool + ((page * num_kv_heads + kv_head) * D + d) * block_size + offset);
    }
  }
}

template <int D>
__device__ __forceinline__ void stage_store(const StagedPair<D>& staged, PairBuffer<D>& buffer) {
#pragma unroll
  for (int j = 0; j < StagedPair<D>::kPerThread; ++j) {
    const int chunk = min(static_cast<int>(threadIdx.x) + j * kBlockThreads, StagedPair<D>::kChunks - 1);
    const int key = chunk / (D / 8), part = chunk - key * (D / 8);
    *reinterpret_cast<bf16x8*>(&buffer.k[key][8 * part]) = staged.k[j];
    const int tile_index = chunk / (2 * D), rest = chunk - tile_index * 2 * D;
    *reinterpret_cast<bf16x8*>(&buffer.v[tile_index][rest >> 1][8 * (rest & 1)]) = staged.v[j];
  }
}

// The pair's operands of this lane, read from LDS.
template <int D>
__device__ __forceinline__ void read_pair(TilePair<D>& pair, const PairBuffer<D>& buffer, bool has_b, int g, int r) {
  pair.has_b = has_b;
#pragma unroll
  for (int s = 0; s < TilePair<D>::KS; ++s) {
    const int d0 = 32 * s + 8 * g;
    if (d0 < D) {
      pair.k_a[s] = *reinterpret_cast<const bf16x8*>(&buffer.k[r][d0]);
      pair.k_b[s] = *reinterpret_cast<const bf16x8*>(&buffer.k[kTileKeys + r][d0]);
    } else {
      pair.k_a[s] = ms::zero_bf16x8();
      pair.k_b[s] = ms::zero_bf16x8();
    }
  }
#pragma unroll
  for (int c = 0; c < TilePair<D>::CS; ++c) {
    pair.v_a[c] = *reinterpret_cast<const bf16x4*>(&buffer.v[0][16 * c + r][4 * g]);
    pair.v_b[c] = *reinterpret_cast<const bf16x4*>(&buffer.v[1][16 * c + r][4 * g]);
  }
}

template <int D, int HB>
__global__ __launch_bounds__(kBlockThreads) void attention_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ key_pool, const bf16* __restrict__ value_pool,
    const int32_t* __restrict__ block_table, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_token, const int32_t* __restrict__ tile_count,
    bf16* __restrict__ out, int num_q_heads, int num_kv_heads, int block_size, int max_blocks, float scale,
    int window) {
  constexpr int KS = TilePair<D>::KS, CS = TilePair<D>::CS;
  __shared__ PairBuffer<D> buffers[2];

  const int lane = threadIdx.x & 63;
  const int wave = ms::uniform(threadIdx.x >> 6);   // the same in all lanes: kept in a scalar register
  const int g = lane >> 4;
  const int r = lane & 15;

  const int tile_index = blockIdx.x;
  const int group = num_q_heads / num_kv_heads;
  const int head_blocks = (group + HB - 1) / HB;
  const int kv_head = blockIdx.y / head_blocks;
  const int head0 = kv_head * group + (blockIdx.y - kv_head * head_blocks) * HB;
  const int heads_here = min(HB, kv_head * group + group - head0);

  // The workgroup's tile: up to 64 consecutive tokens of one sequence; wave w owns tokens 16 w .. 16 w + 15.
  const int token0 = tile_token[tile_index];
  const int count = tile_count[tile_index];
  const int32_t* table = block_table + static_cast<int64_t>(tile_seq[tile_index]) * max_blocks;
  const int first_pos = positions[token0];
  const int last_key = first_pos + count - 1;          // all keys up to it are written
  const int first_lo = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  const int t0 = first_lo / kTileKeys;
  const int t1 = last_key / kTileKeys + 1;

  const int my_count = max(0, min(kQueryTile, count - kQueryTile * wave));
  // query column r of this lane; a column past the wave's tokens repeats the last one and is not stored
  const int64_t my_token = token0 + (my_count > 0 ? kQueryTile * wave + min(r, my_count - 1) : 0);
  const int pos = positions[my_token];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int wave_last_key = my_count > 0 ? first_pos + kQueryTile * wave + my_count - 1 : -1;
  const int wave_first_pos = first_pos + kQueryTile * wave;
  const int wave_first_lo = (window > 0 && wave_first_pos - window + 1 > 0) ? wave_first_pos - window + 1 : 0;
  const int wave_last_lo = (window > 0 && wave_last_key - window + 1 > 0) ? wave_last_key - window + 1 : 0;
  const float scale_log2 = scale * 1.4426950408889634f;

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

  // Three pairs in flight in registers, two buffers in LDS: the loads of pair i + 3
  // are issued before pair i is consumed.  The loop is unrolled by hand over the three
  // register sets: a copy from one set to another would have to wait for its loads.
  StagedPair<D> ring0, ring1, ring2;
  stage_load<D>(ring0, t0, t1, table, key_pool, value_pool, num_kv_heads, kv_head, block_size);
  stage_load<D>(ring1, t0 + 2, t1, table, key_pool, value_pool, num_kv_heads, kv_head, block_size);
  stage_load<D>(ring2, t0 + 4, t1, table, key_pool, value_pool, num_kv_heads, kv_head, block_size);
  int parity = 0;
  auto step = [&](StagedPair<D>& staged, int t) {
    PairBuffer<D>& buffer = buffers[parity];
    stage_store<D>(staged, buffer);
    stage_load<D>(staged, t + 6, t1, table, key_pool, value_pool, num_kv_heads, kv_head, block_size);
    __syncthreads();    // the pair is in LDS; every wave is done with the other buffer's previous content
    if (t < t1 && t * kTileKeys <= wave_last_key && (t + 2) * kTileKeys > wave_first_lo) {
      TilePair<D> pair;
      read_pair<D>(pair, buffer, t + 1 < t1, g, r);
      // every key of the pair visible to every query of the wave: no masks
      const bool all_visible = (t + 2) * kTileKeys - 1 <= wave_first_pos && t * kTileKeys >= wave_last_lo;
      consume_pair<D, HB>(st, pair, q_reg, t, lo, pos, last_key, scale_log2, g, all_visible);
    }
    parity ^= 1;
  };
  // Straight-line body (three steps, no exit between them): steps past the end load
  // and store a repeated pair and consume nothing.
  for (int t = t0; t < t1; t += 6) {
    step(ring0, t);
    step(ring1, t + 2);
    step(ring2, t + 4);
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
      if (row >= my_count) continue;
      bf16* dst = out + ((static_cast<int64_t>(token0) + kQueryTile * wave + row) * num_q_heads + head0 + hb) * D;
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
  hipLaunchKernelGGL((attention_prefill_kernel<D, HB>), grid, dim3(kBlockThreads), 0, stream, static_cast<const bf16*>(q),
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
// at most 64 consecutive tokens of one sequence: tile_seq (row of block_table),
// tile_token (index of its first token), tile_count (1..64), all int32 [num_tiles].
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
  const int hb = group >= 4 ? 4 : (group >= 2 ? 2 : 1);   // query heads of one workgroup
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
