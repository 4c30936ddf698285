// Paged causal attention for rows that bring runs of query tokens (prompts and
// their portions), bfloat16 storage, matrix cores.
//
// A workgroup owns a tile of up to 64 consecutive query tokens of one sequence and HB
// query heads that share a kv head: 64 * HB columns, 32 to a wave (16 tokens of two
// heads, or 32 tokens of one).  It walks the keys 0 .. (its last token's position) in
// pairs of tiles of 16; its threads load a pair together (16 bytes a thread) into an
// LDS buffer, and every wave reads its matrix-core operands from there.  The keys are
// dealt out to PARTS parts of the workgroup (two parts of two heads, or four parts of
// one head: eight waves either way, two to a SIMD), which are joined through LDS at
// the end.  A workgroup may take two tiles one after the other, a long one and a short
// one, so that all workgroups of a launch have about the same number of keys to walk.  With
// 32x32x16 products
//
//   S^T[key, column]  = K[key, :] . Q[column, :]       A = 32 keys, B = Q^T
//   P = exp(S * scale - m), masked to lo <= key <= position of the column's token
//   O^T[d, column]   += V^T[d, keys] . P^T[keys, column]
//
// a column's scores, its running maximum and sum and its outputs all live in the two
// lanes column and column + 32: the online softmax needs one exchange between the
// halves of the wave a step, and rescaling and the final division are per lane.
// Every key and value read from memory serves all 64 * HB columns.  The mask is by
// absolute position, so a portion of a prompt sees the history in the cache and
// itself (reference: miniserve/model/qwen3.py:237-249, where the scores of a chunk
// are a dense product over the gathered history).
#include "attention_tiles.hpp"

namespace {

using ms::bf16;
using ms::bf16x4;
using ms::bf16x8;
using ms::floatx16;
using ms::kTileKeys;

constexpr int kXcds = 8;    // dies of the chip, each with an L2 of its own (a wrong number costs speed only)
constexpr int kWaveColumns = 32;      // columns (token, head) of one wave

// Softmax arithmetic runs in base 2: the scale and log2(e) enter the exponent's
// argument by one fused multiply-add and exp2 is one instruction.  The running
// maximum of a column moves only when a step exceeds it by more than kMaxSlack (in
// base-2 units): weights may then be as large as 2^kMaxSlack instead of 1, which
// 32-bit sums and bfloat16 weights hold without loss, and the rescaling of the
// output - the most expensive vector work of a step - is skipped for the steps in
// which no column's maximum moved.
constexpr float kMaxSlack = 6.0f;

// Keys and values of one pair of tiles in LDS.  Rows are padded so that lanes that
// read different rows spread over the banks (16 lanes that read 16 bytes each of
// consecutive rows touch every bank once, for keys and for values).
//
// A row of values holds the 16 keys of its tile in the order in which the product
// P.V wants them: the scores' product leaves lane half h with the keys 4h..4h+3 and
// 8+4h..8+4h+3 of a tile, so the groups of four keys lie in the order 0, 2, 1, 3 and a
// lane reads its eight values as one 16-byte word.
//
// Key rows of 128 elements are not padded (eight buffers of them must fit the LDS):
// the 16-byte chunk c of row r lies at chunk c ^ (r & 15) instead.
template <int D>
struct alignas(16) PairBuffer {
  static constexpr bool kSwizzled = D == 128;
  static constexpr int kKeyRow = kSwizzled ? D : D + 8;      // elements; 16-byte aligned rows
  static constexpr int kValueRow = 24;                       // 16 keys of one value column + padding
  bf16 k[2 * kTileKeys][kKeyRow];
  bf16 v[2][D][kValueRow];
  // where the 8 elements from d = 8 * chunk of key row `row` lie
  __device__ __forceinline__ bf16* key_chunk(int row, int chunk) {
    return &k[row][8 * (kSwizzled ? (chunk ^ (row & 15)) : chunk)];
  }
  __device__ __forceinline__ const bf16* key_chunk(int row, int chunk) const {
    return &k[row][8 * (kSwizzled ? (chunk ^ (row & 15)) : chunk)];
  }
};

// The share of one thread in the cooperative load of a pair: 16-byte chunks, the
// same number for keys and for values, tile by tile, so that every load has a base
// that is the same in all lanes (a scalar register pair) and a 32-bit lane offset
// that never changes.
template <int D, int THREADS>
struct StagedPair {
  static constexpr int kTileChunks = 2 * D;                    // of one tile's keys; as many of its values
  static constexpr int kPerTile = (kTileChunks + THREADS - 1) / THREADS;
  bf16x8 k[2][kPerTile], v[2][kPerTile];
};

// chunk of a tile -> element offsets in the cache (from the tile's first key, and from
// the same offset of the page's value rows) and in the LDS buffer
template <int D, int THREADS>
struct ChunkPlace {
  int key, part;     // keys: (key 0..15, 8 consecutive d)
  int d, half;       // values: (column d, keys 8 half .. 8 half + 7)
  __device__ __forceinline__ ChunkPlace(int thread, int j) {
    // small heads have fewer chunks than threads: the surplus threads repeat the last chunk
    const int chunk = min(thread + j * THREADS, StagedPair<D, THREADS>::kTileChunks - 1);
    key = chunk / (D / 8);
    part = chunk - key * (D / 8);
    d = chunk >> 1;
    half = chunk & 1;
  }
};

// Where the two tiles of a pair lie in the cache: the page of each and the offset of its
// first key in the page.  The same in every lane (scalar registers); looked up from the
// block table two rounds before the pair's loads are issued, so that nothing waits for
// the table.
struct PairPages {
  int32_t page[2];
  int offset[2];
};

__device__ __forceinline__ PairPages find_pair(int tile, int end_tile, const int32_t* __restrict__ table,
                                               int block_size) {
  // A pair past the end repeats the last one and a missing second tile repeats the
  // first; what they hold lies beyond the last key and is masked.
  tile = min(tile, end_tile - 1);
  PairPages pages;
#pragma unroll
  for (int side = 0; side < 2; ++side) {
    const int this_tile = side == 1 && tile + 1 < end_tile ? tile + 1 : tile;
    if (block_size == kTileKeys) {      // a page is a tile: no division
      pages.page[side] = ms::uniform(table[this_tile]);
      pages.offset[side] = 0;
    } else {
      const int first_key = this_tile * kTileKeys;
      pages.page[side] = ms::uniform(table[first_key / block_size]);
      pages.offset[side] = first_key % block_size;
    }
  }
  return pages;
}

// page_stride: elements of one page of a pool (all its kv heads); head_base: where the
// workgroup's kv head begins in a page.  Both are the same for keys and values.
template <int D, int THREADS>
__device__ __forceinline__ void stage_load(StagedPair<D, THREADS>& staged, int thread, const PairPages& pages,
                                           const bf16* __restrict__ key_pool, const bf16* __restrict__ value_pool,
                                           int64_t page_stride, int head_base, int block_size) {
  // No branch stands around a load: the counters that order the loads stay exact.
#pragma unroll
  for (int side = 0; side < 2; ++side) {
    const int64_t slab = pages.page[side] * page_stride + head_base;
    const bf16* keys = key_pool + slab + pages.offset[side] * D;
    const bf16* values = value_pool + slab + pages.offset[side];
#pragma unroll
    for (int j = 0; j < StagedPair<D, THREADS>::kPerTile; ++j) {
      const ChunkPlace<D, THREADS> place(thread, j);
      staged.k[side][j] = ms::load_bf16x8(keys + static_cast<uint32_t>(place.key * D + 8 * place.part));
      staged.v[side][j] = ms::load_bf16x8(values + static_cast<uint32_t>(place.d * block_size + 8 * place.half));
    }
  }
}

template <int D, int THREADS>
__device__ __forceinline__ void stage_store(const StagedPair<D, THREADS>& staged, int thread, PairBuffer<D>& buffer) {
#pragma unroll
  for (int side = 0; side < 2; ++side)
#pragma unroll
    for (int j = 0; j < StagedPair<D, THREADS>::kPerTile; ++j) {
      const ChunkPlace<D, THREADS> place(thread, j);
      *reinterpret_cast<bf16x8*>(buffer.key_chunk(side * kTileKeys + place.key, place.part)) = staged.k[side][j];
      // keys 8 half .. 8 half + 7: the groups 2 half and 2 half + 1, which lie at 4 half and 8 + 4 half
      const bf16x8 values = staged.v[side][j];
      *reinterpret_cast<bf16x4*>(&buffer.v[side][place.d][4 * place.half]) = bf16x4{values[0], values[1], values[2], values[3]};
      *reinterpret_cast<bf16x4*>(&buffer.v[side][place.d][8 + 4 * place.half]) =
          bf16x4{values[4], values[5], values[6], values[7]};
    }
}

// What a wave keeps of its 32 columns: this lane holds column `lane & 31`; of the
// 32 x 32 outputs of a product it holds rows 8 (v / 4) + 4 h + v % 4, h = lane / 32.
template <int D>
struct PrefillState {
  static constexpr int CS = (D + 31) / 32;   // blocks of 32 rows of O^T
  floatx16 o[CS];
  float run_max;    // scaled by log2(e) * scale; the same in both lanes of a column
  float run_sum;    // of this lane's keys only; the two lanes are added at the end
};

// One pair of key tiles (32 keys from `key0`) against the wave's 32 columns.  `masked`
// (the same in all lanes): some key of the pair is hidden from some column, or lies
// beyond what the sequence has written.  One body serves both cases, so that the
// outputs stay in the same registers whichever way a step goes.
template <int D>
__device__ __forceinline__ void consume_pair(PrefillState<D>& st, const PairBuffer<D>& buffer,
                                             const bf16x8 (&q_reg)[D / 16], int key0, int lo, int pos, int last_key,
                                             float scale_log2, int h, int column, bool masked) {
  constexpr int KS = D / 16, CS = PrefillState<D>::CS;
  floatx16 s;
#pragma unroll
  for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
  for (int step = 0; step < KS; ++step) {
    const bf16x8 keys = *reinterpret_cast<const bf16x8*>(buffer.key_chunk(column, 2 * step + h));
    s = ms::mfma_32x32x16(keys, q_reg[step], s);
  }
  // The values of the step are asked for now; they arrive while the weights are made.
  // slot x of the contraction index of half j: key0 + 16 j + 8 (x / 4) + 4 h + x % 4,
  // for P (registers 8 j + x below) and for V alike.
  bf16x8 values[CS][2];
#pragma unroll
  for (int c = 0; c < CS; ++c) {
    const int d = (D % 32 == 0) ? 32 * c + column : min(32 * c + column, D - 1);
#pragma unroll
    for (int j = 0; j < 2; ++j) values[c][j] = *reinterpret_cast<const bf16x8*>(&buffer.v[j][d][8 * h]);
  }
  // register v: key0 + 8 (v / 4) + 4 h + v % 4
  if (masked) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int key = key0 + 8 * (v / 4) + 4 * h + (v % 4);
      s[v] = (key >= lo && key <= pos) ? s[v] : -INFINITY;
    }
    // A stale value (a slot beyond what the sequence has written) times a zero weight
    // must not become NaN: such slots exist only in steps that are masked.
#pragma unroll
    for (int c = 0; c < CS; ++c)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int x = 0; x < 8; ++x)
          if (key0 + 16 * j + 8 * (x / 4) + 4 * h + (x % 4) > last_key) values[c][j][x] = static_cast<__bf16>(0.0f);
  }
  float tile_max = -INFINITY;
#pragma unroll
  for (int v = 0; v < 16; ++v) tile_max = fmaxf(tile_max, s[v]);
  tile_max = ms::max_xor32(tile_max) * scale_log2;
  // the maximum moves only when it is exceeded by more than the slack (or is still unset)
  const bool move = tile_max > st.run_max + kMaxSlack;
  const float new_max = move ? tile_max : st.run_max;
  // a column may have seen no key yet: keep everything at zero
  const float safe_max = new_max == -INFINITY ? 0.f : new_max;
  float tile_sum = 0.f;
  bf16x8 p[2];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const float weight = ms::fast_exp2(fmaf(s[v], scale_log2, -safe_max));
    tile_sum += weight;
    p[v / 8][v % 8] = static_cast<__bf16>(weight);
  }
  if (__any(move)) {
    const float alpha = move ? ms::fast_exp2(st.run_max - safe_max) : 1.0f;
    st.run_sum *= alpha;
#pragma unroll
    for (int c = 0; c < CS; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) st.o[c][v] *= alpha;
  }
  st.run_sum += tile_sum;
  st.run_max = new_max;
#pragma unroll
  for (int c = 0; c < CS; ++c)
#pragma unroll
    for (int j = 0; j < 2; ++j) st.o[c] = ms::mfma_32x32x16(values[c][j], p[j], st.o[c]);
}

// At the end the parts of a workgroup share the finishing: of the blocks of 32 rows of
// O^T, block c is finished (joined over the parts, divided by the sum, stored) by part
// c % PARTS.  What a wave publishes for that: its maximum, its sum, and the blocks that
// another part finishes, lane by lane.
template <int D, int PARTS>
struct MergeSlot {
  static constexpr int CS = PrefillState<D>::CS;
  static constexpr int kBlocks = CS - CS / PARTS;      // most blocks that a part does not finish itself
  float value[kBlocks * 16 + 2][ms::kWave];
  // where part `part` keeps block c (which it does not finish): behind its other such blocks
  __device__ static __forceinline__ int place(int part, int c) {
    const int own_below = c > part ? (c - part - 1) / PARTS + 1 : 0;
    return c - own_below;
  }
};

template <int D, int HB, int PARTS>
constexpr size_t prefill_lds_bytes() {
  constexpr size_t buffers = 2 * PARTS * sizeof(PairBuffer<D>);
  constexpr size_t slots = PARTS * 2 * HB * sizeof(MergeSlot<D, PARTS>);
  return buffers > slots ? buffers : slots;
}

template <int D, int HB, int PARTS>
__global__ __launch_bounds__(128 * HB * PARTS) MS_WAVES_PER_EU(2, 2) void attention_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ key_pool, const bf16* __restrict__ value_pool,
    const int32_t* __restrict__ block_table, const int32_t* __restrict__ tile_seq,
    const int32_t* __restrict__ tile_token, const int32_t* __restrict__ tile_count,
    const int32_t* __restrict__ tile_first, bf16* __restrict__ out, int num_tiles, int paired, int num_q_heads, int num_kv_heads, int block_size,
    int max_blocks, float scale, int window) {
  // The workgroup is PARTS parts of 2 HB waves.  All hold the same 64 HB columns; part p
  // takes the pairs of key tiles p, p + PARTS, p + 2 PARTS, ... of the tile's range: two
  // waves on every SIMD, one in the matrix cores while the other is in its softmax, and
  // 1 / PARTS of the steps for the longest tile.  Each part loads its own pairs into its
  // own LDS buffers; at the end they exchange their states through LDS and each finishes
  // a share of the outputs.
  constexpr int PART_THREADS = 128 * HB;
  constexpr int PART_WAVES = 2 * HB;
  constexpr int KS = D / 16, CS = PrefillState<D>::CS;
  __shared__ __align__(16) unsigned char lds[prefill_lds_bytes<D, HB, PARTS>()];
  PairBuffer<D>* buffers = reinterpret_cast<PairBuffer<D>*>(lds);        // [parity][part]
  using Slot = MergeSlot<D, PARTS>;
  Slot* slots = reinterpret_cast<Slot*>(lds);                            // [part][wave]

  const int lane = threadIdx.x & 63;
  const int wave_of_group = ms::uniform(threadIdx.x >> 6);   // the same in all lanes: kept in a scalar register
  const int part_id = wave_of_group / PART_WAVES;
  const int wave = wave_of_group - part_id * PART_WAVES;
  const int thread = threadIdx.x - part_id * PART_THREADS;
  const int h = lane >> 5;
  const int column = lane & 31;

  const int group = num_q_heads / num_kv_heads;
  const int head_blocks = (group + HB - 1) / HB;
  // Which tile and which heads: the chip hands consecutive workgroups of a launch to its eight
  // XCDs in turn, and each XCD has an L2 of its own.  The launch is read so that an XCD works
  // through the tiles of one kv head after the other: what its workgroups read of keys and values
  // at a time is one head's, which they share in that L2 (16,384 tokens of 16 heads:
  // 911 -> 957 TFLOP/s; no difference at 2,048).  Where the heads do not divide among the XCDs,
  // heads run fastest over the launch.
  const int linear = ms::uniform(static_cast<int>(blockIdx.x + blockIdx.y * gridDim.x));
  const int grid_x = static_cast<int>(gridDim.x), grid_y = static_cast<int>(gridDim.y);
  int block_x, block_y;
  if (grid_y % kXcds == 0) {
    const int xcd = linear % kXcds, turn = linear / kXcds;
    block_y = xcd * (grid_y / kXcds) + turn / grid_x;
    block_x = turn - (turn / grid_x) * grid_x;
  } else {
    block_y = linear % grid_y;
    block_x = linear / grid_y;
  }
  const int kv_head = block_y / head_blocks;
  const int head0 = kv_head * group + (block_y - kv_head * head_blocks) * HB;
  const int heads_here = min(HB, kv_head * group + group - head0);
  const float scale_log2 = scale * 1.4426950408889634f;
  const int64_t page_stride = static_cast<int64_t>(num_kv_heads) * block_size * D;
  const int head_base = kv_head * block_size * D;

  // The tiles come sorted by the keys they walk, fewest first.  Long tiles go out first;
  // a paired workgroup takes the b-th longest and then the b-th shortest.
  const int passes = (paired && block_x != num_tiles - 1 - block_x) ? 2 : 1;
#pragma unroll 1
  for (int pass = 0; pass < passes; ++pass) {
    const int tile_index = pass == 0 ? num_tiles - 1 - block_x : block_x;
    if (pass > 0) __syncthreads();      // the hand-over of the tile before is read

    // The workgroup's tile: up to 64 consecutive tokens of one sequence, at consecutive
    // positions from the tile's first (all four numbers come with one trip to memory).
    const int token0 = tile_token[tile_index];
    const int count = tile_count[tile_index];
    const int32_t* table = block_table + static_cast<int64_t>(tile_seq[tile_index]) * max_blocks;
    const int first_pos = tile_first[tile_index];
    const int last_key = first_pos + count - 1;          // all keys up to it are written
    const int first_lo = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
    const int t0 = first_lo / kTileKeys;
    const int t1 = last_key / kTileKeys + 1;

    // The wave's columns: with one head 32 tokens, else 16 tokens of two heads.
    const int wave_token = HB == 1 ? kWaveColumns * wave : 16 * wave;
    const int wave_span = HB == 1 ? kWaveColumns : 16;
    const int my_head = HB == 1 ? 0 : (column >> 4);
    const int my_local = HB == 1 ? column : (column & 15);
    const int my_count = max(0, min(wave_span, count - wave_token));
    // a column past the wave's tokens repeats the last one and is not stored
    const int my_offset = my_count > 0 ? wave_token + min(my_local, my_count - 1) : 0;
    const int64_t my_token = token0 + my_offset;
    const bool head_live = my_head < heads_here;
    const int pos = first_pos + my_offset;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int wave_first_pos = first_pos + wave_token;
    const int wave_last_key = my_count > 0 ? wave_first_pos + my_count - 1 : -1;
    const int wave_first_lo = (window > 0 && wave_first_pos - window + 1 > 0) ? wave_first_pos - window + 1 : 0;
    const int wave_last_lo = (window > 0 && wave_last_key - window + 1 > 0) ? wave_last_key - window + 1 : 0;

    bf16x8 q_reg[KS];
#pragma unroll
    for (int step = 0; step < KS; ++step)
      q_reg[step] = head_live ? ms::load_bf16x8(q + (my_token * num_q_heads + head0 + my_head) * D + 16 * step + 8 * h)
                              : ms::zero_bf16x8();

    PrefillState<D> st;
#pragma unroll
    for (int c = 0; c < CS; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) st.o[c][v] = 0.f;
    st.run_max = -INFINITY;
    st.run_sum = 0.f;

    // Pairs in flight in registers, two buffers in LDS for each part: the loads of a pair
    // are issued kDepth rounds before it is consumed (a round is shorter than the way to
    // memory and back), two where the registers hold two (a part of 128 threads stages
    // twice as much a thread, and two pairs would spill).  No branch stands between a load
    // and its use; all parts make the same number of rounds, two to a turn of the loop so
    // that each buffer and each pair in flight is named at compile time.  A round is
    // 2 PARTS tiles of keys.
    constexpr int kRound = 2 * PARTS;
    constexpr int kDepth = StagedPair<D, PART_THREADS>::kPerTile > 1 ? 1 : 2;
    StagedPair<D, PART_THREADS> ahead[kDepth];
    PairPages pages[kDepth];
#pragma unroll
    for (int i = 0; i < kDepth; ++i) {
      const int first = t0 + 2 * part_id + kRound * i;
      stage_load<D, PART_THREADS>(ahead[i], thread, find_pair(first, t1, table, block_size), key_pool, value_pool,
                                  page_stride, head_base, block_size);
      pages[i] = find_pair(first + kDepth * kRound, t1, table, block_size);
    }
    for (int round_tile = t0; round_tile < t1; round_tile += 2 * kRound) {
#pragma unroll
      for (int parity = 0; parity < 2; ++parity) {
        constexpr int kUnused = 0;
        const int i = kDepth == 2 ? parity : kUnused;
        const int t = round_tile + kRound * parity + 2 * part_id;
        PairBuffer<D>& buffer = buffers[PARTS * parity + part_id];
        stage_store<D, PART_THREADS>(ahead[i], thread, buffer);
        stage_load<D, PART_THREADS>(ahead[i], thread, pages[i], key_pool, value_pool, page_stride, head_base,
                                    block_size);
        pages[i] = find_pair(t + 2 * kDepth * kRound, t1, table, block_size);
        __syncthreads();    // the pair is in LDS; every wave is done with the other buffers' previous content
        if (t < t1 && t * kTileKeys <= wave_last_key && (t + 2) * kTileKeys > wave_first_lo) {
          // every key of the pair visible to every column of the wave: no masks
          const bool all_visible = (t + 2) * kTileKeys - 1 <= wave_first_pos && t * kTileKeys >= wave_last_lo;
          consume_pair<D>(st, buffer, q_reg, t * kTileKeys, lo, pos, last_key, scale_log2, h, column, !all_visible);
        }
      }
    }

    // The parts exchange their states; the states of a column are joined as steps of the
    // online softmax are, the parts in their order whichever part does the sum.
    __syncthreads();    // everybody is done with what the memory held before
    {
      Slot& mine = slots[part_id * PART_WAVES + wave];
#pragma unroll
      for (int c = 0; c < CS; ++c) {
        if (c % PARTS == part_id) continue;
        const int at = 16 * Slot::place(part_id, c);
#pragma unroll
        for (int v = 0; v < 16; ++v) mine.value[at + v][lane] = st.o[c][v];
      }
      mine.value[16 * Slot::kBlocks][lane] = st.run_max;
      mine.value[16 * Slot::kBlocks + 1][lane] = st.run_sum;
    }
    __syncthreads();
    if (part_id >= CS) continue;      // no block of rows is this part's to finish
    float joint = st.run_max;
#pragma unroll
    for (int q = 0; q < PARTS; ++q)
      if (q != part_id) joint = fmaxf(joint, slots[q * PART_WAVES + wave].value[16 * Slot::kBlocks][lane]);
    // a part may have seen no key of a column: its share is zero
    float factor[PARTS];
    float total = 0.f;
#pragma unroll
    for (int q = 0; q < PARTS; ++q) {
      const Slot& theirs = slots[q * PART_WAVES + wave];
      const float part_max = q == part_id ? st.run_max : theirs.value[16 * Slot::kBlocks][lane];
      const float part_sum = q == part_id ? st.run_sum : theirs.value[16 * Slot::kBlocks + 1][lane];
      factor[q] = part_max == -INFINITY ? 0.f : ms::fast_exp2(part_max - joint);
      total += part_sum * factor[q];
    }
    // this lane: column's rows d = 32 c + 8 (v / 4) + 4 h + v % 4; its sum is shared with lane + 32
    total += __shfl_xor(total, 32, ms::kWave);
    const float inv = 1.0f / total;
    const bool stores = head_live && my_local < my_count;
    bf16* dst = out + (my_token * num_q_heads + head0 + my_head) * D;
#pragma unroll
    for (int c = 0; c < CS; ++c) {
      if (c % PARTS != part_id) continue;
      float row[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) row[v] = 0.f;
#pragma unroll
      for (int q = 0; q < PARTS; ++q) {
        if (q == part_id) {
#pragma unroll
          for (int v = 0; v < 16; ++v) row[v] = fmaf(st.o[c][v], factor[q], row[v]);
        } else {
          const Slot& theirs = slots[q * PART_WAVES + wave];
          const int at = 16 * Slot::place(q, c);
#pragma unroll
          for (int v = 0; v < 16; ++v) row[v] = fmaf(theirs.value[at + v][lane], factor[q], row[v]);
        }
      }
      if (!stores) continue;
#pragma unroll
      for (int quad = 0; quad < 4; ++quad) {
        const int d = 32 * c + 8 * quad + 4 * h;
        if (D % 32 != 0 && d >= D) continue;
        const uint32_t low = static_cast<uint32_t>(ms::float_to_bf16_bits(row[4 * quad] * inv)) |
                             (static_cast<uint32_t>(ms::float_to_bf16_bits(row[4 * quad + 1] * inv)) << 16);
        const uint32_t high = static_cast<uint32_t>(ms::float_to_bf16_bits(row[4 * quad + 2] * inv)) |
                              (static_cast<uint32_t>(ms::float_to_bf16_bits(row[4 * quad + 3] * inv)) << 16);
        *reinterpret_cast<uint2*>(dst + d) = make_uint2(low, high);
      }
    }
  }
}

template <int D, int HB, int PARTS>
void launch_prefill(const void* q, const void* key_pool, const void* value_pool, const void* block_table,
                    const void* tile_seq, const void* tile_token, const void* tile_count, const void* tile_first,
                    void* out, int num_tiles, int paired, int num_q_heads, int num_kv_heads, int block_size,
                    int max_blocks, float scale, int window, hipStream_t stream) {
  const int head_blocks = (num_q_heads / num_kv_heads + HB - 1) / HB;
  const dim3 grid(paired ? (num_tiles + 1) / 2 : num_tiles, num_kv_heads * head_blocks);
  hipLaunchKernelGGL((attention_prefill_kernel<D, HB, PARTS>), grid, dim3(128 * HB * PARTS), 0, stream,
                     static_cast<const bf16*>(q), static_cast<const bf16*>(key_pool),
                     static_cast<const bf16*>(value_pool), static_cast<const int32_t*>(block_table),
                     static_cast<const int32_t*>(tile_seq), static_cast<const int32_t*>(tile_token),
                     static_cast<const int32_t*>(tile_count), static_cast<const int32_t*>(tile_first),
                     static_cast<bf16*>(out), num_tiles, paired, num_q_heads, num_kv_heads, block_size, max_blocks,
                     scale, window);
}

template <int D>
void launch_prefill_heads(int hb, const void* q, const void* key_pool, const void* value_pool,
                          const void* block_table, const void* tile_seq, const void* tile_token,
                          const void* tile_count, const void* tile_first, void* out, int num_tiles, int paired,
                          int num_q_heads, int num_kv_heads, int block_size, int max_blocks, float scale, int window,
                          hipStream_t stream) {
  if (hb == 1) {
    launch_prefill<D, 1, 4>(q, key_pool, value_pool, block_table, tile_seq, tile_token, tile_count, tile_first, out,
                            num_tiles, paired, num_q_heads, num_kv_heads, block_size, max_blocks, scale, window, stream);
  } else {
    launch_prefill<D, 2, 2>(q, key_pool, value_pool, block_table, tile_seq, tile_token, tile_count, tile_first, out,
                            num_tiles, paired, num_q_heads, num_kv_heads, block_size, max_blocks, scale, window, stream);
  }
}

}  // namespace

// Whether ms_attention_prefill takes this geometry: head size a multiple of 16 up to
// 128, pages of a multiple of 16 keys.
extern "C" int ms_attention_prefill_supported(int head_dim, int block_size) {
  return head_dim >= 16 && head_dim <= 128 && head_dim % 16 == 0 && block_size % kTileKeys == 0;
}

// q, out: bfloat16 [num_tokens, num_q_heads, head_dim]; key_pool: [pages, kv_heads,
// block_size, head_dim]; value_pool: [pages, kv_heads, head_dim, block_size].  The
// query tokens are cut into num_tiles tiles of at most 64 consecutive tokens of one
// sequence, at consecutive positions: tile_seq (row of block_table), tile_token (index
// of its first token), tile_count (1..64), tile_first (position of its first token),
// all int32 [num_tiles].
// tile_order: not 0 if the tiles come in the order of the keys they walk, fewest first
// (then a workgroup may take a long and a short one; in any other order every workgroup
// takes one tile).
extern "C" int ms_attention_prefill(const void* q, const void* key_pool, const void* value_pool,
                                    const void* block_table, const void* tile_seq, const void* tile_token,
                                    const void* tile_count, const void* tile_first, void* out, int num_tiles,
                                    int tile_order, int num_q_heads, int num_kv_heads, int head_dim, int block_size,
                                    int max_blocks, float scale, int window, hipStream_t stream) {
  MS_REQUIRE(num_tiles > 0, "attention_prefill: no tiles");
  MS_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0,
             "attention_prefill: %d query heads are not a multiple of %d kv heads", num_q_heads, num_kv_heads);
  MS_REQUIRE(ms_attention_prefill_supported(head_dim, block_size),
             "attention_prefill: head_dim %d (multiples of 16 up to 128) or block_size %d (multiples of 16) "
             "is not supported",
             head_dim, block_size);
  MS_REQUIRE(max_blocks > 0 && window >= 0, "attention_prefill: bad table width or window");
  MS_REQUIRE(static_cast<int64_t>(num_kv_heads) * block_size * head_dim < (int64_t{1} << 31),
             "attention_prefill: a page of %d kv heads x %d keys x %d is too large", num_kv_heads, block_size, head_dim);
  const int group = num_q_heads / num_kv_heads;
  // Two query heads of a kv head to a workgroup (every key and value loaded serves both,
  // the keys dealt out to two parts) is the rule.  One head a workgroup, the keys dealt
  // out to four parts, gives twice the workgroups and half the steps for the longest
  // tile, at the price of loading every key and value for 64 columns instead of 128.  It
  // is taken for kv heads with one query head and for launches that would leave a quarter
  // of the chip without a workgroup (1,024 tokens of 16 heads: 25.6 -> 19.0 us).  (For
  // 256 workgroups of two heads it was measured both ways: one prompt of 2,048 tokens
  // gains by it when its tiles go out in pairs, 42 -> 37 us, steps of four portions of
  // 512 tokens with histories lose, 37 -> 46 us: left as the rule has it.)
  const bool sorted = tile_order != 0;
  const int64_t with_two = static_cast<int64_t>(num_tiles) * num_kv_heads * ((group + 1) / 2);
  const int units = ms_compute_units();      // a launch wants a workgroup for each
  const int hb = (group >= 2 && with_two >= units - units / 4) ? 2 : 1;
  const int64_t workgroups = static_cast<int64_t>(num_tiles) * num_kv_heads * ((group + hb - 1) / hb);
  // A long and a short tile to a workgroup where the pairs still fill the chip (256
  // compute units hold one workgroup each): then every workgroup walks about the same
  // number of keys (8,192 tokens of 16 heads: 396 -> 294 us).  A small launch keeps a tile
  // a workgroup: the longest tile sets its time either way, and a second tile costs a
  // workgroup a second start.
  const int paired = sorted && workgroups >= 2 * units - units / 4;
  MS_REQUIRE(num_kv_heads * ((group + hb - 1) / hb) <= 65535, "attention_prefill: too many heads");
#define MS_PREFILL_CASE(DIM)                                                                                       \
  case DIM:                                                                                                        \
    launch_prefill_heads<DIM>(hb, q, key_pool, value_pool, block_table, tile_seq, tile_token, tile_count, tile_first, \
                              out, num_tiles, paired, num_q_heads, num_kv_heads, block_size, max_blocks, scale,     \
                              window, stream);                                                                     \
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
