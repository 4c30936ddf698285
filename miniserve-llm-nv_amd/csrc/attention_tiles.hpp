// Tiles of keys and values as the matrix-core attention kernels read them from
// the paged cache (keys [page, kv_head, offset, d], values [page, kv_head, d, offset]).
#pragma once

#include "mfma.hpp"

namespace ms {

constexpr int kTileKeys = 16;

// The keys and values of two tiles (32 keys), as they are loaded: operands of the
// matrix cores without any rearrangement.
template <int D>
struct TilePair {
  static constexpr int KS = (D + 31) / 32;   // 32-wide slices of d for Q.K
  static constexpr int CS = D / 16;          // 16-wide slices of d for P.V
  bf16x8 k_a[KS], k_b[KS];
  bf16x4 v_a[CS], v_b[CS];
  bool has_b;
};

// Where the two tiles of a pair lie: the page of each and the offset of its first key
// in the page (the same in all lanes of a wave).  Looked up one step before the pair's
// loads go out, so that those do not wait for the block table.
struct PairPlace {
  int32_t page_a, page_b;
  int off_a, off_b;
  bool has_b;
};

__device__ __forceinline__ PairPlace find_pair(int tile, int end_tile, const int32_t* __restrict__ table,
                                               int block_size) {
  // a pair past the end is never loaded; it is looked up as the last tile so that the
  // table is not read beyond its row
  tile = min(tile, end_tile - 1);
  PairPlace place;
  place.has_b = tile + 1 < end_tile;
  const int key_a = tile * kTileKeys;
  const int key_b = place.has_b ? key_a + kTileKeys : key_a;
  if (block_size == kTileKeys) {      // a page is a tile: no division
    place.page_a = table[tile];
    place.page_b = table[place.has_b ? tile + 1 : tile];
    place.off_a = place.off_b = 0;
  } else {
    place.page_a = table[key_a / block_size];
    place.off_a = key_a % block_size;
    place.page_b = table[key_b / block_size];
    place.off_b = key_b % block_size;
  }
  return place;
}

template <int D>
__device__ __forceinline__ void load_pair(TilePair<D>& pair, const PairPlace& place, const bf16* __restrict__ key_pool,
                                          const bf16* __restrict__ value_pool, int num_kv_heads, int kv_head,
                                          int block_size, int g, int r) {
  const bool has_b = place.has_b;
  pair.has_b = has_b;
  const int64_t slab_a = static_cast<int64_t>(place.page_a) * num_kv_heads + kv_head;
  const int64_t slab_b = static_cast<int64_t>(place.page_b) * num_kv_heads + kv_head;
  const bf16* k_row_a = key_pool + (slab_a * block_size + place.off_a + r) * D;
  const bf16* k_row_b = key_pool + (slab_b * block_size + place.off_b + r) * D;
  const bf16* v_a = value_pool + slab_a * D * block_size + place.off_a + 4 * g;
  const bf16* v_b = value_pool + slab_b * D * block_size + place.off_b + 4 * g;
#pragma unroll
  for (int s = 0; s < TilePair<D>::KS; ++s) {
    const int d0 = 32 * s + 8 * g;
    pair.k_a[s] = d0 < D ? load_bf16x8(k_row_a + d0) : zero_bf16x8();
    pair.k_b[s] = (has_b && d0 < D) ? load_bf16x8(k_row_b + d0) : zero_bf16x8();
  }
#pragma unroll
  for (int c = 0; c < TilePair<D>::CS; ++c) {
    const int64_t d = 16 * c + r;
    pair.v_a[c] = load_bf16x4(v_a + d * block_size);
    pair.v_b[c] = has_b ? load_bf16x4(v_b + d * block_size) : zero_bf16x4();
  }
}

}  // namespace ms
