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
//
// The thresholds of top-k and top-p are found digit by digit, four bits a pass over
// the candidates.  With top-k or top-p only tokens near the row's maximum can stay:
// one pass over the row finds a distance below the maximum within which all of them
// lie, they are gathered into LDS in token order (at most 4096), and every later
// pass runs over that short list; a row whose candidates do not fit, and a row with
// neither top-k nor top-p, is handled over its whole length.
#include "common.hpp"
#include "miniserve_hip.h"

#include <mutex>

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / ms::kWave;
constexpr int kDigits = 15;     // candidates of one pass of a threshold search: four bits

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

// What the choice is made from: the whole row, or the few tokens of it that can
// still matter, gathered in LDS in token order.  value(i) is logit / temperature.
struct RowView {
  static constexpr bool kInDeviceMemory = true;
  const float* x;
  float temp;
  int size;
  __device__ __forceinline__ float value(int i) const { return x[i] / temp; }
  __device__ __forceinline__ int index(int i) const { return i; }
};

template <bool InDeviceMemory>
struct ListViewAt {
  static constexpr bool kInDeviceMemory = InDeviceMemory;
  const float* values;
  const int* indices;
  int size;
  __device__ __forceinline__ float value(int i) const { return values[i]; }
  __device__ __forceinline__ int index(int i) const { return indices[i]; }
};
using ListView = ListViewAt<false>;          // gathered in LDS
using LongListView = ListViewAt<true>;       // too long for that: where the gathering kernel left it

constexpr int kListCap = 4096;      // tokens that the short list holds at most
// Distances below the row's maximum (in units of logit / temperature) at which the
// row is cut to make the short list: the first of them that keeps enough is taken.
constexpr int kLadder = 10;
constexpr float kLadderDepth[kLadder] = {0.25f, 0.5f, 1.f, 2.f, 4.f, 6.f, 9.f, 13.f, 18.f, 26.f};

struct Scratch {
  float* f_scratch;       // [kWaves]
  int* i_scratch;         // [kWaves]
  float* seg_sum;         // [kThreads]
  int* seg_count;         // [kThreads]
  int* shared_index;
  float* shared_total;
  int (*digit_count)[kDigits];     // [kWaves][kDigits]
  float (*digit_mass)[kDigits];    // [kWaves][kDigits]
};

// The same choice among at most kSmallView tokens, one to a thread: no thresholds are
// searched; a token's rank (by value, lower index first among equals), the mass ahead of
// it and the running mass up to it are sums over the few tokens, which every thread takes
// in the same order.  seg_sum holds the values, then the weights; seg_count the indices.
constexpr int kSmallView = 256;

template <typename View>
__device__ int choose_among_few(const View& view, int limit_index, float scaled_max, int k, float p, float uniform,
                                float whole_mass, float mass_before, const Scratch& sc) {
  const int tid = threadIdx.x;
  const int n = view.size;
  const bool live = tid < n;
  const float value = live ? view.value(tid) : 0.f;
  const int index = live ? view.index(tid) : limit_index;
  const float weight = live ? expf(value - scaled_max) : 0.f;
  float* values = sc.seg_sum;
  float* weights = sc.seg_sum + kSmallView;
  int* indices = sc.seg_count;
  __syncthreads();                     // whoever read these arrays last is done
  if (live) values[tid] = value, indices[tid] = index;
  __syncthreads();
  bool kept = live;
  if (live && k > 0 && k < n) {
    int rank = 0;
    for (int j = 0; j < n; ++j) rank += values[j] > value || (values[j] == value && indices[j] < index);
    kept = rank < k;
  }
  if (live) weights[tid] = kept ? weight : 0.f;
  __syncthreads();
  if (p < 1.f) {
    float kept_mass = 0.f, ahead = 0.f;
    for (int j = 0; j < n; ++j) {
      kept_mass += weights[j];
      ahead += values[j] > value ? weights[j] : 0.f;
    }
    const float limit = p * (whole_mass >= 0.f ? whole_mass : kept_mass);
    kept = kept && !(ahead > limit);
    __syncthreads();                   // every thread has read the weights
    if (live) weights[tid] = kept ? weight : 0.f;
    __syncthreads();
  }
  float total = 0.f, running = 0.f;
  for (int j = 0; j < n; ++j) {
    total += weights[j];
    if (j == tid) running = total;     // the running mass up to and with this token
  }
  const float target = (k == 0 && !(p < 1.f) && whole_mass >= 0.f) ? uniform * whole_mass - mass_before
                                                                     : uniform * total;
  if (tid == 0) *sc.shared_index = limit_index;
  __syncthreads();
  if (live && kept && running > target) atomicMin(sc.shared_index, index);
  __syncthreads();
  const int chosen = *sc.shared_index;
  __syncthreads();
  // no token's running mass passes the target (rounding at the very end): the last kept one
  if (chosen == limit_index) {
    int last_kept = -1;
    for (int j = 0; j < n; ++j)
      if (weights[j] > 0.f) last_kept = max(last_kept, indices[j]);
    return last_kept >= 0 ? last_kept : indices[0];
  }
  return chosen;
}

// f(value, index) for the elements tid, tid + kThreads, ... of the view, in that order.
// Of a view in device memory eight at a time with their loads issued together: a loop that
// loads an element and then decides on it waits for memory once per element.
constexpr int kLoadsAhead = 8;

template <typename View, typename F>
__device__ __forceinline__ void for_each_strided(const View& view, int n, int tid, F&& f) {
  if constexpr (!View::kInDeviceMemory) {
    for (int i = tid; i < n; i += kThreads) f(view.value(i), view.index(i));
    return;
  }
  for (int base = tid; base < n; base += kLoadsAhead * kThreads) {
    float value[kLoadsAhead];
    int index[kLoadsAhead];
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u) {
      const int i = min(base + u * kThreads, n - 1);      // past the end: loaded again, not used
      value[u] = view.value(i);
      index[u] = view.index(i);
    }
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u)
      if (base + u * kThreads < n) f(value[u], index[u]);
  }
}

// The same for the consecutive elements begin .. end - 1 of one thread; f returns false to stop.
template <typename View, typename F>
__device__ __forceinline__ void for_each_in_order(const View& view, int begin, int end, F&& f) {
  if constexpr (!View::kInDeviceMemory) {
    for (int i = begin; i < end; ++i)
      if (!f(view.value(i), view.index(i))) return;
    return;
  }
  for (int base = begin; base < end; base += kLoadsAhead) {
    float value[kLoadsAhead];
    int index[kLoadsAhead];
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u) {
      const int i = min(base + u, end - 1);
      value[u] = view.value(i);
      index[u] = view.index(i);
    }
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u)
      if (base + u < end && !f(value[u], index[u])) return;
  }
}

// temperature -> top-k -> top-p -> draw over `view`; `limit_index`: an index beyond
// every token's; `whole_mass`: the mass of all tokens where the view holds only some
// of them and top-k is off (top_p is a share of that), else negative; `mass_before`:
// with top-k and top-p off and a view that is one part of the row, the mass of the
// tokens before it (the draw is then at uniform * whole_mass).  `preset_p_threshold`: the
// threshold of top-p where it was found elsewhere (p is 1 then, and whole_mass and
// mass_before are those of the kept tokens).  All threads of the workgroup call it and get
// the same result.
template <typename View>
__device__ int choose(const View& view, int limit_index, float scaled_max, int k, float p, float uniform,
                      float whole_mass, float mass_before, const Scratch& sc,
                      const uint32_t* preset_p_threshold = nullptr) {
  const int tid = threadIdx.x;
  const int n = view.size;
  // Contiguous segment of this thread, for everything that needs token order.
  const int seg = (n + kThreads - 1) / kThreads;
  const int seg_begin = min(tid * seg, n);
  const int seg_end = min(seg_begin + seg, n);

  if (n <= kSmallView && preset_p_threshold == nullptr)
    return choose_among_few(view, limit_index, scaled_max, k, p, uniform, whole_mass, mass_before, sc);

  Keep keep;
  keep.k_threshold = 0u;
  keep.tie_limit = limit_index;
  keep.p_threshold = preset_p_threshold ? *preset_p_threshold : 0u;

  // ---- top-k ----------------------------------------------------------------
  if (k > 0 && k < n) {
    // The k-th largest ordered value, four bits a pass: a thread counts, for each of the
    // 15 candidates threshold | c << shift, the values at or above it; the counts fall as c
    // rises, and the largest c that still has k values is the next digit.
    uint32_t threshold = 0u;
    for (int shift = 28; shift >= 0; shift -= 4) {
      int count[kDigits];
#pragma unroll
      for (int c = 0; c < kDigits; ++c) count[c] = 0;
      // A value whose bits above this digit differ from the threshold's lies above every
      // candidate or below every one: it is counted once, not fifteen times (over a long
      // view, where whole waves meet such values; among the few of a short list the branch
      // costs more than it saves).
      int above = 0;
      for_each_strided(view, n, tid, [&](float v, int) {
        const uint32_t o = ordered(v);
        if constexpr (View::kInDeviceMemory) {
          if (shift < 28 && ((o ^ threshold) >> (shift + 4)) != 0u) {
            above += o > threshold;
          } else {
            const int digit = static_cast<int>((o >> shift) & 15u);
#pragma unroll
            for (int c = 0; c < kDigits; ++c) count[c] += c < digit;
          }
        } else {
#pragma unroll
          for (int c = 0; c < kDigits; ++c) count[c] += o >= (threshold | (static_cast<uint32_t>(c + 1) << shift));
        }
      });
#pragma unroll
      for (int c = 0; c < kDigits; ++c) count[c] += above;
      __syncthreads();                    // the tables' last readers are done
#pragma unroll
      for (int c = 0; c < kDigits; ++c) {
        const int v = ms::wave_sum_int(count[c]);
        if ((tid & (ms::kWave - 1)) == 0) sc.digit_count[tid / ms::kWave][c] = v;
      }
      __syncthreads();
      if (tid < kDigits) {
        int total = 0;
        for (int w = 0; w < kWaves; ++w) total += sc.digit_count[w][tid];
        sc.digit_count[0][tid] = total;      // (only this thread reads column tid)
      }
      __syncthreads();
      int digit = 0;
      for (int c = 0; c < kDigits; ++c)
        if (sc.digit_count[0][c] >= k) digit = c + 1;
      threshold |= static_cast<uint32_t>(digit) << shift;
    }
    int greater = 0, equal = 0;
    for_each_in_order(view, seg_begin, seg_end, [&](float v, int) {
      const uint32_t o = ordered(v);
      greater += o > threshold;
      equal += o == threshold;
      return true;
    });
    const int total_greater = block_sum_int(greater, sc.i_scratch);
    const int wanted = k - total_greater;  // >= 1 equal values to keep, lowest indices first
    sc.seg_count[tid] = equal;
    __syncthreads();
    if (tid == 0) {
      int running = 0;
      for (int t = 0; t < kThreads; ++t) {
        const int c = sc.seg_count[t];
        sc.seg_count[t] = running;  // exclusive prefix
        running += c;
      }
      *sc.shared_index = limit_index;
    }
    __syncthreads();
    int seen = sc.seg_count[tid];
    int* const tie_index = sc.shared_index;
    for_each_in_order(view, seg_begin, seg_end, [&, tie_index](float v, int index) {
      if (ordered(v) == threshold) {
        ++seen;
        if (seen == wanted) *tie_index = index;  // exactly one thread reaches `wanted`
      }
      return true;
    });
    __syncthreads();
    keep.k_threshold = threshold;
    keep.tie_limit = *sc.shared_index;
    __syncthreads();
  }

  // ---- top-p ----------------------------------------------------------------
  if (p < 1.f) {
    float mass = 0.f;
    for_each_strided(view, n, tid, [&](float v, int index) {
      if (keep(ordered(v), index)) mass += expf(v - scaled_max);
    });
    const float kept_mass = ms::block_sum(mass, sc.f_scratch);
    const float limit = p * (whole_mass >= 0.f ? whole_mass : kept_mass);
    // Largest t with mass{ordered >= t} > limit; tokens at or above it stay.  Four bits a
    // pass, as for top-k, with the mass at or above each candidate in place of the count.
    uint32_t threshold = 0u;
    for (int shift = 28; shift >= 0; shift -= 4) {
      float part[kDigits];
#pragma unroll
      for (int c = 0; c < kDigits; ++c) part[c] = 0.f;
      float above = 0.f;      // of values above every candidate (see top-k)
      for_each_strided(view, n, tid, [&](float v, int index) {
        const uint32_t o = ordered(v);
        if (o >= threshold && keep(o, index)) {
          const float weight = expf(v - scaled_max);
          if constexpr (View::kInDeviceMemory) {
            if (shift < 28 && ((o ^ threshold) >> (shift + 4)) != 0u) {
              above += weight;
            } else {
              const int digit = static_cast<int>((o >> shift) & 15u);
#pragma unroll
              for (int c = 0; c < kDigits; ++c) part[c] += c < digit ? weight : 0.f;
            }
          } else {
#pragma unroll
            for (int c = 0; c < kDigits; ++c)
              part[c] += o >= (threshold | (static_cast<uint32_t>(c + 1) << shift)) ? weight : 0.f;
          }
        }
      });
#pragma unroll
      for (int c = 0; c < kDigits; ++c) part[c] += above;
      __syncthreads();
#pragma unroll
      for (int c = 0; c < kDigits; ++c) {
        const float v = ms::wave_sum(part[c]);
        if ((tid & (ms::kWave - 1)) == 0) sc.digit_mass[tid / ms::kWave][c] = v;
      }
      __syncthreads();
      if (tid < kDigits) {
        float total = 0.f;
        for (int w = 0; w < kWaves; ++w) total += sc.digit_mass[w][tid];
        sc.digit_mass[0][tid] = total;
      }
      __syncthreads();
      int digit = 0;
      for (int c = 0; c < kDigits; ++c)
        if (sc.digit_mass[0][c] > limit) digit = c + 1;
      threshold |= static_cast<uint32_t>(digit) << shift;
    }
    keep.p_threshold = threshold;
  }

  // ---- draw -----------------------------------------------------------------
  float mine = 0.f;
  int last_kept = -1;
  for_each_in_order(view, seg_begin, seg_end, [&](float v, int index) {
    if (keep(ordered(v), index)) {
      mine += expf(v - scaled_max);
      last_kept = index;
    }
    return true;
  });
  __syncthreads();
  sc.seg_sum[tid] = mine;
  sc.seg_count[tid] = last_kept;
  __syncthreads();
  if (tid == 0) {
    float running = 0.f;
    int last = -1;
    for (int t = 0; t < kThreads; ++t) {
      const float s = sc.seg_sum[t];
      sc.seg_sum[t] = running;  // exclusive prefix, in token order
      running += s;
      if (sc.seg_count[t] > last) last = sc.seg_count[t];
    }
    *sc.shared_total = running;
    *sc.shared_index = last;  // fallback: the last kept token
  }
  __syncthreads();
  const float target = (k == 0 && !(p < 1.f) && whole_mass >= 0.f) ? uniform * whole_mass - mass_before
                                                                     : uniform * *sc.shared_total;
  __syncthreads();
  float running = sc.seg_sum[tid];
  int* const first_past = sc.shared_index;
  for_each_in_order(view, seg_begin, seg_end, [&, first_past](float v, int index) {
    if (keep(ordered(v), index)) {
      running += expf(v - scaled_max);
      if (running > target) {
        atomicMin(first_past, index);
        return false;
      }
    }
    return true;
  });
  __syncthreads();
  return *sc.shared_index;
}

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
  __shared__ int digit_count[kWaves][kDigits];
  __shared__ float digit_mass[kWaves][kDigits];
  __shared__ int ladder_count[kWaves][kLadder];
  __shared__ float ladder_mass[kWaves][kLadder + 1];
  __shared__ int list_base[kWaves + 1];
  __shared__ int list_rung;
  __shared__ float list_whole_mass;
  __shared__ float list_values[kListCap];
  __shared__ int list_indices[kListCap];

  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & (ms::kWave - 1);
  const int wave = tid / ms::kWave;
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  const float temp = temperature ? temperature[row] : 0.f;
  Scratch sc;        // member by member: as one constant aggregate of LDS addresses the compiler cannot emit it
  sc.f_scratch = f_scratch;
  sc.i_scratch = i_scratch;
  sc.seg_sum = seg_sum;
  sc.seg_count = seg_count;
  sc.shared_index = &shared_index;
  sc.shared_total = &shared_total;
  sc.digit_count = digit_count;
  sc.digit_mass = digit_mass;

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

  const float scaled_max = row_max / temp;
  const int k = top_k ? top_k[row] : 0;
  const float p = top_p ? top_p[row] : 1.f;
  const bool cut_k = k > 0 && k < vocab;
  const bool cut_p = p < 1.f;

  // ---- the short list ---------------------------------------------------------
  // With top-k or top-p only tokens near the maximum can stay.  One pass counts, for
  // each rung of a ladder of distances below the maximum, the tokens at or above it
  // (and their mass): the first rung that holds k tokens (top-k), or more than top_p
  // of the whole mass (top-p alone), holds every token that can stay.  If they fit,
  // they are gathered in token order and the choice is made among them; else, and
  // without top-k and top-p, it is made over the whole row.  A wave reads a contiguous
  // part of the row, so that its share of the list is contiguous too.
  if (cut_k || cut_p) {
    const int chunk = ((vocab + kWaves - 1) / kWaves + ms::kWave - 1) / ms::kWave * ms::kWave;
    const int chunk_begin = min(wave * chunk, vocab);
    const int chunk_end = min(chunk_begin + chunk, vocab);
    int count[kLadder];
    float mass[kLadder + 1];
#pragma unroll
    for (int c = 0; c < kLadder; ++c) count[c] = 0, mass[c] = 0.f;
    mass[kLadder] = 0.f;
    for (int i = chunk_begin + lane; i < chunk_end; i += ms::kWave) {
      const float v = x[i] / temp;
      const float depth = scaled_max - v;
      const float weight = cut_k ? 0.f : expf(v - scaled_max);
      mass[kLadder] += weight;
#pragma unroll
      for (int c = 0; c < kLadder; ++c) {
        const bool in = depth <= kLadderDepth[c];
        count[c] += in;
        mass[c] += in ? weight : 0.f;
      }
    }
#pragma unroll
    for (int c = 0; c < kLadder; ++c) {
      const int total = ms::wave_sum_int(count[c]);
      const float sum = ms::wave_sum(mass[c]);
      if (lane == 0) ladder_count[wave][c] = total, ladder_mass[wave][c] = sum;
    }
    {
      const float sum = ms::wave_sum(mass[kLadder]);
      if (lane == 0) ladder_mass[wave][kLadder] = sum;
    }
    __syncthreads();
    if (tid == 0) {
      float whole = 0.f;
      for (int w = 0; w < kWaves; ++w) whole += ladder_mass[w][kLadder];
      int rung = -1;
      for (int c = 0; c < kLadder && rung < 0; ++c) {
        int total = 0;
        float sum = 0.f;
        for (int w = 0; w < kWaves; ++w) total += ladder_count[w][c], sum += ladder_mass[w][c];
        // (a little more than top_p of the mass: the sums here and those of the choice differ in rounding)
        const bool enough = cut_k ? total >= k : sum > (p + 1e-4f) * whole;
        if (enough && total <= kListCap) rung = c;
        if (total > kListCap) break;
      }
      list_rung = rung;
      list_whole_mass = whole;
      if (rung >= 0) {
        int running = 0;
        for (int w = 0; w < kWaves; ++w) {
          list_base[w] = running;
          running += ladder_count[w][rung];
        }
        list_base[kWaves] = running;
      }
    }
    __syncthreads();
    const int rung = list_rung;
    if (rung >= 0) {
      float deepest = 0.f;
#pragma unroll
      for (int c = 0; c < kLadder; ++c)
        if (c == rung) deepest = kLadderDepth[c];
      int written = list_base[wave];
      for (int base = chunk_begin; base < chunk_end; base += ms::kWave) {
        const int i = base + lane;
        float v = 0.f;
        bool in = false;
        if (i < chunk_end) {
          v = x[i] / temp;
          in = scaled_max - v <= deepest;
        }
        const unsigned long long mask = __ballot(in);
        if (in) {
          const int place = written + __popcll(mask & ((1ull << lane) - 1ull));
          list_values[place] = v;
          list_indices[place] = i;
        }
        written += __popcll(mask);
      }
      __syncthreads();
      const ListView list{list_values, list_indices, list_base[kWaves]};
      const int chosen = choose(list, vocab, scaled_max, cut_k ? k : 0, p, uniform[row],
                                cut_k ? -1.f : list_whole_mass, 0.f, sc);
      if (tid == 0) out[row] = chosen;
      return;
    }
  }
  const RowView whole{x, temp, vocab};
  const int chosen = choose(whole, vocab, scaled_max, cut_k ? k : 0, p, uniform[row], -1.f, 0.f, sc);
  if (tid == 0) out[row] = chosen;
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

// ---- the greedy choice for callers that cannot allocate ---------------------------------
//
// The partial results of stage 1 lie in a file-scope device array instead of buffers
// that the caller brings: kStaticArgmaxMaxRows rows x kStaticArgmaxChunks chunks x
// (one float + one int32) = 512 KiB, which every GPU that the library runs on holds
// until the process ends.  In host code the array's name is only a stand-in; its
// device address is asked for once per device and kept.
constexpr int kStaticArgmaxMaxRows = 1024;
constexpr int kStaticArgmaxChunks = 64;
constexpr size_t kStaticArgmaxBytes = static_cast<size_t>(kStaticArgmaxMaxRows) * kStaticArgmaxChunks * 8;
static __device__ __align__(256) unsigned char scratch[kStaticArgmaxBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void* g_scratch_of_device[kMaxDevices] = {};

// The address of `scratch` on the current device (asked for at the first call on that device).
int scratch_of_current_device(void** address) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return ms_fail("argmax_rows_static: hipGetDevice: %s", hipGetErrorString(err));
  MS_REQUIRE(device >= 0 && device < kMaxDevices, "argmax_rows_static: device %d is outside 0..%d", device,
             kMaxDevices - 1);
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (g_scratch_of_device[device] == nullptr) {
    void* found = nullptr;
    err = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (err != hipSuccess || found == nullptr)
      return ms_fail("argmax_rows_static: hipGetSymbolAddress on device %d: %s", device, hipGetErrorString(err));
    g_scratch_of_device[device] = found;
  }
  *address = g_scratch_of_device[device];
  return 0;
}

}  // namespace

extern "C" int ms_argmax_rows_static(const void* logits, void* out, int rows, int vocab, hipStream_t stream) {
  MS_REQUIRE(logits != nullptr && out != nullptr, "argmax_rows_static: null operand");
  MS_REQUIRE(vocab > 0, "argmax_rows_static: a vocabulary of %d", vocab);
  MS_REQUIRE(rows > 0 && rows <= kStaticArgmaxMaxRows,
             "argmax_rows_static: %d rows are outside 1..%d (the static scratch holds no more; "
             "ms_argmax_rows takes buffers of any size)",
             rows, kStaticArgmaxMaxRows);
  void* base = nullptr;
  if (int status = scratch_of_current_device(&base)) return status;
  const int chunks = vocab < kStaticArgmaxChunks ? vocab : kStaticArgmaxChunks;
  // Stage 1 writes every one of the rows x chunks entries that stage 2 reads, so nothing
  // of an earlier call is seen and nothing needs clearing.
  float* chunk_max = static_cast<float*>(base);
  int32_t* chunk_index = reinterpret_cast<int32_t*>(static_cast<unsigned char*>(base) + kStaticArgmaxBytes / 2);
  hipLaunchKernelGGL(argmax_chunks_kernel, dim3(chunks, rows), dim3(kArgmaxThreads), 0, stream,
                     static_cast<const float*>(logits), chunk_max, chunk_index, vocab, chunks);
  MS_CHECK_LAUNCH("argmax_chunks (static)");
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(ms::kWave), 0, stream, chunk_max, chunk_index,
                     static_cast<int32_t*>(out), chunks);
  MS_CHECK_LAUNCH("argmax_rows (static)");
  return 0;
}

// ---- the same choice for a large vocabulary: a row is read by many workgroups ----------
//
// One workgroup a row reads 600 KB of logits several times at the speed of one
// compute unit.  Here the passes over the row are cut into kRowChunks chunks, a
// workgroup each: (1) finiteness, maximum and its lowest index per chunk; (2) the
// ladder's counts and masses per chunk; (3) the short list, every chunk writing its
// share at its place in token order; (4) one workgroup a row makes the choice: among
// the list, or, without top-k and top-p, inside the chunk that the running mass
// singles out, or - no rung of the ladder holds the candidates - over the whole row as above.
// The list lies in device memory and may be as long as the row; the last stage copies
// it into LDS when it is short.  Between (3) and (4), for rows with top-p alone and a long
// nucleus, the chunks search the threshold together (sample_nucleus_kernel, below) and
// nothing is gathered.  Tables between the stages (per row): chunk_max,
// chunk_arg [chunks]; ladder_count [chunks][kLadder]; ladder_mass [chunks][kLadder + 1];
// the tables of the search; list_values, list_indices [vocab].
constexpr int kRowChunks = 32;
constexpr int kChunkThreads = 256;
constexpr int kChunkWaves = kChunkThreads / ms::kWave;

// Top-p alone over a row whose nucleus is no short list (a flat row: most of the vocabulary
// stays): the threshold is searched by all chunks together, eight bits a pass.  A pass adds
// the mass of every token to the bin of its next eight bits, in integers (a token's weight
// times 2^40, rounded down), so that the sums do not depend on the order in which the
// workgroups add; the tables of the passes and what the search leaves for the choice:
constexpr int kNucleusPasses = 4;
constexpr int kNucleusBins = 256;
constexpr float kNucleusScale = 1099511627776.0f;      // 2^40
// A list of up to this many tokens is searched by the one workgroup of the choice (about
// 5 us per thousand tokens); a longer one, or none, by the chunks (some 80 us whatever the length).
constexpr int kNucleusFrom = 24576;

struct RowTables {
  float* chunk_max;
  int* chunk_arg;
  int* ladder_count;
  float* ladder_mass;
  int* nucleus_flag;                  // 1: the row's threshold is searched by the chunks together
  uint32_t* nucleus_threshold;        // the result: tokens whose ordered value reaches it stay
  float* kept_mass;                   // [chunks]: the mass of the tokens that stay
  unsigned long long* histogram;      // [kNucleusPasses][kNucleusBins]
  unsigned long long* search_state;   // [kNucleusPasses][3]: what the search knew after each pass (NucleusSearch)
  float* list_values;
  int* list_indices;
};

constexpr size_t kRowFixedFloats = static_cast<size_t>(kRowChunks) * (2 + kLadder + kLadder + 1) + 2 + kRowChunks +
                                   2 * static_cast<size_t>(kNucleusPasses) * (kNucleusBins + 3);
static_assert((kRowChunks * (2 + kLadder + kLadder + 1) + 2 + kRowChunks) % 2 == 0, "the histogram is read as 64-bit words");

__host__ __device__ inline size_t row_table_floats(int vocab) {
  return kRowFixedFloats + 2 * static_cast<size_t>(vocab);
}

__device__ __forceinline__ RowTables row_tables(float* workspace, int row, int vocab) {
  float* base = workspace + static_cast<size_t>(row) * row_table_floats(vocab);
  RowTables t;
  t.chunk_max = base;
  t.chunk_arg = reinterpret_cast<int*>(base + kRowChunks);
  t.ladder_count = reinterpret_cast<int*>(base + 2 * kRowChunks);
  t.ladder_mass = base + 2 * kRowChunks + kRowChunks * kLadder;
  float* next = base + 2 * kRowChunks + kRowChunks * (2 * kLadder + 1);
  t.nucleus_flag = reinterpret_cast<int*>(next);
  t.nucleus_threshold = reinterpret_cast<uint32_t*>(next + 1);
  t.kept_mass = next + 2;
  t.histogram = reinterpret_cast<unsigned long long*>(next + 2 + kRowChunks);
  t.search_state = t.histogram + kNucleusPasses * kNucleusBins;
  t.list_values = base + kRowFixedFloats;
  t.list_indices = reinterpret_cast<int*>(t.list_values + vocab);
  return t;
}

__device__ __forceinline__ int chunk_length(int vocab) {
  return ((vocab + kRowChunks - 1) / kRowChunks + ms::kWave - 1) / ms::kWave * ms::kWave;
}

// Which rung of the ladder makes the short list (-1: none), from the tables of stage 2;
// every caller gets the same answer.  `whole`: the mass of the whole row.
__device__ int choose_rung(const RowTables& t, bool cut_k, int k, float p, float* whole_out, int* total_out) {
  float whole = 0.f;
  for (int c = 0; c < kRowChunks; ++c) whole += t.ladder_mass[c * (kLadder + 1) + kLadder];
  *whole_out = whole;
  for (int r = 0; r < kLadder; ++r) {
    int total = 0;
    float sum = 0.f;
    for (int c = 0; c < kRowChunks; ++c) {
      total += t.ladder_count[c * kLadder + r];
      sum += t.ladder_mass[c * (kLadder + 1) + r];
    }
    // (a little more than top_p of the mass: the sums here and those of the choice differ in rounding)
    const bool enough = cut_k ? total >= k : sum > (p + 1e-4f) * whole;
    if (enough) {
      *total_out = total;
      return r;
    }
  }
  return -1;
}

__global__ __launch_bounds__(kChunkThreads) void sample_scan_kernel(const float* __restrict__ logits,
                                                                    float* __restrict__ workspace, int vocab) {
  __shared__ float f_scratch[kChunkWaves];
  __shared__ int i_scratch[kChunkWaves];
  __shared__ int shared_index;
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  const RowTables t = row_tables(workspace, row, vocab);
  const int length = chunk_length(vocab);
  const int begin = min(chunk * length, vocab), end = min(begin + length, vocab);
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  float best = -INFINITY;
  int best_index = vocab, bad = 0;
  for (int i = begin + tid; i < end; i += kChunkThreads) {
    const float v = x[i];
    if (!(fabsf(v) <= 3.402823466e38f)) bad = 1;
    if (v > best) {
      best = v;
      best_index = i;
    }
  }
  bad = ms::wave_sum_int(bad);
  if ((tid & (ms::kWave - 1)) == 0) i_scratch[tid / ms::kWave] = bad;
  if (tid == 0) shared_index = vocab;
  const float chunk_best = ms::block_max(best, f_scratch);    // has barriers: i_scratch and shared_index are visible
  if (best == chunk_best) atomicMin(&shared_index, best_index);
  __syncthreads();
  if (tid == 0) {
    int any_bad = 0;
    for (int w = 0; w < kChunkWaves; ++w) any_bad += i_scratch[w];
    t.chunk_max[chunk] = chunk_best;                 // -inf for a chunk past the row's end
    t.chunk_arg[chunk] = any_bad ? -1 : shared_index;
    if (chunk == 0) *t.nucleus_flag = 0;
  }
  // every chunk clears its share of the tables that the search of a nucleus adds into
  constexpr int kShare = kNucleusPasses * kNucleusBins / kRowChunks;
  if (tid < kShare) t.histogram[chunk * kShare + tid] = 0ull;
}

// The row's maximum and whether any chunk met a non-finite value, from stage 1's table.
__device__ __forceinline__ float row_maximum(const RowTables& t, bool* bad) {
  float row_max = -INFINITY;
  bool any_bad = false;
  for (int c = 0; c < kRowChunks; ++c) {
    row_max = fmaxf(row_max, t.chunk_max[c]);
    any_bad = any_bad || t.chunk_arg[c] < 0;
  }
  *bad = any_bad;
  return row_max;
}

__global__ __launch_bounds__(kChunkThreads) void sample_ladder_kernel(const float* __restrict__ logits,
                                                                      const float* __restrict__ temperature,
                                                                      const int32_t* __restrict__ top_k,
                                                                      float* __restrict__ workspace, int vocab) {
  __shared__ int count_s[kChunkWaves][kLadder];
  __shared__ float mass_s[kChunkWaves][kLadder + 1];
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & (ms::kWave - 1), wave = tid / ms::kWave;
  const RowTables t = row_tables(workspace, row, vocab);
  const float temp = temperature[row];
  bool bad;
  const float row_max = row_maximum(t, &bad);
  if (bad || temp == 0.f) return;
  const int k = top_k ? top_k[row] : 0;
  const bool cut_k = k > 0 && k < vocab;
  const float scaled_max = row_max / temp;
  const int length = chunk_length(vocab);
  const int begin = min(chunk * length, vocab), end = min(begin + length, vocab);
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  int count[kLadder];
  float mass[kLadder + 1];
#pragma unroll
  for (int c = 0; c < kLadder; ++c) count[c] = 0, mass[c] = 0.f;
  mass[kLadder] = 0.f;
  for (int i = begin + tid; i < end; i += kChunkThreads) {
    const float v = x[i] / temp;
    const float depth = scaled_max - v;
    const float weight = cut_k ? 0.f : expf(v - scaled_max);
    mass[kLadder] += weight;
#pragma unroll
    for (int c = 0; c < kLadder; ++c) {
      const bool in = depth <= kLadderDepth[c];
      count[c] += in;
      mass[c] += in ? weight : 0.f;
    }
  }
#pragma unroll
  for (int c = 0; c < kLadder; ++c) {
    const int total = ms::wave_sum_int(count[c]);
    const float sum = ms::wave_sum(mass[c]);
    if (lane == 0) count_s[wave][c] = total, mass_s[wave][c] = sum;
  }
  {
    const float sum = ms::wave_sum(mass[kLadder]);
    if (lane == 0) mass_s[wave][kLadder] = sum;
  }
  __syncthreads();
  if (tid <= kLadder) {
    float sum = 0.f;
    for (int w = 0; w < kChunkWaves; ++w) sum += mass_s[w][tid];
    t.ladder_mass[chunk * (kLadder + 1) + tid] = sum;
    if (tid < kLadder) {
      int total = 0;
      for (int w = 0; w < kChunkWaves; ++w) total += count_s[w][tid];
      t.ladder_count[chunk * kLadder + tid] = total;
    }
  }
}

__global__ __launch_bounds__(kChunkThreads) void sample_gather_kernel(const float* __restrict__ logits,
                                                                      const float* __restrict__ temperature,
                                                                      const int32_t* __restrict__ top_k,
                                                                      const float* __restrict__ top_p,
                                                                      float* __restrict__ workspace, int vocab,
                                                                      int search_nucleus) {
  __shared__ int rung_s, base_s;
  __shared__ int wave_count[kChunkWaves];
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & (ms::kWave - 1), wave = tid / ms::kWave;
  const RowTables t = row_tables(workspace, row, vocab);
  const float temp = temperature[row];
  bool bad;
  const float row_max = row_maximum(t, &bad);
  if (bad || temp == 0.f) return;
  const int k = top_k ? top_k[row] : 0;
  const float p = top_p ? top_p[row] : 1.f;
  const bool cut_k = k > 0 && k < vocab;
  if (!cut_k && !(p < 1.f)) return;
  if (tid == 0) {
    float whole;
    int total = 0;
    const int rung = choose_rung(t, cut_k, k, p, &whole, &total);
    int base = 0;
    if (rung >= 0)
      for (int c = 0; c < chunk; ++c) base += t.ladder_count[c * kLadder + rung];
    // top-p alone and no short list: the chunks search the threshold together (the kernels
    // after this one), nothing is gathered
    const bool together = search_nucleus && !cut_k && (rung < 0 || total > kNucleusFrom);
    if (together && chunk == 0) *t.nucleus_flag = 1;
    rung_s = together ? -1 : rung;
    base_s = base;
  }
  __syncthreads();
  const int rung = rung_s;
  if (rung < 0) return;
  float deepest = 0.f;
#pragma unroll
  for (int c = 0; c < kLadder; ++c)
    if (c == rung) deepest = kLadderDepth[c];
  const float scaled_max = row_max / temp;
  const int length = chunk_length(vocab);
  const int begin = min(chunk * length, vocab), end = min(begin + length, vocab);
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  int written = base_s;
  // 256 consecutive tokens a round; a token's place: what was written before, the
  // tokens of the waves before its own in this round, those of the lanes before it
  for (int first = begin; first < end; first += kChunkThreads) {
    const int i = first + tid;
    float v = 0.f;
    bool in = false;
    if (i < end) {
      v = x[i] / temp;
      in = scaled_max - v <= deepest;
    }
    const unsigned long long mask = __ballot(in);
    __syncthreads();                         // the last round's counts are read
    if (lane == 0) wave_count[wave] = __popcll(mask);
    __syncthreads();
    int before = 0, round_total = 0;
    for (int w = 0; w < kChunkWaves; ++w) {
      before += w < wave ? wave_count[w] : 0;
      round_total += wave_count[w];
    }
    if (in) {
      const int place = written + before + __popcll(mask & ((1ull << lane) - 1ull));
      if (place < vocab) {                  // (it is: the places are the ranks of tokens of the row)
        t.list_values[place] = v;
        t.list_indices[place] = i;
      }
    }
    written += round_total;
  }
}

// What the search knows after some of its passes: the bits of the threshold found so far,
// the mass of the tokens that lie above every value with those bits, and the mass that the
// kept tokens must exceed.
struct NucleusSearch {
  uint32_t prefix;
  unsigned long long above;
  unsigned long long limit;
};

// Inclusive sum over this lane and the higher lanes of the wave.
__device__ __forceinline__ unsigned long long wave_sum_from_here_up(unsigned long long v) {
  const int lane = threadIdx.x & (ms::kWave - 1);
#pragma unroll
  for (int step = 1; step < ms::kWave; step <<= 1) {
    const unsigned low = __shfl_down(static_cast<unsigned>(v), step, ms::kWave);
    const unsigned high = __shfl_down(static_cast<unsigned>(v >> 32), step, ms::kWave);
    if (lane + step < ms::kWave) v += (static_cast<unsigned long long>(high) << 32) | low;
  }
  return v;
}

// The state after pass `pass`, from the state before it (kept in the row's tables by the
// kernel before this one; nothing before pass 0) and the pass's histogram.  All 256 threads
// of the workgroup call it, a thread a bin, and get the same answer; chunk 0 keeps it for
// the next kernel.
__device__ NucleusSearch nucleus_search_after(const RowTables& t, int pass, float p, bool keep_it,
                                              unsigned long long* group_s, unsigned long long* word_s, int* digit_s) {
  const int tid = threadIdx.x;
  NucleusSearch state{0u, 0ull, 0ull};
  if (pass > 0) {
    state.prefix = static_cast<uint32_t>(t.search_state[3 * (pass - 1)]);
    state.above = t.search_state[3 * (pass - 1) + 1];
    state.limit = t.search_state[3 * (pass - 1) + 2];
  }
  const unsigned long long bin = t.histogram[pass * kNucleusBins + tid];
  unsigned long long reached = wave_sum_from_here_up(bin);      // this bin and the higher ones of its wave
  if ((tid & (ms::kWave - 1)) == 0) group_s[tid / ms::kWave] = reached;
  if (tid == 0) *digit_s = 0;
  __syncthreads();
  for (int g = tid / ms::kWave + 1; g < kChunkWaves; ++g) reached += group_s[g];
  reached += state.above;
  if (pass == 0) {
    if (tid == 0) *word_s = reached;                 // the whole row's mass
    __syncthreads();
    state.limit = static_cast<unsigned long long>(static_cast<double>(p) * static_cast<double>(*word_s));
    __syncthreads();
  }
  // the threshold's next eight bits: the highest bin from which on the mass still exceeds the limit
  if (reached > state.limit) atomicMax(digit_s, tid);
  __syncthreads();
  const int digit = *digit_s;
  if (tid == digit) *word_s = reached - bin;
  __syncthreads();
  state.above = *word_s;
  state.prefix |= static_cast<uint32_t>(digit) << (24 - 8 * pass);
  if (keep_it && tid == 0) {
    t.search_state[3 * pass] = state.prefix;
    t.search_state[3 * pass + 1] = state.above;
    t.search_state[3 * pass + 2] = state.limit;
  }
  __syncthreads();
  return state;
}

// One pass of the search (pass 0 .. kNucleusPasses - 1), or (pass == kNucleusPasses) what
// the choice needs of its result: the threshold and every chunk's mass of kept tokens.
__global__ __launch_bounds__(kChunkThreads) void sample_nucleus_kernel(const float* __restrict__ logits,
                                                                       const float* __restrict__ temperature,
                                                                       const float* __restrict__ top_p,
                                                                       float* __restrict__ workspace, int vocab,
                                                                       int pass) {
  static_assert(kChunkThreads == kNucleusBins, "a thread a bin");
  __shared__ unsigned long long mine_s[kNucleusBins];
  __shared__ unsigned long long group_s[kChunkWaves];
  __shared__ unsigned long long word_s;
  __shared__ int digit_s;
  __shared__ float mass_s[kChunkWaves];
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  const RowTables t = row_tables(workspace, row, vocab);
  if (*t.nucleus_flag == 0) return;
  const float temp = temperature[row];
  const float p = top_p[row];
  bool bad;
  const float scaled_max = row_maximum(t, &bad) / temp;
  // (kernel `pass` works out what pass - 1 found; the first has nothing to work out)
  NucleusSearch found{0u, 0ull, 0ull};
  if (pass > 0) found = nucleus_search_after(t, pass - 1, p, chunk == 0, group_s, &word_s, &digit_s);
  const int length = chunk_length(vocab);
  const int begin = min(chunk * length, vocab), end = min(begin + length, vocab);
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  if (pass < kNucleusPasses) {
    const int shift = 24 - 8 * pass;
    mine_s[tid] = 0ull;
    __syncthreads();
    for (int i = begin + tid; i < end; i += kChunkThreads) {
      const float v = x[i] / temp;
      const uint32_t o = ordered(v);
      // (in pass 0 every token has the bits above the pass's: there are none)
      if (pass == 0 || ((o ^ found.prefix) >> (shift + 8)) == 0u) {
        const unsigned long long weight = static_cast<unsigned long long>(expf(v - scaled_max) * kNucleusScale);
        if (weight != 0ull) atomicAdd(&mine_s[(o >> shift) & 255u], weight);
      }
    }
    __syncthreads();
    if (mine_s[tid] != 0ull) atomicAdd(&t.histogram[pass * kNucleusBins + tid], mine_s[tid]);
    return;
  }
  // the search is over: found.prefix is the threshold
  float mass = 0.f;
  for (int i = begin + tid; i < end; i += kChunkThreads) {
    const float v = x[i] / temp;
    if (ordered(v) >= found.prefix) mass += expf(v - scaled_max);
  }
  mass = ms::wave_sum(mass);
  if ((tid & (ms::kWave - 1)) == 0) mass_s[tid / ms::kWave] = mass;
  __syncthreads();
  if (tid == 0) {
    float sum = 0.f;
    for (int w = 0; w < kChunkWaves; ++w) sum += mass_s[w];
    t.kept_mass[chunk] = sum;
    if (chunk == 0) *t.nucleus_threshold = found.prefix;
  }
}

// The view of one chunk of a row, for the draw without top-k and top-p.
struct ChunkView {
  static constexpr bool kInDeviceMemory = true;
  const float* x;
  float temp;
  int begin;
  int size;
  __device__ __forceinline__ float value(int i) const { return x[begin + i] / temp; }
  __device__ __forceinline__ int index(int i) const { return begin + i; }
};

__global__ __launch_bounds__(kThreads) void sample_choose_kernel(const float* __restrict__ logits,
                                                                 const float* __restrict__ temperature,
                                                                 const int32_t* __restrict__ top_k,
                                                                 const float* __restrict__ top_p,
                                                                 const float* __restrict__ uniform,
                                                                 float* __restrict__ workspace,
                                                                 int32_t* __restrict__ out, int vocab) {
  __shared__ float f_scratch[kWaves];
  __shared__ int i_scratch[kWaves];
  __shared__ float seg_sum[kThreads];
  __shared__ int seg_count[kThreads];
  __shared__ int shared_index;
  __shared__ float shared_total;
  __shared__ int digit_count[kWaves][kDigits];
  __shared__ float digit_mass[kWaves][kDigits];
  __shared__ int rung_s, total_s, chunk_s;
  __shared__ float whole_s, before_s;
  __shared__ float list_values[kListCap];
  __shared__ int list_indices[kListCap];

  const int row = blockIdx.x, tid = threadIdx.x;
  const RowTables t = row_tables(workspace, row, vocab);
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  const float temp = temperature[row];
  Scratch sc;        // member by member: as one constant aggregate of LDS addresses the compiler cannot emit it
  sc.f_scratch = f_scratch;
  sc.i_scratch = i_scratch;
  sc.seg_sum = seg_sum;
  sc.seg_count = seg_count;
  sc.shared_index = &shared_index;
  sc.shared_total = &shared_total;
  sc.digit_count = digit_count;
  sc.digit_mass = digit_mass;
  bool bad;
  const float row_max = row_maximum(t, &bad);
  if (bad) {
    if (tid == 0) out[row] = -1;
    return;
  }
  if (temp == 0.f) {
    // the first chunk that holds the maximum has its lowest index
    if (tid == 0) {
      int index = vocab;
      for (int c = kRowChunks - 1; c >= 0; --c)
        if (t.chunk_max[c] == row_max) index = t.chunk_arg[c];
      out[row] = index;
    }
    return;
  }
  const float scaled_max = row_max / temp;
  const int k = top_k ? top_k[row] : 0;
  const float p = top_p ? top_p[row] : 1.f;
  const bool cut_k = k > 0 && k < vocab;
  const bool cut_p = p < 1.f;
  const float u = uniform[row];

  if (cut_p && !cut_k && *t.nucleus_flag != 0) {
    // The chunks have searched the threshold together and left every chunk's mass of kept
    // tokens: the chunk in which the running mass passes uniform * the kept mass is found
    // from those, and the draw is made inside it, among its kept tokens.
    if (tid == 0) {
      float kept = 0.f;
      for (int c = 0; c < kRowChunks; ++c) kept += t.kept_mass[c];
      const float target = u * kept;
      float running = 0.f, before = 0.f;
      int chunk = -1, last_live = 0;
      for (int c = 0; c < kRowChunks; ++c) {
        const float mass = t.kept_mass[c];
        if (mass > 0.f) last_live = c;
        if (chunk < 0 && running + mass > target) {
          chunk = c;
          before = running;
        }
        running += mass;
      }
      if (chunk < 0) {                          // rounding: the target lies at the very end
        chunk = last_live;
        before = -INFINITY;                     // nothing in the chunk passes the target: its last kept token is taken
      }
      chunk_s = chunk;
      before_s = before;
      whole_s = kept;
    }
    __syncthreads();
    const int length = chunk_length(vocab);
    const int begin = min(chunk_s * length, vocab), end = min(begin + length, vocab);
    const ChunkView part{x, temp, begin, end - begin};
    const uint32_t threshold = *t.nucleus_threshold;
    const int chosen = choose(part, vocab, scaled_max, 0, 1.f, u, whole_s, before_s, sc, &threshold);
    if (tid == 0) out[row] = chosen;
    return;
  }
  if (cut_k || cut_p) {
    if (tid == 0) {
      float whole;
      int total = 0;
      rung_s = choose_rung(t, cut_k, k, p, &whole, &total);
      whole_s = whole;
      total_s = total;
    }
    __syncthreads();
    if (rung_s >= 0) {
      const int n = total_s;
      int chosen;
      if (n <= kListCap) {
        for (int i = tid; i < n; i += kThreads) {
          list_values[i] = t.list_values[i];
          list_indices[i] = t.list_indices[i];
        }
        __syncthreads();
        const ListView list{list_values, list_indices, n};
        chosen = choose(list, vocab, scaled_max, cut_k ? k : 0, p, u, cut_k ? -1.f : whole_s, 0.f, sc);
      } else {
        const LongListView list{t.list_values, t.list_indices, n};      // a long list stays where it is
        chosen = choose(list, vocab, scaled_max, cut_k ? k : 0, p, u, cut_k ? -1.f : whole_s, 0.f, sc);
      }
      if (tid == 0) out[row] = chosen;
      return;
    }
    const RowView whole{x, temp, vocab};
    const int chosen = choose(whole, vocab, scaled_max, cut_k ? k : 0, p, u, -1.f, 0.f, sc);
    if (tid == 0) out[row] = chosen;
    return;
  }

  // Neither top-k nor top-p: the chunk in which the running mass passes uniform * whole
  // is found from the chunks' masses, and the draw is made inside it.
  if (tid == 0) {
    float whole = 0.f;
    for (int c = 0; c < kRowChunks; ++c) whole += t.ladder_mass[c * (kLadder + 1) + kLadder];
    const float target = u * whole;
    float running = 0.f;
    int chunk = -1;
    float before = 0.f;
    int last_live = 0;
    for (int c = 0; c < kRowChunks; ++c) {
      const float mass = t.ladder_mass[c * (kLadder + 1) + kLadder];
      if (mass > 0.f) last_live = c;
      if (chunk < 0 && running + mass > target) {
        chunk = c;
        before = running;
      }
      running += mass;
    }
    if (chunk < 0) {                          // rounding: the target lies at the very end
      chunk = last_live;
      before = -INFINITY;                     // nothing in the chunk passes the target: its last token is taken
    }
    chunk_s = chunk;
    before_s = before;
    whole_s = whole;
  }
  __syncthreads();
  const int length = chunk_length(vocab);
  const int begin = min(chunk_s * length, vocab), end = min(begin + length, vocab);
  const ChunkView part{x, temp, begin, end - begin};
  const int chosen = choose(part, vocab, scaled_max, 0, 1.f, u, whole_s, before_s, sc);
  if (tid == 0) out[row] = chosen;
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

// Bytes of the workspace that ms_sample_rows_chunked needs for `rows` rows of `vocab` tokens.
extern "C" size_t ms_sample_rows_workspace_bytes(int rows, int vocab) {
  return static_cast<size_t>(rows > 0 ? rows : 0) * row_table_floats(vocab > 0 ? vocab : 0) * sizeof(float);
}

// The same choice as ms_sample_rows for a large vocabulary, the passes over a row
// shared by 32 workgroups; temperature is not null.  workspace: device memory of
// ms_sample_rows_workspace_bytes(rows, vocab), aligned to 8 bytes, the caller's until the
// call's work on the stream is done.  search_nucleus: not 0 if some row may have top-p
// without top-k (then the kernels that search such a row's threshold with all chunks are
// launched; a row decides for itself whether it needs them); 0 spares their launches.
extern "C" int ms_sample_rows_chunked(const void* logits, const void* temperature, const void* top_k,
                                      const void* top_p, const void* uniform, void* out, void* workspace,
                                      size_t workspace_bytes, int rows, int vocab, int search_nucleus,
                                      hipStream_t stream) {
  MS_REQUIRE(rows > 0 && rows <= 65535 && vocab > 0, "sample_rows_chunked: bad shape %d x %d", rows, vocab);
  MS_REQUIRE(temperature && uniform, "sample_rows_chunked: temperature and uniform numbers are needed");
  MS_REQUIRE(workspace && workspace_bytes >= ms_sample_rows_workspace_bytes(rows, vocab),
             "sample_rows_chunked: the workspace has %zu bytes, %zu are needed", workspace_bytes,
             ms_sample_rows_workspace_bytes(rows, vocab));
  MS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7u) == 0, "sample_rows_chunked: the workspace is not aligned to 8 bytes");
  float* tables = static_cast<float*>(workspace);
  const dim3 grid(kRowChunks, rows);
  const int together = search_nucleus != 0 && top_p != nullptr;
  hipLaunchKernelGGL(sample_scan_kernel, grid, dim3(kChunkThreads), 0, stream, static_cast<const float*>(logits),
                     tables, vocab);
  MS_CHECK_LAUNCH("sample_scan");
  hipLaunchKernelGGL(sample_ladder_kernel, grid, dim3(kChunkThreads), 0, stream, static_cast<const float*>(logits),
                     static_cast<const float*>(temperature), static_cast<const int32_t*>(top_k), tables, vocab);
  MS_CHECK_LAUNCH("sample_ladder");
  hipLaunchKernelGGL(sample_gather_kernel, grid, dim3(kChunkThreads), 0, stream, static_cast<const float*>(logits),
                     static_cast<const float*>(temperature), static_cast<const int32_t*>(top_k),
                     static_cast<const float*>(top_p), tables, vocab, together);
  MS_CHECK_LAUNCH("sample_gather");
  if (together) {
    for (int pass = 0; pass <= kNucleusPasses; ++pass) {
      hipLaunchKernelGGL(sample_nucleus_kernel, grid, dim3(kChunkThreads), 0, stream, static_cast<const float*>(logits),
                         static_cast<const float*>(temperature), static_cast<const float*>(top_p), tables, vocab, pass);
      MS_CHECK_LAUNCH("sample_nucleus");
    }
  }
  hipLaunchKernelGGL(sample_choose_kernel, dim3(rows), dim3(kThreads), 0, stream, static_cast<const float*>(logits),
                     static_cast<const float*>(temperature), static_cast<const int32_t*>(top_k),
                     static_cast<const float*>(top_p), static_cast<const float*>(uniform), tables,
                     static_cast<int32_t*>(out), vocab);
  MS_CHECK_LAUNCH("sample_choose");
  return 0;
}
