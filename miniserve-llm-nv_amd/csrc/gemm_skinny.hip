// Matrix product for few rows (decoding): out[M, N] = x[M, K] . W[N, K]^T with
// M <= 64, bfloat16 inputs, 32-bit accumulation on the matrix cores.  The weight
// matrix is streamed exactly once at 16 bytes a lane; the step is bound by that
// stream, so the kernel is built around keeping many loads in flight.
//
//   C^T[n, m] += W[n, k] x[m, k]        A = W tile (16 rows x 32 k), B = x^T
//
// A workgroup of 8 waves owns RB blocks of 16 rows of W; the waves split K between
// them in steps of 32 (wave w takes steps w, w + 8, ...), so that one round of the
// workgroup reads 512 contiguous bytes of every row.  The waves' partial tiles are
// summed through LDS in a fixed order; every output element is written by one
// workgroup: results do not depend on anything but their own row of x and of W.
//
// With more than 16 rows of x and a matrix of few rows the launch is cut along M as well
// (blockIdx.y): a workgroup takes 16 rows of x against its rows of W, so that what it
// reads of x (from the caches) stays near what it streams of W; the workgroups that
// share rows of W stand 'gridDim.x' apart in the launch order, which puts them on the
// same die and lets all but the first find those rows in its cache.
//
// Epilogues (what the reference does in separate torch calls):
//   0  out = bf16(C)                                   nn.Linear (qwen3.py:174-176)
//   1  out_f32 = C                                     logits (qwen3.py:558)
//   2  out_f32 += C                                    residual add (qwen3.py:367-368, 381-382)
//   3  out = bf16(silu(C[gate row]) * C[up row])       gated activation (layers.py:86-87);
//      the workgroup owns row n of the gate half and row n + N/2 of the up half
//   4  as 2, and the RMSNorm that follows the residual add is prepared: beside the new
//      residual value v the workgroup stores bf16(w_norm[n] * v), the operand of the product
//      behind that norm, and the sum of v^2 over its own columns for every row, into a slot
//      of its own (no atomics: the sums have a fixed order).  The product behind the norm
//      (ms_gemm_skinny_scaled) adds the workgroups' sums in their order, and
//      scales its own sums by 1 / rms: the norm is no kernel and no prologue of its own.
#include "mfma.hpp"

namespace {

using ms::bf16;
using ms::bf16x8;
using ms::floatx4;

constexpr int kWavesPerGroup = 8;
constexpr int kGroupThreads = kWavesPerGroup * ms::kWave;

enum Epilogue : int { kStoreBf16 = 0, kStoreF32 = 1, kAddF32 = 2, kSiluMul = 3, kAddF32Ahead = 4 };

// What the epilogue 4 leaves for the product behind the norm, and what that product reads.
struct NormAhead {
  const bf16* weight;   // of the norm, [n of the producer]
  bf16* x;              // [m, n]: bf16(weight * residual)
  float* squares;       // [groups, m]: every producer workgroup's sum of squares of its columns
  int groups;           // of the producer (its gridDim.x); for the consumer: how many to add
  float eps;
};
// rows of W from which two blocks of 10 rows and more a workgroup still make 256 workgroups
constexpr int kTwoBlockRows = 5120;

// NORM: x is not given; the product is taken of the RMSNorm of the 32-bit residual
// stream h, with the normalisation moved behind the sum so that nothing waits for
// the row statistics:
//   out[m, n] = rsqrt(mean(h[m, :]^2) + eps) * sum_k W[n, k] * bf16(w_norm[k] * h[m, k])
// The squares are summed by the same loop that makes the operands; every workgroup
// sums them in the same fixed order.  (The separate norm kernel rounds the
// normalised value before the multiply by the weight, as the reference does; here
// the one rounding is of w_norm * h.  Both carry 8 significant bits.)
// UNROLL: k-steps whose loads are issued together (more for long rows: more bytes in flight)
template <int MB, int RB, bool NORM, int UNROLL, bool SCALED>
__global__ __launch_bounds__(kGroupThreads) void gemm_skinny_kernel(const bf16* __restrict__ x,
                                                                    const float* __restrict__ h,
                                                                    const bf16* __restrict__ norm_weight, float eps,
                                                                    const bf16* __restrict__ w, bf16* out_bf16,
                                                                    float* out_f32, int m, int n, int k,
                                                                    int epilogue, int rows, NormAhead ahead) {
  // ahead: epilogue 4 writes it.  SCALED: x is the `ahead.x` of a product before; the sums are
  // scaled by 1 / sqrt(mean of squares + eps), the squares taken from ahead.squares.
  // rows: how many of the 16 rows of a block are this workgroup's (16, or 8 or 4 for a
  // matrix of few rows, so that there are workgroups enough to fill the chip)
  __shared__ float c_s[kWavesPerGroup][RB * MB][16][16];
  __shared__ float square_s[kWavesPerGroup][16];
  __shared__ float tile_square_s[RB * MB][16];      // epilogue 4: a tile's sum of squares a row
  __shared__ float inv_rms_s[MB * 16];              // SCALED: 1 / rms of the workgroup's rows of x

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int g = lane >> 4;
  const int r = lane & 15;

  // Rows of W of this workgroup: block rb starts at row_start[rb].
  const int half = n / 2;
  int row_start[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    if (epilogue == kSiluMul) {
      // RB is even: blocks 0..RB/2-1 are gate rows, the others the matching up rows
      const int pair = rb % (RB / 2 > 0 ? RB / 2 : 1);
      row_start[rb] = (blockIdx.x * (RB / 2 > 0 ? RB / 2 : 1) + pair) * rows + (rb >= RB / 2 ? half : 0);
    } else {
      row_start[rb] = (blockIdx.x * RB + rb) * rows;
    }
  }
  const int row_limit = epilogue == kSiluMul ? half : n;   // rows of one half for the gated form

  const bf16* w_row[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    // a row past the end is read from the last row and never stored
    int local = row_start[rb] - (epilogue == kSiluMul && rb >= RB / 2 ? half : 0) + r;
    local = min(local, row_limit - 1);
    const int row = local + (epilogue == kSiluMul && rb >= RB / 2 ? half : 0);
    w_row[rb] = w + static_cast<int64_t>(row) * k;
  }
  const int m_base = blockIdx.y * (16 * MB);      // the workgroup's first row of x
  const bf16* x_row[MB];
  bool x_live[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int row = m_base + 16 * mb + r;
    x_live[mb] = row < m;
    x_row[mb] = NORM ? nullptr : x + static_cast<int64_t>(min(row, m - 1)) * k;
  }

  floatx4 acc[RB][MB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = floatx4{0.f, 0.f, 0.f, 0.f};

  // The += epilogue reads the output before it adds: the first value that this thread
  // will add to is asked for now, so that it has arrived when the sums are made (no
  // other thread writes it).
  float residual_ahead = 0.f;
  const bool adds = epilogue == kAddF32 || epilogue == kAddF32Ahead;
  if (adds && threadIdx.x < RB * MB * 256) {
    const int n_local = threadIdx.x & 15, m_local = (threadIdx.x >> 4) & 15, tile = threadIdx.x >> 8;
    const int rb = tile / MB, mb = tile - rb * MB;
    const int row_m = m_base + 16 * mb + m_local, col_n = row_start[rb] + n_local;
    if (row_m < m && col_n < row_limit && n_local < rows) residual_ahead = out_f32[static_cast<int64_t>(row_m) * n + col_n];
  }

  // NORM: this lane makes column m = r of x from row r of h, and sums its squares
  const float* h_row = NORM ? h + static_cast<int64_t>(min(r, m - 1)) * k : nullptr;
  float square_sum = 0.f;

  // SCALED: the threads are dealt to the workgroup's rows of x (32, 16 or 8 to a row); each
  // asks now, ahead of the walk along K, for its share of the producer workgroups' sums of
  // that row's squares (the loads go out before the first of W and have arrived when those
  // have), and adds them up after the walk in their order, with what more there may be.
  constexpr int kStatThreads = kGroupThreads / (16 * MB);
  constexpr int kStatAhead = 8;
  float group_square[kStatAhead];
  const int stat_row = threadIdx.x / kStatThreads, stat_part = threadIdx.x % kStatThreads;
  const bool stat_live = SCALED && m_base + stat_row < m;
  const float* stat_from = ahead.squares + m_base + stat_row;
  if (SCALED) {
#pragma unroll
    for (int j = 0; j < kStatAhead; ++j) {
      const int group = stat_part + kStatThreads * j;
      group_square[j] = (stat_live && group < ahead.groups) ? stat_from[static_cast<int64_t>(group) * m] : 0.f;
    }
  }

  const int steps = (k + 31) / 32;
  for (int base = wave; base < steps; base += kWavesPerGroup * UNROLL) {
    bf16x8 a[UNROLL][RB], b[UNROLL][MB];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k0 = 32 * (base + u * kWavesPerGroup) + 8 * g;
      const bool live = k0 < k;      // k is a multiple of 8
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) a[u][rb] = (live && r < rows) ? ms::load_bf16x8(w_row[rb] + k0) : ms::zero_bf16x8();
      if (NORM) {
        // Loads without a branch around them (a slice past the end reads the row's last
        // one and counts for nothing): behind a branch each would be waited for in
        // turn, and the step would cost as many round trips as it has slices.
        const int k_read = live ? k0 : k - 8;
        const float4 lo = *reinterpret_cast<const float4*>(h_row + k_read);
        const float4 hi = *reinterpret_cast<const float4*>(h_row + k_read + 4);
        const bf16x8 nw = ms::load_bf16x8(norm_weight + k_read);
        const bool keep = live && x_live[0];
        const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        bf16x8 made;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float value = keep ? v[i] : 0.f;
          square_sum = fmaf(value, value, square_sum);
          made[i] = static_cast<__bf16>(static_cast<float>(nw[i]) * value);
        }
        b[u][0] = made;
      } else {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          b[u][mb] = (live && x_live[mb]) ? ms::load_bf16x8(x_row[mb] + k0) : ms::zero_bf16x8();
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = ms::mfma_16x16x32(a[u][rb], b[u][mb], acc[rb][mb]);
  }

  // this lane: column m = 16 mb + r, rows 4 g + e of block rb
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int e = 0; e < 4; ++e) c_s[wave][rb * MB + mb][r][4 * g + e] = acc[rb][mb][e];
  if (NORM) {
    square_sum += __shfl_xor(square_sum, 16, ms::kWave);
    square_sum += __shfl_xor(square_sum, 32, ms::kWave);
    if (g == 0) square_s[wave][r] = square_sum;
  }
  if (SCALED) {
    float total = 0.f;
#pragma unroll
    for (int j = 0; j < kStatAhead; ++j) total += group_square[j];
    if (stat_live)
      for (int group = stat_part + kStatThreads * kStatAhead; group < ahead.groups; group += kStatThreads)
        total += stat_from[static_cast<int64_t>(group) * m];
#pragma unroll
    for (int step = 1; step < kStatThreads; step *= 2) total += __shfl_xor(total, step, ms::kWave);
    if (stat_part == 0) inv_rms_s[stat_row] = 1.0f / sqrtf(total / static_cast<float>(k) + ahead.eps);
  }
  __syncthreads();

  // c_s[wave][tile][m_local][n_local]; consecutive threads take consecutive n
  constexpr int kOutBlocks = RB;     // for the gated form half of them are outputs
  const int out_blocks = epilogue == kSiluMul ? RB / 2 : kOutBlocks;
  for (int index = threadIdx.x; index < out_blocks * MB * 256; index += kGroupThreads) {
    const int n_local = index & 15;
    const int m_local = (index >> 4) & 15;
    const int tile = index >> 8;
    const int rb = tile / MB, mb = tile - rb * MB;
    const int row_m = m_base + 16 * mb + m_local;
    const int col_n = row_start[rb] + n_local;
    const bool live = row_m < m && col_n < row_limit && n_local < rows;
    if (epilogue != kAddF32Ahead && !live) continue;      // (epilogue 4: every lane of a row's sixteen takes part in its sum)
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < kWavesPerGroup; ++wv) sum += c_s[wv][tile][m_local][n_local];
    float inv_rms = 1.f;
    if (NORM) {
      float squares = 0.f;
#pragma unroll
      for (int wv = 0; wv < kWavesPerGroup; ++wv) squares += square_s[wv][m_local];
      inv_rms = 1.0f / sqrtf(squares / static_cast<float>(k) + eps);
      sum *= inv_rms;
    } else if (SCALED) {
      inv_rms = inv_rms_s[16 * mb + m_local];
      sum *= inv_rms;
    }
    if (epilogue == kStoreBf16) {
      out_bf16[static_cast<int64_t>(row_m) * n + col_n] = ms::from_float<bf16>(sum);
    } else if (epilogue == kStoreF32) {
      out_f32[static_cast<int64_t>(row_m) * n + col_n] = sum;
    } else if (epilogue == kAddF32) {
      float* place = out_f32 + static_cast<int64_t>(row_m) * n + col_n;
      *place = (index == static_cast<int>(threadIdx.x) ? residual_ahead : *place) + sum;
    } else if (epilogue == kAddF32Ahead) {
      float square = 0.f;
      if (live) {
        const int64_t at = static_cast<int64_t>(row_m) * n + col_n;
        const float value = (index == static_cast<int>(threadIdx.x) ? residual_ahead : out_f32[at]) + sum;
        out_f32[at] = value;
        ahead.x[at] = ms::from_float<bf16>(ms::to_float(ahead.weight[col_n]) * value);
        square = value * value;
      }
      // the sixteen columns of the tile's row: a fixed tree over the lanes
      square += __shfl_xor(square, 1, ms::kWave);
      square += __shfl_xor(square, 2, ms::kWave);
      square += __shfl_xor(square, 4, ms::kWave);
      square += __shfl_xor(square, 8, ms::kWave);
      if (n_local == 0) tile_square_s[tile][m_local] = square;
    } else {
      float up = 0.f;
#pragma unroll
      for (int wv = 0; wv < kWavesPerGroup; ++wv) up += c_s[wv][(rb + RB / 2) * MB + mb][m_local][n_local];
      up *= inv_rms;
      const float gate = ms::round_to<bf16>(sum);
      up = ms::round_to<bf16>(up);
      out_bf16[static_cast<int64_t>(row_m) * half + col_n] = ms::from_float<bf16>(gate / (1.0f + __expf(-gate)) * up);
    }
  }
  if (epilogue == kAddF32Ahead) {
    // this workgroup's share of every row's squares: its tiles of that row, in their order
    __syncthreads();
    if (threadIdx.x < MB * 16) {
      const int mb = threadIdx.x >> 4, m_local = threadIdx.x & 15;
      const int row_m = m_base + 16 * mb + m_local;
      float total = 0.f;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) total += tile_square_s[rb * MB + mb][m_local];
      if (row_m < m) ahead.squares[static_cast<int64_t>(blockIdx.x) * m + row_m] = total;
    }
  }
}

// How a product is cut into workgroups: `rows` of the 16 rows of a block to a workgroup (see
// launch()), `groups` workgroups along N, `m_tiles` along M.
struct Cut {
  int rows, groups, m_tiles;
};

Cut cut_of(int mb_t, int rb_t, int m, int n, int epilogue) {
  const int out_rows = epilogue == kSiluMul ? n / 2 : n;
  const int blocks_per_group = epilogue == kSiluMul ? rb_t / 2 : rb_t;
  Cut cut;
  cut.m_tiles = (m + 16 * mb_t - 1) / (16 * mb_t);
  // How many of the 16 rows of a block a workgroup takes.  The chip has `units` compute
  // units (256 on MI355X); the launch lasts as long as the unit with the most to stream, that is
  // ceil(workgroups / units) times a workgroup's rows: 6144 rows in blocks of 16 are 384
  // workgroups, two for half of the units and one for the others; in blocks of 12 they are
  // 512, two for each, and a quarter less to stream for the busiest.  Fewest rows on the
  // busiest unit wins, more rows a workgroup among equals (fewer workgroups, less of x read).
  cut.rows = 16;
  const int64_t units = ms_compute_units();
  if (rb_t <= 2) {
    int64_t best = INT64_MAX;
    for (int candidate = 16; candidate >= 4; --candidate) {
      const int64_t workgroups =
          static_cast<int64_t>((out_rows + candidate * blocks_per_group - 1) / (candidate * blocks_per_group)) * cut.m_tiles;
      const int64_t busiest = ((workgroups + units - 1) / units) * candidate;
      if (busiest < best) {
        best = busiest;
        cut.rows = candidate;
      }
    }
  }
  cut.groups = (out_rows + cut.rows * blocks_per_group - 1) / (cut.rows * blocks_per_group);
  return cut;
}

template <int MB, int RB, bool NORM = false, bool SCALED = false>
void launch(const void* x, const void* w, void* out_bf16, void* out_f32, int m, int n, int k, int epilogue,
            hipStream_t stream, const void* h = nullptr, const void* norm_weight = nullptr, float eps = 0.f,
            NormAhead ahead = NormAhead{nullptr, nullptr, nullptr, 0, 0.f}) {
  const Cut cut = cut_of(MB, RB, m, n, epilogue);
  // rows of 2048 elements and more: eight k-steps in flight a wave (where the registers allow it)
  if constexpr (MB * RB <= 2) {
    if (k >= 2048) {
      hipLaunchKernelGGL((gemm_skinny_kernel<MB, RB, NORM, 8, SCALED>), dim3(cut.groups, cut.m_tiles), dim3(kGroupThreads), 0,
                         stream, static_cast<const bf16*>(x), static_cast<const float*>(h),
                         static_cast<const bf16*>(norm_weight), eps, static_cast<const bf16*>(w),
                         static_cast<bf16*>(out_bf16), static_cast<float*>(out_f32), m, n, k, epilogue, cut.rows, ahead);
      return;
    }
  }
  hipLaunchKernelGGL((gemm_skinny_kernel<MB, RB, NORM, 4, SCALED>), dim3(cut.groups, cut.m_tiles), dim3(kGroupThreads), 0,
                     stream, static_cast<const bf16*>(x), static_cast<const float*>(h),
                     static_cast<const bf16*>(norm_weight), eps, static_cast<const bf16*>(w),
                     static_cast<bf16*>(out_bf16), static_cast<float*>(out_f32), m, n, k, epilogue, cut.rows, ahead);
}

// Which instantiation serves a product of `m` rows against `n` rows of W: (MB, RB) as the
// entry point below chooses them.
void shape_of(int m, int n, int epilogue, int* mb_t, int* rb_t) {
  const int mb = (m + 15) / 16;
  const int out_rows = epilogue == kSiluMul ? n / 2 : n;
  const bool many_rows = out_rows >= 32768;   // the head: larger tiles, fewer workgroups
  if (mb == 1) {
    *mb_t = 1;
    if (epilogue == kSiluMul) *rb_t = 2;
    else if (many_rows) *rb_t = 4;
    else if (out_rows >= kTwoBlockRows && m >= 4) *rb_t = 2;
    else *rb_t = 1;
  } else if (out_rows <= 2048 && epilogue != kSiluMul) {
    *mb_t = 1;
    *rb_t = 1;
  } else if (epilogue == kSiluMul) {
    *mb_t = mb == 2 ? 2 : 4;
    *rb_t = 2;
  } else if (mb == 2) {
    *mb_t = 2;
    *rb_t = many_rows ? 2 : 1;
  } else {
    *mb_t = 4;
    *rb_t = 1;
  }
}

}  // namespace

extern "C" int ms_gemm_skinny_supported(int m, int n, int k, int epilogue) {
  if (m < 1 || m > 64 || n < 1 || k < 8 || k % 8 != 0) return 0;
  if (epilogue == kSiluMul && n % 2 != 0) return 0;
  return epilogue >= 0 && epilogue <= 3;
}

namespace {

void dispatch(const void* x, const void* w, void* out_bf16, void* out_f32, int m, int n, int k, int epilogue,
              hipStream_t stream, NormAhead ahead, bool scaled) {
  int mb_t, rb_t;
  shape_of(m, n, epilogue, &mb_t, &rb_t);
  // One row block (m <= 16), by the rows of W:
  //   Every workgroup reads all of x beside its rows of W, and the loads of x take the
  //   places of loads of W among those in flight.  From kTwoBlockRows rows of W on, two
  //   blocks a workgroup still give a workgroup to every compute unit, and half as many
  //   workgroups read x (25600 x 5120 at 8 rows: 74 -> 63 us); one row of x costs little either way.
  // More than 16 rows against a matrix of few rows: a workgroup that took all rows of x
  //   would read far more of x than of W.  The launch is cut along M too: 16 rows of x
  //   against 16 (or fewer) rows of W a workgroup.
#define MS_SKINNY_CASE(MB, RB)                                                                                 \
  if (mb_t == MB && rb_t == RB) {                                                                              \
    if (scaled) launch<MB, RB, false, true>(x, w, out_bf16, out_f32, m, n, k, epilogue, stream, nullptr, nullptr, 0.f, ahead); \
    else launch<MB, RB>(x, w, out_bf16, out_f32, m, n, k, epilogue, stream, nullptr, nullptr, 0.f, ahead);      \
    return;                                                                                                    \
  }
  MS_SKINNY_CASE(1, 1);
  MS_SKINNY_CASE(1, 2);
  MS_SKINNY_CASE(1, 4);
  MS_SKINNY_CASE(2, 1);
  MS_SKINNY_CASE(2, 2);
  MS_SKINNY_CASE(4, 1);
  MS_SKINNY_CASE(4, 2);
#undef MS_SKINNY_CASE
}

const NormAhead kNoNormAhead{nullptr, nullptr, nullptr, 0, 0.f};

}  // namespace

// x: bfloat16 [m, k]; w: bfloat16 [n, k]; the output by epilogue: 0 bfloat16 [m, n],
// 1 and 2 float [m, n], 3 bfloat16 [m, n / 2].
extern "C" int ms_gemm_skinny(const void* x, const void* w, void* out_bf16, void* out_f32, int m, int n, int k,
                              int epilogue, hipStream_t stream) {
  MS_REQUIRE(ms_gemm_skinny_supported(m, n, k, epilogue),
             "gemm_skinny: m %d (1..64), n %d, k %d (a multiple of 8) or epilogue %d is not supported", m, n, k,
             epilogue);
  MS_REQUIRE((epilogue == kStoreBf16 || epilogue == kSiluMul) ? out_bf16 != nullptr : out_f32 != nullptr,
             "gemm_skinny: the output of epilogue %d is null", epilogue);
  dispatch(x, w, out_bf16, out_f32, m, n, k, epilogue, stream, kNoNormAhead, false);
  MS_CHECK_LAUNCH("gemm_skinny");
  return 0;
}

// How many workgroups along N the += product of [m, k] against W [n, k] is cut into: the
// first size of the `squares` that ms_gemm_skinny_norm_ahead writes.
extern "C" int ms_gemm_skinny_groups(int m, int n) {
  int mb_t, rb_t;
  shape_of(m, n, kAddF32, &mb_t, &rb_t);
  return cut_of(mb_t, rb_t, m, n, kAddF32).groups;
}

// h[m, n] += x[m, k] . W[n, k]^T as epilogue 2, and for the RMSNorm (weight `norm_weight`
// [n]) and the product that follow: ahead_x[m, n] = bf16(norm_weight * h) and
// squares[group, m] = the sum of h^2 over the columns of workgroup `group`, for the
// ms_gemm_skinny_groups(m, n) workgroups.
extern "C" int ms_gemm_skinny_norm_ahead(const void* x, const void* w, void* h, int m, int n, int k,
                                         const void* norm_weight, void* ahead_x, void* squares,
                                         hipStream_t stream) {
  MS_REQUIRE(ms_gemm_skinny_supported(m, n, k, kAddF32),
             "gemm_skinny_norm_ahead: m %d (1..64), n %d or k %d (a multiple of 8) is not supported", m, n, k);
  MS_REQUIRE(h != nullptr && norm_weight != nullptr && ahead_x != nullptr && squares != nullptr,
             "gemm_skinny_norm_ahead: an output or the norm's weight is null");
  const NormAhead ahead{static_cast<const bf16*>(norm_weight), static_cast<bf16*>(ahead_x),
                        static_cast<float*>(squares), ms_gemm_skinny_groups(m, n), 0.f};
  dispatch(x, w, nullptr, h, m, n, k, kAddF32Ahead, stream, ahead, false);
  MS_CHECK_LAUNCH("gemm_skinny_norm_ahead");
  return 0;
}

// ms_gemm_skinny of the RMSNorm that ms_gemm_skinny_norm_ahead prepared: x is its ahead_x
// [m, k], squares [groups, m] its sums; every sum of the product is scaled by
// 1 / sqrt(sum of the row's squares / k + eps) before the epilogue.
extern "C" int ms_gemm_skinny_scaled(const void* x, const void* w, void* out_bf16, void* out_f32, int m, int n,
                                     int k, int epilogue, const void* squares, int groups, float eps,
                                     hipStream_t stream) {
  MS_REQUIRE(ms_gemm_skinny_supported(m, n, k, epilogue) && epilogue != kAddF32Ahead,
             "gemm_skinny_scaled: m %d (1..64), n %d, k %d (a multiple of 8) or epilogue %d is not supported", m, n,
             k, epilogue);
  MS_REQUIRE((epilogue == kStoreBf16 || epilogue == kSiluMul) ? out_bf16 != nullptr : out_f32 != nullptr,
             "gemm_skinny_scaled: the output of epilogue %d is null", epilogue);
  MS_REQUIRE(squares != nullptr && groups >= 1, "gemm_skinny_scaled: no sums of squares (%d groups)", groups);
  const NormAhead ahead{nullptr, nullptr, const_cast<float*>(static_cast<const float*>(squares)), groups, eps};
  dispatch(x, w, out_bf16, out_f32, m, n, k, epilogue, stream, ahead, true);
  MS_CHECK_LAUNCH("gemm_skinny_scaled");
  return 0;
}

// The same product with the RMSNorm of the 32-bit residual stream as its input:
// x = RMSNorm(h; norm_weight, eps), h: float [m, k], m <= 16, k a multiple of 8.
// Epilogues 0 (bfloat16 [m, n]) and 3 (gated activation, bfloat16 [m, n / 2]).
extern "C" int ms_gemm_skinny_normed(const void* h, const void* norm_weight, float eps, const void* w,
                                     void* out_bf16, int m, int n, int k, int epilogue, hipStream_t stream) {
  MS_REQUIRE(ms_gemm_skinny_supported(m, n, k, epilogue) && m <= 16 && (epilogue == kStoreBf16 || epilogue == kSiluMul),
             "gemm_skinny_normed: m %d (1..16), n %d, k %d (a multiple of 8) or epilogue %d is not supported", m, n,
             k, epilogue);
  MS_REQUIRE(h && norm_weight && w && out_bf16, "gemm_skinny_normed: null operand");
  MS_REQUIRE(eps > 0.f, "gemm_skinny_normed: eps must be positive");
  if (epilogue == kSiluMul) {
    launch<1, 2, true>(nullptr, w, out_bf16, nullptr, m, n, k, epilogue, stream, h, norm_weight, eps);
  } else if (n >= kTwoBlockRows) {
    // the 32-bit rows and the norm's weight are four times the bytes of x: two blocks from one row on
    launch<1, 2, true>(nullptr, w, out_bf16, nullptr, m, n, k, epilogue, stream, h, norm_weight, eps);
  } else {
    launch<1, 1, true>(nullptr, w, out_bf16, nullptr, m, n, k, epilogue, stream, h, norm_weight, eps);
  }
  MS_CHECK_LAUNCH("gemm_skinny_normed");
  return 0;
}
