// Brute-force Euclidean kNN for low-dimensional fp32 points (d <= 8, k <= 32)
// with the pre-filter of knn_lowd_impl.hpp evaluated on the gfx950 matrix
// cores.  Results are bit-identical to the reference's scalar loop
// (csrc/cuda/knn_cuda.cu:52-78): the matrix cores only decide which
// candidates are LOOKED AT, every distance that is kept is the exact fp32
// chain of direct differences.
//
// The filter value of a (query, candidate) pair is
//     t = w - 2 x.y,     w = fl(|x|^2) * (1 - eps),
// the dot product of the augmented rows (x_0 .. x_{d-1}, w) and
// (-2 y_0 .. -2 y_{d-1}, 1).  Every fp32 operand v is split into two bf16
// numbers, v = hi + lo + r with |r| <= 2^-16 |v| (hi = bf16(v),
// lo = bf16(v - hi); bf16 has the exponent range of fp32, so nothing
// overflows or needs scaling), and the four partial products
// hi*hi + lo*hi + hi*lo + lo*lo of up to four components fill the sixteen
// accumulation slots of ONE v_mfma_f32_32x32x16_bf16 (products exact, fp32
// accumulation): 32 candidates x 32 queries per instruction in a quarter of
// the time the fp32 matrix instruction needs, and about a tenth of what the
// vector ALU needs for the same 1,024 filter values.  Two of the sixteen
// slots would multiply w by the zero lo part of the query's 1; they carry
// -cut instead (see below), so that the matrix cores deliver t - cut and the
// vector ALU only has to collect SIGN BITS: one funnel shift per pair
// (v_alignbit_b32, full rate) where a compare into a scalar mask costs twice
// the issue cycles.
//
// A candidate with t >= cut = thresh (1 + eps) - fl(|y|^2) (1 - eps) (+ a tiny
// absolute term) can never have an exact distance below thresh, for
// eps = 2^-14:  |t_computed - t| <= 2^-16 |w| + 2^-15 * 2 sum |x_c y_c| (the
// split) + 50 u (|w| + 2 sum |x_c y_c|) (accumulation, u = 2^-24), the computed
// norms are within (1 +- d u) of the true ones and the exact chain within
// (1 +- (d + 2) u) of |x - y|^2; with 2 |x||y| <= |x|^2 + |y|^2 this gives
//     t - cut <= |x|^2 (-eps + 2^-14.3 + (d + 1) u)
//                + |y|^2 (-eps + 2^-14.9 + d u) + thresh ((d + 3) u - eps) < 0
// with room left for the 50 u |cut| that accumulating -cut along with the
// products adds.  -cut itself enters as the bf16 split of
// -(cut + 2^-15 |cut|), which is never above -cut.
// Operands below the bf16 normal range may be flushed to zero by the matrix
// cores: at most 2^-126 per operand, times the other factor (below 2e15 for
// operands of moderate norm); the absolute term of the cut covers it.  Rows
// whose squared norm is not a moderate finite number enter with zero
// coordinates and w = -1e38 (always looked at; an infinity would meet the
// zero lo part of the query's 1 and turn into NaN), padding rows with w = NaN
// (never pass a compare), queries with such a norm get cut = +inf and zero
// coordinates (look at every real row).
//
// Mapping: a workgroup owns 128 queries of one segment (4 waves x 32) and one
// slice of the segment's x rows; x streams through LDS in tiles of TX rows,
// each row once as the packed bf16 operand and once as fp32 coordinates for
// the exact distances.  Per 32-row step lane l supplies candidate row l % 32
// (both lane halves the same 16 bytes) and the hi (l < 32) or lo (l >= 32)
// parts of query l % 32; it receives the filter values of query l % 32
// against the 16 rows 8 (v / 4) + 4 (l / 32) + v % 4.  So lanes l and l + 32
// share a query and split its candidates: each keeps its own sorted list (its
// rows arrive in ascending order, so its own k-th distance is a strict
// bound), the two exchange their k-th distances after every drain, and the
// lists are united at the end.  A lane whose 16 sign bits of a step are not
// all clear parks (step, sign mask) in a per-lane LDS queue; the parked rows
// are resolved by all lanes together, exactly, when a queue fills up or the
// tile ends -- as in knn_lowd_impl.hpp.  Slices, shared bounds (`tau`) and the merge of partial
// lists are those of knn_lowd_impl.hpp with tiles of 128 queries.
//
// Start of a scan.  With empty lists every row passes, and until the bounds
// have come down most rows do: three quarters of all insertions of a scan
// over 4,096 rows fall into its first 1,024.  So before the first tile is
// scanned, its filter values are formed once without a cut: of the 16 values
// a lane receives per step it takes the smallest, evaluates that row exactly,
// and keeps the ceil(k / 2) smallest of these distances (one row per step:
// all different, and different from the partner lane's).  The larger of the
// two lanes' ceil(k / 2)-th distances bounds the query's k-th distance (at
// least k rows lie at or below it), and it is a bound of the quality "the
// k-th of 64 minima of 16": about k + k / 4 rows of the first tile pass
// it instead of k (1 + ln(1024 / k)).  The lists then fill from rows that
// pass this bound, in the scan proper.
#pragma once

#include "knn_mfma_impl.hpp"

namespace pca {

#ifdef PCA_MC_STATS
// (instrumented builds only) 0 drain rounds, 1 rounds with an insertion,
// 2 lane-rounds with a row, 3 lane-rounds with an insertion, 4 steps,
// 5 steps with a parked mask, 6 drains, 7 parked lane-steps
__device__ unsigned long long g_mc_stats[8];
#define PCA_MC_COUNT(i, v) atomicAdd(&g_mc_stats[i], (unsigned long long)(v))
#else
#define PCA_MC_COUNT(i, v) ((void)0)
#endif

constexpr int kMcQueries = 128; // queries per workgroup
// unsliced scans of up to this many LDS tiles start with a bound from sampled
// rows (measured on 64 x 2,048 / 32 x 4,096 points: 12-30 % less time in the
// kernel for k = 7 .. 31; slices of longer scans pay the sampling once each
// and already share their bounds: 2-8 % more time on 8 x 16,384 points)
#ifndef PCA_MC_SEED_TILES
#define PCA_MC_SEED_TILES 8
#endif
constexpr int kMcSeedTiles = PCA_MC_SEED_TILES;
// launches of up to this many workgroups (three per CU of a 256-CU device)
// take the kernel variants compiled without a register limit
constexpr int kMcRoomyGrid = 768;
constexpr int kMcQueueCap = 8; // parked steps per lane

template <int DIM> struct McShape {
  // matrix instructions per 32-row step: four augmented components each
  static constexpr int NI = (DIM + 1 + 3) / 4;
  static constexpr int XF = DIM <= 4 ? 4 : 8; // fp32 coordinates per row
  // a packed row: NI operand quads, then the coordinates (16-byte units)
  static constexpr int REC = NI + XF / 4;
  static constexpr int TX = DIM <= 4 ? 1024 : 256; // rows per LDS tile
};

constexpr float kMcEps = 1.0f / 16384.0f; // 2^-14

// fl(|y|^2) (1 - eps) rounded towards -inf, or +inf for a norm that is not a
// moderate finite number (the filter is then switched off for the query).
__device__ __forceinline__ float mc_damped_norm(float ysq) {
  if (!(ysq <= kFilterNormLimit))
    return __builtin_inff();
  const double c = (double)ysq * (1.0 - (double)kMcEps);
  float f = (float)c;
  if ((double)f > c)
    f = __uint_as_float(__float_as_uint(f) - 1u); // f > c >= 0
  return f;
}

// An upper bound of thresh (1 + eps) - ysq_damped + 2e-21 in three float
// operations: the fused multiply-add is within half an ulp of the exact
// value, the second one adds four ulps.  (2e-21: 48 accumulated terms, each
// off by at most 2^-126 * 2e15 when the matrix cores flush an operand.)
__device__ __forceinline__ float mc_filter_cut(float thresh,
                                               float ysq_damped) {
  if (ysq_damped == __builtin_inff())
    return __builtin_inff(); // examine everything exactly
  const float r = __builtin_fmaf(thresh, 1.0f + kMcEps, -ysq_damped);
  return __builtin_fmaf(__builtin_fabsf(r), 2.384185791015625e-07f, r) +
         2e-21f;
}

// One packed x row: per matrix instruction four hi parts and four lo parts
// (bf16) of the augmented row (x_0 .. x_{d-1}, w, 0 ...), then the fp32
// coordinates for the exact distances.
template <int DIM>
__device__ __forceinline__ void mc_pack_row(const float (&x)[DIM],
                                            uint4 (&out)[McShape<DIM>::REC]) {
  constexpr int NI = McShape<DIM>::NI;
  constexpr int XF = McShape<DIM>::XF;
#pragma unroll
  for (int e = 0; e < XF; e += 4) {
    uint32_t v[4];
#pragma unroll
    for (int f = 0; f < 4; ++f)
      v[f] = (e + f < DIM) ? __float_as_uint(x[e + f]) : 0u;
    out[NI + e / 4] = make_uint4(v[0], v[1], v[2], v[3]);
  }
  float s = x[0] * x[0];
#pragma unroll
  for (int c = 1; c < DIM; ++c)
    s = __builtin_fmaf(x[c], x[c], s);
  const bool moderate = s <= kFilterNormLimit;
  // a row whose norm is not a moderate finite number always passes the
  // filter and is judged by its exact distance alone
  const float w = moderate ? s * (1.0f - kMcEps) : -1e38f;
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    uint32_t hi[4], lo[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int c = 4 * i + e;
      hi[e] = 0;
      lo[e] = 0;
      if (c < DIM) {
        if (moderate)
          mc_split(x[c], hi[e], lo[e]);
      } else if (c == DIM) {
        if (moderate)
          mc_split(w, hi[e], lo[e]);
        else
          hi[e] = __float_as_uint(w) >> 16;
      }
    }
    out[i] = make_uint4(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16),
                        lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16));
  }
}

// Everything the search kernel needs prepared, in one launch (workgroups of
// kPlanThreads threads over max(n, m) rows):
//   * every x row packed once per call; the search kernel's workgroups, each
//     of which streams its whole segment through LDS, then just copy;
//   * the shared bounds of sliced segments set to their start value (tau);
//   * by the first workgroup: the segment pointers when the caller passed
//     example ids (src), and the first work item of every segment (the plan,
//     when work_start is given).
struct McSetup {
  const float *x;
  int n, d_in;
  uint4 *out;
  float *tau; // [m] or NULL
  // the compaction's block sums to clear (DenseResult::edge_sums), or NULL
  unsigned long long *edge_sums = nullptr;
  int edge_blocks = 0;
  int m;
  float tau_value;
  const int64_t *ptr_y; // plan input (src.ptr_y when src is used)
  int num_segments, per_item;
  int *work_start; // NULL: no plan
  SegmentSource src;
};

template <int DIM>
__global__ __launch_bounds__(kPlanThreads) void mc_setup_kernel(McSetup a) {
  constexpr int REC = McShape<DIM>::REC;
  __shared__ int partial[kPlanThreads];
  if (a.edge_sums != nullptr)
    for (int b = blockIdx.x * kPlanThreads + threadIdx.x; b < a.edge_blocks;
         b += gridDim.x * kPlanThreads)
      a.edge_sums[b] = 0ull;
  if (blockIdx.x == 0 && a.work_start != nullptr) {
    if (a.src.ids_x != nullptr) {
      pointers_from_ids(a.src, a.num_segments);
      __syncthreads();
    }
    plan_segments(a.ptr_y, a.m, a.num_segments, a.per_item, a.work_start,
                  partial);
  }
  const int row = blockIdx.x * kPlanThreads + threadIdx.x;
  if (a.tau != nullptr && row < a.m)
    a.tau[row] = a.tau_value;
  const float *__restrict__ x = a.x;
  uint4 *__restrict__ out = a.out;
  const int n = a.n, d_in = a.d_in;
  if (row >= n)
    return;
  float v[DIM];
#pragma unroll
  for (int c = 0; c < DIM; ++c)
    v[c] = c < d_in ? x[(size_t)row * d_in + c] : 0.0f;
  uint4 packed[REC];
  mc_pack_row<DIM>(v, packed);
#pragma unroll
  for (int i = 0; i < REC; ++i)
    out[(size_t)row * REC + i] = packed[i];
}

// NEAREST: the search of the `nearest` operator -- one neighbour, limit 1e38,
// the reference's order among equal distances (see device_utils.hpp) -- whose
// result goes to p.out_nearest as a row number (0 when nothing qualified).
// (launch bounds: 5-8 dimensions with lists of 16 came out at 136 registers,
// up to 3 dimensions with lists of 24 at 138-140: three waves per SIMD; asked
// for four - 128 registers, up to 12 spilled words - they run 5 % and 10 %
// faster on clouds that fill the device, 2 % slower on 16 x 4,096 points;
// ROOMY: the same kernel without that limit, for launches of at most three
// workgroups per CU, which gain nothing from a fourth and lose to the spills)
template <int DIM, int K, bool NEAREST = false, bool ROOMY = false>
__global__ __launch_bounds__(
    kBlock,
    (!ROOMY && ((DIM == 8 && K == 16) || (DIM <= 3 && K == 24))) ? 4 : 1) void
knn_lowd_mc_kernel(KnnLowdParams p) {
  static_assert(!NEAREST || K == 1, "nearest keeps one neighbour");
  constexpr float kLimit = SearchLimit<NEAREST>::value;
  constexpr int NI = McShape<DIM>::NI;
  constexpr int XF = McShape<DIM>::XF;
  constexpr int TX = McShape<DIM>::TX;
  constexpr int TQ = kMcQueries;
  constexpr int QCAP = kMcQueueCap;
  constexpr int PT = TX / kBlock; // rows staged per thread

  constexpr int REC = McShape<DIM>::REC;
  // the tile's packed rows, every 16-byte unit of a row in a plane of its
  // own: the lanes of a wave read the same unit of 32 consecutive rows, and
  // with the units of one row side by side (32 bytes from row to row in three
  // dimensions) two lanes met in every bank
  __shared__ __attribute__((aligned(16))) uint4 rows_lds[REC][TX];
  // parked steps: (step << 16) | mask of the lane's 16 rows that passed
  __shared__ uint32_t queue[QCAP][kBlock];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int half = lane >> 5;
  const int col = lane & 31;

  // this workgroup's work item = (slice, tile of queries), from its number
  // (handing the items out XCD by XCD, so that neighbours share an L2, was
  // tried: a third of the HBM reads and 25 % more time on 8 scans of
  // 60,000-200,000 points -- at 2 % of the HBM roof the reads cost nothing,
  // the hand-out through atomics does)
  const int total_tiles = p.work_start[p.num_segments];
  if (total_tiles == 0)
    return;
  const int chunk = blockIdx.x / total_tiles;
  const int tile = blockIdx.x - chunk * total_tiles;
  if (chunk >= p.num_chunks)
    return;
  const int item = chunk * total_tiles + tile;
  const int seg = find_segment(p.work_start, p.num_segments, tile);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int q = y_begin + (tile - p.work_start[seg]) * TQ + wave * 32 + col;
  const bool valid = q < y_end;
  const int d_in = p.d_in;
  const int k = p.k;

  const int seg_len = x_end - x_begin;
  const int chunk_len =
      ((seg_len + p.num_chunks - 1) / p.num_chunks + TX - 1) / TX * TX;
  const int c_begin = min(x_end, x_begin + chunk * chunk_len);
  const int c_count = min(x_end, c_begin + chunk_len) - c_begin;
  const int num_tiles = (c_count + TX - 1) / TX;


  // ---- per-lane query state ---------------------------------------------
  float yq[DIM];
#pragma unroll
  for (int c = 0; c < DIM; ++c)
    yq[c] = (valid && c < d_in) ? p.y[(size_t)q * d_in + c] : 0.0f;
  float ysq = yq[0] * yq[0];
#pragma unroll
  for (int c = 1; c < DIM; ++c)
    ysq = __builtin_fmaf(yq[c], yq[c], ysq);
  const bool y_moderate = ysq <= kFilterNormLimit;
  // B operands: the hi (lanes 0-31) or lo (lanes 32-63) parts of
  // (-2 y, 1, 0 ...), four components per instruction, given twice (against
  // the hi and the lo parts of the row)
  mc_bf16x8_t yb[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    uint32_t part[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int c = 4 * i + e;
      // (a lane without a query multiplies everything by zero and starts
      // from a large positive value: nothing passes)
      float v = 0.0f;
      if (c < DIM)
        v = (valid && y_moderate) ? -2.0f * yq[c] : 0.0f;
      else if (c == DIM)
        v = valid ? 1.0f : 0.0f;
      uint32_t hi, lo;
      mc_split(v, hi, lo);
      part[e] = half ? lo : hi;
    }
    const uint32_t w0 = part[0] | (part[1] << 16);
    const uint32_t w1 = part[2] | (part[3] << 16);
    const uint4 packed = make_uint4(w0, w1, w0, w1);
    yb[i] = __builtin_bit_cast(mc_bf16x8_t, packed);
  }

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - k) ? lowest_key() : SearchLimit<NEAREST>::empty();
  // exact distances must be strictly below thresh; a lane without a query
  // accepts nothing
  const float ysq_damped = mc_damped_norm(ysq);
  float thresh = valid ? kLimit : -__builtin_inff();
  float cut = valid ? mc_filter_cut(thresh, ysq_damped) : -1e38f;
  float shared = kLimit; // bound inherited from other slices / partner
  float posted = kLimit;
  // The filter tests the SIGN of t - cut: -cut rides along in the two
  // accumulation slots that would otherwise multiply w by the (zero) lo part
  // of the query's 1.  On the row side the upper lanes put 1 where they hold
  // w_hi and w_lo (two operations per step, see the scan loop); on the query
  // side they carry the hi and lo parts of -cut', cut' = cut + 2^-15 |cut|
  // (so that the 2^-16 |cut'| the split may lose never lowers the cut).  An
  // infinite cut (filter switched off) enters as the largest finite bf16.
  constexpr int WI = DIM / 4;  // matrix instruction that holds component DIM
  constexpr int WE = DIM % 4;  // ... as its WE-th component
  const uint32_t one_keep =
      half ? ~(0xffffu << (16 * (WE & 1))) : 0xffffffffu;
  const uint32_t one_bits = half ? (0x3f80u << (16 * (WE & 1))) : 0u;
  const uint4 yb_plain = __builtin_bit_cast(uint4, yb[WI]);
  auto refresh_cut = [&]() {
    if (half) {
      float neg = -__builtin_fmaf(__builtin_fabsf(cut), 3.0517578125e-05f, cut);
      uint32_t hi, lo;
      if (__builtin_fabsf(neg) < 1e38f) {
        mc_split(neg, hi, lo);
      } else {
        hi = neg < 0.0f ? 0xff7fu : 0x7f7fu;
        lo = 0;
      }
      uint4 b = yb_plain;
      const uint32_t keep = ~(0xffffu << (16 * (WE & 1)));
      const uint32_t sh = 16 * (WE & 1);
      if (WE < 2) {
        b.x = (b.x & keep) | (hi << sh);
        b.z = (b.z & keep) | (lo << sh);
      } else {
        b.y = (b.y & keep) | (hi << sh);
        b.w = (b.w & keep) | (lo << sh);
      }
      yb[WI] = __builtin_bit_cast(mc_bf16x8_t, b);
    }
  };
  refresh_cut();
  // parked steps of this lane: queue[0 .. qcount)[tid]; qnext is the byte
  // offset in `queue` at which the next one goes
  constexpr int QROW = kBlock * (int)sizeof(uint32_t);
  const int qfirst = tid * (int)sizeof(uint32_t);
  int qnext = qfirst;

  auto set_thresh = [&](float v) {
    if (valid) {
      thresh = v;
      cut = mc_filter_cut(v, ysq_damped);
    }
  };

  // ---- tile staging -------------------------------------------------------
  uint4 stage[PT][REC];
  // a padding row: w = NaN (hi part of component DIM), never passes a compare
  auto pad_quad = [](int i) {
    uint4 o = make_uint4(0u, 0u, 0u, 0u);
    if (i == DIM / 4) {
      const uint32_t nan_bits = 0x7fc0u << (16 * (DIM % 2));
      if (DIM % 4 < 2)
        o.x = nan_bits;
      else
        o.y = nan_bits;
    }
    return o;
  };

  auto load_tile = [&](int t) {
#pragma unroll
    for (int r = 0; r < PT; ++r) {
      const int pos = t * TX + r * kBlock + tid;
      const size_t g = (size_t)c_begin + pos;
      const bool ok = pos < c_count;
#pragma unroll
      for (int i = 0; i < REC; ++i)
        stage[r][i] = ok ? p.x_split[g * REC + i] : pad_quad(i);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int r = 0; r < PT; ++r)
#pragma unroll
      for (int i = 0; i < REC; ++i)
        rows_lds[i][r * kBlock + tid] = stage[r][i];
  };

  auto sync_bounds = [&]() {
    if (valid) {
      const float own = key_dist(best[K - 1]);
      const float seen = __hip_atomic_load(&p.tau[q], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
      if (own < seen && own < posted) {
        // squared distances are non-negative: floats order like their bits
        __hip_atomic_fetch_min(reinterpret_cast<int *>(&p.tau[q]),
                               (int)__float_as_uint(own), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        posted = own;
      } else if (seen < posted) {
        posted = seen;
        // another list's k-th distance: equality must still pass
        shared = __builtin_fminf(shared, next_up_positive(seen));
        set_thresh(__builtin_fminf(thresh, shared));
      }
    }
    refresh_cut();
  };

  // What the two lanes of a query tell each other about its final k-th
  // distance (equality admitted: their rows interleave).
  auto partner_bounds = [&]() {
    // the partner's k-th distance bounds the query's final k-th distance too
    // (equality admitted: its rows interleave with this lane's)
    const float own = key_dist(best[K - 1]);
    const auto both = __builtin_amdgcn_permlane32_swap(
        __float_as_uint(own), __float_as_uint(own), false, false);
    float partner = __uint_as_float(half ? both[0] : both[1]);
    // So does the larger of the two lanes' (k - c)-th distances for any
    // c <= k / 2: together the lists hold 2 (k - c) >= k rows at or below it.
    // The lanes see every other group of rows, so with c = k / 2 this is close
    // to the k-th distance of both lists united -- about half as many rows
    // get past it as past a lane's own k-th distance.  (The entry is picked
    // by a uniform branch: c takes one of five values for a list width.)
    if (K >= 2) {
      const int c = k >> 1;
      float mid = kLimit;
#pragma unroll
      for (int cc = (K >= 8 ? K / 2 - 4 : 0); cc <= K / 2; ++cc)
        if (cc >= 1 && cc == c) {
          asm volatile(""); // (keeps this a branch)
          mid = key_dist(best[K - 1 - cc]);
        }
      const auto mids = __builtin_amdgcn_permlane32_swap(
          __float_as_uint(mid), __float_as_uint(mid), false, false);
      const float partner_mid = __uint_as_float(half ? mids[0] : mids[1]);
      partner = __builtin_fminf(partner, __builtin_fmaxf(mid, partner_mid));
    }
    if (valid && partner < kLimit) {
      shared = __builtin_fminf(shared, next_up_positive(partner));
      if (shared < thresh)
        set_thresh(shared);
    }
  };

  // Resolves the parked candidates: in every round each lane takes the next
  // row of its parked steps (steps in the order they were parked, rows in
  // ascending order) and all 64 lanes evaluate their exact distances from the
  // tile in LDS together.
  auto drain = [&](int g_base, int rows) {
    bool changed = false; // wave-uniform
    PCA_MC_COUNT(6, lane == 0);
    const int qcount = (qnext - qfirst) / QROW;
    int taken = 0;         // parked steps this lane has started on
    uint32_t pending = 0;  // rows of the current step still to look at
    int step_base = 0;     // first of this lane's rows in that step
    for (;;) {
      if (pending == 0 && taken < qcount) {
        const uint32_t word = queue[taken][tid];
        ++taken;
        pending = word & 0xffffu;
        step_base = (int)(word >> 16) * 32 + 4 * half;
      }
      const bool has = pending != 0;
      if (!__any(has))
        break;
      PCA_MC_COUNT(0, lane == 0);
      PCA_MC_COUNT(2, has);
      // bit 15 - v of the mask stands for accumulator v = row
      // 8 (v / 4) + v % 4 of the lane's rows: highest bit first
      const int bit = 31 - __builtin_clz(has ? pending : 1u);
      const int v = 15 - bit;
      pending &= ~(1u << bit);
      const int j = has ? step_base + 2 * (v & 12) + (v & 3) : 0;
      float row[XF];
#pragma unroll
      for (int e = 0; e < XF; e += 4) {
        const uint4 q4 = rows_lds[NI + e / 4][j];
        row[e] = __uint_as_float(q4.x);
        row[e + 1] = __uint_as_float(q4.y);
        row[e + 2] = __uint_as_float(q4.z);
        row[e + 3] = __uint_as_float(q4.w);
      }
      const float d0 = row[0] - yq[0];
      float d = d0 * d0;
#pragma unroll
      for (int c = 1; c < DIM; ++c) {
        const float dc = row[c] - yq[c];
        d = __builtin_fmaf(dc, dc, d);
      }
      // (j < rows: a padding row is never a candidate, whatever the filter
      // made of it)
      const bool ok = has && j < rows && d < thresh;
      if (!__any(ok))
        continue;
      PCA_MC_COUNT(1, lane == 0);
      PCA_MC_COUNT(3, ok);
      const uint32_t row_id = NEAREST
                                  ? nearest_tie((uint32_t)(g_base + j - x_begin))
                                  : (uint32_t)(g_base + j);
      const double key =
          ok ? make_key(d, row_id) : SearchLimit<NEAREST>::empty();
      sorted_insert<K>(best, key);
      float own_bound = key_dist(best[K - 1]);
      // (`nearest`: a later row of EQUAL distance can still win the tie)
      if (NEAREST && own_bound < kLimit)
        own_bound = next_up_positive(own_bound);
      // (the filter's cut follows once, after the last round)
      if (valid)
        thresh = __builtin_fminf(own_bound, shared);
      changed = true;
    }
    qnext = qfirst;
    if (!changed)
      return;
    set_thresh(thresh);
    partner_bounds();
    refresh_cut();
  };

  if (num_tiles > 0)
    load_tile(0);

  for (int t = 0; t < num_tiles; ++t) {
    // one LDS buffer: the next tile waits in registers while this one is
    // scanned (other workgroups of the CU cover the two barriers)
    __syncthreads();
    store_tile();
    __syncthreads();
    if (t + 1 < num_tiles)
      load_tile(t + 1);
    // (early in a scan the bounds move fastest: tiles 0, 1, 3, 7, then every
    // sync_mask + 1 tiles)
    if (p.tau && (t < 8 ? (t & (t + 1)) == 0
                        : (t & p.sync_mask) == p.sync_mask))
      sync_bounds();
    const int g_base = c_begin + t * TX;
    const int rows = min(TX, c_count - t * TX);
    const int steps32 = (rows + 31) / 32;

    // a bound before the first row is looked at (see "Start of a scan")
    constexpr int SEEDS = K / 2;
    const bool seeded = !NEAREST && K >= 8 && t == 0 &&
                        steps32 >= 2 * SEEDS && num_tiles <= kMcSeedTiles &&
                        p.num_chunks == 1;
    if (!NEAREST && K >= 8 && seeded) {
      float seed[SEEDS > 0 ? SEEDS : 1];
#pragma unroll
      for (int j = 0; j < SEEDS; ++j)
        seed[j] = __builtin_inff();
      // no cut in the product: the slots that carry it multiply by zero
      yb[WI] = __builtin_bit_cast(mc_bf16x8_t, yb_plain);
      uint4 a_seed[NI];
#pragma unroll
      for (int i = 0; i < NI; ++i)
        a_seed[i] = rows_lds[i][col];
      for (int rt = 0; rt < steps32; ++rt) {
        mfma_acc_t acc = {0};
#pragma unroll
        for (int i = 0; i < NI; ++i)
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              __builtin_bit_cast(mc_bf16x8_t, a_seed[i]), yb[i], acc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < NI; ++i)
          a_seed[i] = rows_lds[i][min(rt + 1, TX / 32 - 1) * 32 + col];
        // the smallest of the 16 values, its accumulator number in the four
        // lowest bits (which of two nearly equal rows is taken does not
        // matter; a NaN -- padding -- loses against any number)
        float tagged[16];
#pragma unroll
        for (int v = 0; v < 16; ++v)
          tagged[v] = __uint_as_float((__float_as_uint(acc[v]) & ~15u) |
                                      (uint32_t)v);
        float m0 = min3f(tagged[0], tagged[1], tagged[2]);
        float m1 = min3f(tagged[3], tagged[4], tagged[5]);
        float m2 = min3f(tagged[6], tagged[7], tagged[8]);
        float m3 = min3f(tagged[9], tagged[10], tagged[11]);
        float m4 = min3f(tagged[12], tagged[13], tagged[14]);
        m0 = min3f(m0, m1, m2);
        m3 = min3f(m3, m4, tagged[15]);
        const int v = (int)(__float_as_uint(__builtin_fminf(m0, m3)) & 15u);
        const int j = rt * 32 + 4 * half + 2 * (v & 12) + (v & 3);
        float row[XF];
#pragma unroll
        for (int e = 0; e < XF; e += 4) {
          const uint4 q4 = rows_lds[NI + e / 4][j];
          row[e] = __uint_as_float(q4.x);
          row[e + 1] = __uint_as_float(q4.y);
          row[e + 2] = __uint_as_float(q4.z);
          row[e + 3] = __uint_as_float(q4.w);
        }
        const float d0 = row[0] - yq[0];
        float d = d0 * d0;
#pragma unroll
        for (int c = 1; c < DIM; ++c) {
          const float dc = row[c] - yq[c];
          d = __builtin_fmaf(dc, dc, d);
        }
        // (a padding row, a NaN or a distance beyond the limit is no sample)
        const float sample = (j < rows && d < kLimit) ? d : __builtin_inff();
#pragma unroll
        for (int e = SEEDS - 1; e >= 1; --e)
          seed[e] = __builtin_amdgcn_fmed3f(seed[e - 1], seed[e], sample);
        seed[0] = __builtin_fminf(seed[0], sample);
      }
      // the ceil(k / 2)-th smallest sample of this lane and of its partner
      const int mine = (k + 1) / 2 - 1;
      float own = __builtin_inff();
#pragma unroll
      for (int e = 0; e < SEEDS; ++e)
        if (e == mine) {
          asm volatile(""); // (keeps this a branch)
          own = seed[e];
        }
      const auto both = __builtin_amdgcn_permlane32_swap(
          __float_as_uint(own), __float_as_uint(own), false, false);
      const float partner = __uint_as_float(half ? both[0] : both[1]);
      const float bound = __builtin_fmaxf(own, partner);
      if (valid && bound < kLimit) {
        // (equality must pass: the rows at the bound are among the k nearest)
        shared = __builtin_fminf(shared, next_up_positive(bound));
        if (shared < thresh)
          set_thresh(shared);
      }
      refresh_cut();
    }

    uint4 a_next[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i)
      a_next[i] = rows_lds[i][col];
    for (int rt = 0; rt < steps32; ++rt) {
      mfma_acc_t acc = {0};
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        uint4 a = a_next[i];
        if (i == WI) {
          // upper lanes: 1 in place of w_hi and w_lo (times -cut' parts)
          if (WE < 2) {
            a.x = (a.x & one_keep) | one_bits;
            a.z = (a.z & one_keep) | one_bits;
          } else {
            a.y = (a.y & one_keep) | one_bits;
            a.w = (a.w & one_keep) | one_bits;
          }
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            __builtin_bit_cast(mc_bf16x8_t, a), yb[i], acc, 0, 0, 0);
      }
      // the next step's rows are on their way while this step is filtered
      // (the last read stays inside the tile)
#pragma unroll
      for (int i = 0; i < NI; ++i)
        a_next[i] = rows_lds[i][min(rt + 1, TX / 32 - 1) * 32 + col];

      // accumulator v = t - cut of row 8 (v / 4) + 4 half + v % 4: its sign
      // bit says "look at this row".  One funnel shift per accumulator
      // gathers the 16 signs of a lane (bit 15 - v); compares into scalar
      // masks would cost twice as many issue cycles each.
      uint32_t mask = 0;
#pragma unroll
      for (int v = 0; v < 16; ++v)
        mask = __builtin_amdgcn_alignbit(mask, __float_as_uint(acc[v]), 31);
      PCA_MC_COUNT(4, lane == 0);
      if (__any(mask != 0)) {
        PCA_MC_COUNT(5, lane == 0);
        PCA_MC_COUNT(7, mask != 0);
        if (mask != 0) {
          *reinterpret_cast<uint32_t *>(
              reinterpret_cast<char *>(&queue[0][0]) + qnext) =
              ((uint32_t)rt << 16) | mask;
          qnext += QROW;
        }
        // (the first drains of a scan come early -- after steps 0, 1, 3, 7,
        // 15 and 31 of its first tile -- while the lists are empty or their
        // bounds still loose and many rows pass)
        if (__any(qnext >= qfirst + QCAP * QROW) ||
            (t == 0 && !seeded && (rt & (rt + 1)) == 0))
          drain(g_base, rows);
      }
    }
    // parked positions refer to this tile: resolve them before it goes away
    drain(g_base, rows);
  }

  // ---- results ----------------------------------------------------------
  // unite the two half lists of each query in the lower lane
  unite_halves<K>(best, k, half);

  if (half == 0) {
    if (p.num_chunks == 1) {
      if (valid) {
        if constexpr (NEAREST)
          write_nearest(best[0], q, x_begin, p.out_nearest);
        else
          note_edges<K>(best, k, q,
                        write_dense<K>(best, k, q, p.out_idx, p.out_dist,
                                       p.out_count),
                        p.edge_sums, p.self_pos, p.kept);
      }
    } else {
      // sorted keys of this slice, [item][slot][query of the tile]
      double *dst = p.partial + (size_t)item * k * TQ + wave * 32 + col;
#pragma unroll
      for (int j = 0; j < K; ++j) {
        const int e = j - (K - k);
        if (e >= 0)
          dst[(size_t)e * TQ] = best[j];
      }
    }
  }
}

// One padded dimension of the dispatch table (instantiated in its own
// translation unit so the dimensions build in parallel).
template <int DIM>
hipError_t launch_knn_lowd_mc_dim(const KnnLowdParams &p, int kbucket,
                                  int grid, hipStream_t stream);
// Fills a.out (n * McShape<DIM>::REC entries) with the packed rows, and the
// rest of McSetup.
template <int DIM>
hipError_t launch_mc_setup(const McSetup &a, hipStream_t stream);
#define PCA_LOWD_MC_DEFINE(DIM_)                                               \
  template <>                                                                  \
  hipError_t launch_mc_setup<DIM_>(const McSetup &a, hipStream_t stream) {     \
    const int rows = a.n > a.m ? a.n : a.m;                                    \
    hipLaunchKernelGGL((mc_setup_kernel<DIM_>),                                \
                       dim3((rows + kPlanThreads - 1) / kPlanThreads),         \
                       dim3(kPlanThreads), 0, stream, a);                      \
    return hipGetLastError();                                                  \
  }                                                                            \
  template <>                                                                  \
  hipError_t launch_knn_lowd_mc_dim<DIM_>(const KnnLowdParams &p, int kbucket, \
                                          int grid, hipStream_t stream) {      \
    switch (kbucket) {                                                         \
    case 8:                                                                    \
      hipLaunchKernelGGL((knn_lowd_mc_kernel<DIM_, 8>), dim3(grid),            \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 16:                                                                   \
      hipLaunchKernelGGL((knn_lowd_mc_kernel<DIM_, 16>), dim3(grid),           \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 24:                                                                   \
      if (DIM_ <= 3 && grid <= kMcRoomyGrid)                                   \
        hipLaunchKernelGGL((knn_lowd_mc_kernel<DIM_, 24, false, true>),        \
                           dim3(grid), dim3(kBlock), 0, stream, p);            \
      else                                                                     \
        hipLaunchKernelGGL((knn_lowd_mc_kernel<DIM_, 24>), dim3(grid),         \
                           dim3(kBlock), 0, stream, p);                        \
      break;                                                                   \
    case 32:                                                                   \
      hipLaunchKernelGGL((knn_lowd_mc_kernel<DIM_, 32>), dim3(grid),           \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 1: /* the `nearest` search */                                         \
      hipLaunchKernelGGL((knn_lowd_mc_kernel<DIM_, 1, true>), dim3(grid),      \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    default:                                                                   \
      return hipErrorInvalidValue;                                             \
    }                                                                          \
    return hipGetLastError();                                                  \
  }

} // namespace pca
