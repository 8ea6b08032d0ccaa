// Brute-force kNN for low-dimensional fp32 points (d <= 8) on gfx950.
//
// Computes what knn_kernel of the reference computes
// (csrc/cuda/knn_cuda.cu:30-84: one thread per query, linear scan of the
// query's segment of x, sorted insertion list), with a different machine
// mapping:
//
//   * a work item is (query tile, x chunk): 256 * QPT queries of ONE segment
//     (found from the work_start table, never crossing a segment boundary)
//     against one of S equal slices of that segment's x rows.  Slicing x
//     evens out ragged segments and gives small problems enough workgroups;
//     with S > 1 every item leaves its sorted top-k keys in a partial buffer
//     and knn_lowd_merge_kernel merges the S lists of each query;
//   * each lane owns QPT queries, their coordinates live in registers;
//   * x rows stream through LDS in tiles of TX points, staged with coalesced
//     global loads, double-buffered, stored component-major so that the inner
//     loop reads four candidates per ds_read_b128 and every lane of the wave
//     reads the same address (broadcast, no bank conflicts); the next group's
//     reads are issued before the current group is evaluated;
//   * distances use direct differences and one fused multiply-add per
//     dimension in ascending dimension order -- bit-identical to
//     `dist += (x - y) * (x - y)` as a GPU compiler contracts it;
//   * the running top-k of a query is a register-resident ascending list of K
//     64-bit (distance, row) keys (see device_utils.hpp), updated with a
//     branch-free min/max insertion network;
//   * candidates are pre-filtered against the list's current worst distance
//     (for the Euclidean metric with the 3-instruction expanded form described
//     at filter_cut below); the lanes that pass are collected with a ballot
//     into scalar registers, so the common "nobody passed" case is one scalar
//     branch; the few candidates that pass are parked -- just their position
//     in the tile -- in a small per-lane LDS queue, and only when some lane's
//     queue is nearly full (or the tile ends) do all 64 lanes together take
//     the exact distance of their parked candidates from LDS and run the
//     insertion network, so the wave pays neither K slots of insertion nor an
//     exact distance each time one of its lanes accepts a candidate;
//   * with S > 1 the items of one query share their pruning bound through
//     `tau` (one float per query, device-scope atomic min): the k-th best
//     distance any slice has reached bounds the final k-th distance from
//     above, so every slice may drop candidates farther than that.  A bound
//     taken from another slice admits equality (ties are settled by row in
//     the merge), the slice's own k-th distance is a strict bound because all
//     later candidates of the slice have higher rows.
//
// Results per query: rows [K-k, K) of the list = the k best (distance, row)
// pairs in ascending order; slots never filled keep row -1 (segment smaller
// than k, or candidates at distance >= 1e10 / NaN, which the reference never
// inserts either).
#pragma once

#include "device_utils.hpp"
#include "launchers.hpp"

namespace pca {

constexpr int kLowdTileX = 1024; // candidates per LDS tile
constexpr int kLowdQueueCap = 16;
constexpr int kLowdGroup = 4; // candidates per inner-loop step

// Everything a low-dimensional kNN launch needs (passed by value).
struct KnnLowdParams {
  const float *x;
  const float *y;
  const int64_t *ptr_x;
  const int64_t *ptr_y;
  int n, m, d_in, num_segments, k;
  const int *work_start; // [num_segments + 1] first query tile of each segment
  int num_chunks;        // S: slices of every segment's x rows
  const uint4 *x_split;  // matrix-core kernel: packed rows of x
  float *tau;            // [m] shared pruning bounds or NULL
  int sync_mask = 3;     // ... bounds are exchanged when (tile & mask) == mask
  double *partial;       // [S * tiles][k][tile queries] keys (S > 1) or NULL
  int *out_idx;          // dense results (written here only when S == 1)
  float *out_dist;
  int *out_count;
  int64_t *out_nearest;  // [m] result of the `nearest` search, else unused
  // for the compaction (DenseResult; NULL: not asked for): slots it will
  // write per kCompactBlockQueries queries, the slot of the query's own row
  // and the count without it
  unsigned long long *edge_sums = nullptr;
  int *self_pos = nullptr;
  int *kept = nullptr;
  // second pass behind another search (knn_merge_kernel): nothing runs while
  // *gate is 0, and only queries with a non-zero redo_q entry are written
  const int *gate = nullptr;
  const int *redo_q = nullptr;
};

__device__ __forceinline__ float next_up_positive(float v) {
  return __uint_as_float(__float_as_uint(v) + 1u); // v >= 0, finite
}

// Writes the real slots of a sorted key list as dense results.
template <int K>
__device__ __forceinline__ int write_dense(const double (&best)[K], int k,
                                           int q, int *out_idx,
                                           float *out_dist, int *out_count) {
  const size_t row = (size_t)q * k;
  int found = 0;
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const int e = j - (K - k);
    if (e >= 0 && best[j] < empty_key()) {
      out_idx[row + e] = key_row(best[j]);
      if (out_dist)
        out_dist[row + e] = key_dist(best[j]);
      ++found;
    }
  }
  out_count[q] = found;
  return found;
}

// sums[block] += value for every lane that gets here (any subset of a wave;
// 0 <= value < 128), with one atomic per distinct block among them: the lanes
// of a wave hold neighbouring queries, and atomics on one address take turns
// in the L2 (65,536 single ones on 256 addresses cost 45 us).
__device__ __forceinline__ void add_to_block_sum(unsigned long long *sums,
                                                 int block, int value) {
  const int lane = (int)(threadIdx.x & (kWave - 1));
  bool done = false;
  for (;;) {
    const uint64_t waiting = __ballot(!done);
    if (waiting == 0)
      break;
    const int leader = (int)__builtin_ctzll(waiting);
    const int lead_block = __shfl(block, leader);
    const bool mine = !done && block == lead_block;
    int total = 0;
#pragma unroll
    for (int b = 0; b < 7; ++b)
      total += __builtin_popcountll(__ballot(mine && ((value >> b) & 1))) << b;
    if (lane == leader)
      atomicAdd(&sums[lead_block], (unsigned long long)total);
    done = done || mine;
  }
}

// What the compaction wants to know about the list just written (see
// DenseResult): adds the query's slots to its block's sum and, for graph
// results (self_pos given), notes where the query's own row sits.
template <int K>
__device__ __forceinline__ void note_edges(const double (&best)[K], int k,
                                           int q, int found,
                                           unsigned long long *edge_sums,
                                           int *self_pos, int *kept) {
  if (edge_sums == nullptr)
    return;
  int keep = found;
  if (self_pos != nullptr) {
    int self = -1;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int e = j - (K - k);
      if (e >= 0 && best[j] < empty_key() && key_row(best[j]) == q)
        self = e;
    }
    keep -= self >= 0 ? 1 : 0;
    self_pos[q] = self;
    kept[q] = keep;
  }
  add_to_block_sum(edge_sums, q / kCompactBlockQueries, keep);
}

// Result of a `nearest` search: the row behind the smallest key, or 0 when no
// candidate was below the limit (csrc/cuda/nearest_cuda.cu:32,64 in the
// reference: `best_idx` starts at 0).
__device__ __forceinline__ void write_nearest(double best, int q, int x_begin,
                                              int64_t *out) {
  const bool found = best < SearchLimit<true>::empty();
  const uint32_t tie = (uint32_t)__double2loint(best);
  out[q] = found ? (int64_t)x_begin + (int64_t)nearest_rel(tie) : 0;
}

// Squared distance exactly as the reference accumulates it: direct
// differences, one fused multiply-add per component, ascending components.
template <int DIM, int NCX, int U>
__device__ __forceinline__ float exact_sqdist(const float (&cx)[NCX][U], int u,
                                              const float (&y)[DIM]) {
  const float d0 = cx[0][u] - y[0];
  float acc = d0 * d0;
#pragma unroll
  for (int c = 1; c < DIM; ++c) {
    const float dc = cx[c][u] - y[c];
    acc = __builtin_fmaf(dc, dc, acc);
  }
  return acc;
}

// ---------------------------------------------------------------------------
// Pre-filter of the Euclidean search.
//
// The exact distance costs 2 instructions per component (subtract, FMA).  The
// expanded form |x|^2 - 2 x.y (+ |y|^2, constant per query) costs one FMA per
// component but loses accuracy when |x - y| << |x|, so it cannot decide on its
// own.  It can REJECT: let u = 2^-24 and
//     t   = fma-chain(x_c * (-2 y_c)) started from  w = fl(|x|^2) * (1 - 32u)
//     cut = thresh * (1 + 32u) - fl(|y|^2) * (1 - 32u)   (rounded up)
// Every rounding error of the chain is bounded by 3.01u (2|x|^2 + |y|^2), the
// computed norms are within (1 +- u)^3 of the true ones and the exact distance
// d satisfies |x-y|^2 <= d (1 + 5.01u); together
//     d < thresh   ==>   t < cut,
// i.e. a candidate with t >= cut can never be accepted and is dropped after
// 3 FMAs + its share of a min3/compare.  Candidates with t < cut (the true
// neighbours plus a sliver of width ~4e-6 (|x|^2 + |y|^2 + thresh)) get the
// exact distance and are tested against thresh as before, so results stay
// bit-identical to the direct loop.  Points whose squared norm overflows or is
// not finite get w = -inf (always examined exactly); padding rows get
// w = +inf (never examined).
// ---------------------------------------------------------------------------
constexpr float kFilterDamp = 1.0f - 1.9073486328125e-06f; // 1 - 2^-19
constexpr float kFilterNormLimit = 1e30f;

__device__ __forceinline__ float filter_cut(float thresh, float ysq) {
  if (!(ysq <= kFilterNormLimit))
    return __builtin_inff(); // examine everything exactly
  const double eps = 1.9073486328125e-06; // 2^-19 = 32u
  const double c = (double)thresh * (1.0 + eps) - (double)ysq * (1.0 - eps) +
                   1e-37;
  float f = (float)c;
  if ((double)f < c) // round towards +inf
    f = __uint_as_float(f >= 0.0f ? __float_as_uint(f) + 1u
                                  : __float_as_uint(f) - 1u);
  return f;
}

// Waves per SIMD asked of the compiler where it would otherwise stop just
// above a register limit (512 / waves per lane): lists of 64 entries and, in
// up to four dimensions, of 100 came out at 270-282 registers - one wave -
// and run faster at two with a few dozen spilled words; lists of 32 entries
// with one query per lane at 133 instead of the 128 that four waves take.
template <int DIM, int K, int QPT>
constexpr int knn_lowd_min_waves() {
  return (K == 64 || (K == 100 && DIM <= 4)) ? 2
         : (K == 32 && QPT == 1 && DIM <= 4) ? 4
                                             : 1;
}

template <int DIM, int K, int QPT, bool COSINE>
__global__ __launch_bounds__(kBlock, (knn_lowd_min_waves<DIM, K, QPT>())) void
knn_lowd_kernel(KnnLowdParams p) {
  constexpr int TX = kLowdTileX;
  constexpr int QCAP = kLowdQueueCap;
  constexpr int U = kLowdGroup;
  // Euclidean search runs the expanded-form pre-filter (see above);
  // -DPCA_KNN_DIRECT builds the plain direct-difference loop instead
#ifdef PCA_KNN_DIRECT
  constexpr bool FILTER = false;
#else
  constexpr bool FILTER = !COSINE;
#endif
  // LDS holds one more component per point: |x| for the cosine distance, the
  // damped squared norm for the pre-filter
  constexpr int NC = (COSINE || FILTER) ? DIM + 1 : DIM;
  constexpr int PT = TX / kBlock; // points staged per thread
  constexpr int TQ = kBlock * QPT;

  __shared__ __attribute__((aligned(16))) float xs[2][NC][TX];
  // parked candidates: position inside the current tile
  __shared__ uint16_t queue[QPT][QCAP][kBlock];

  const int tid = threadIdx.x;
  const int total_tiles = p.work_start[p.num_segments];
  if (total_tiles == 0)
    return;
  // items are ordered slice-major: all tiles of slice 0 first, so that
  // neighbouring workgroups scan the same x rows and later slices start with
  // the bounds earlier ones have published
  const int chunk = blockIdx.x / total_tiles;
  const int tile = blockIdx.x - chunk * total_tiles;
  if (chunk >= p.num_chunks)
    return;
  const int seg = find_segment(p.work_start, p.num_segments, tile);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int q_base = y_begin + (tile - p.work_start[seg]) * TQ;
  const int d_in = p.d_in;
  const int k = p.k;

  // this item's slice of the segment: S equal parts, whole LDS tiles each
  const int seg_len = x_end - x_begin;
  const int chunk_len =
      ((seg_len + p.num_chunks - 1) / p.num_chunks + TX - 1) / TX * TX;
  const int c_begin = min(x_end, x_begin + chunk * chunk_len);
  const int c_count = min(x_end, c_begin + chunk_len) - c_begin;
  const int num_tiles = (c_count + TX - 1) / TX;

  // ---- per-lane query state -------------------------------------------
  int q[QPT];
  float yq[QPT][DIM];
  float ynorm[QPT];    // |y| (cosine)
  float ym2[QPT][DIM]; // -2 * y: the pre-filter's multipliers
  float ysq[QPT];      // |y|^2
  double best[QPT][K];
  float thresh[QPT]; // exact distances must be strictly below this
  float bound[QPT];  // what the scan loop compares against: thresh, or the
                     // pre-filter threshold derived from thresh and |y|^2
  float shared[QPT]; // strict bound derived from other slices' results
  float posted[QPT]; // smallest k-th distance seen in / written to tau
  int qcount[QPT];

  auto set_thresh = [&](int qi, float v) {
    thresh[qi] = v;
    bound[qi] = FILTER ? filter_cut(v, ysq[qi]) : v;
  };

#pragma unroll
  for (int qi = 0; qi < QPT; ++qi) {
    q[qi] = q_base + qi * kBlock + tid;
    const bool valid = q[qi] < y_end;
#pragma unroll
    for (int c = 0; c < DIM; ++c)
      yq[qi][c] =
          (valid && c < d_in) ? p.y[(size_t)q[qi] * d_in + c] : 0.0f;
    float s = yq[qi][0] * yq[qi][0];
#pragma unroll
    for (int c = 1; c < DIM; ++c)
      s = __builtin_fmaf(yq[qi][c], yq[qi][c], s);
    ysq[qi] = s;
    ynorm[qi] = __builtin_sqrtf(s);
#pragma unroll
    for (int c = 0; c < DIM; ++c)
      ym2[qi][c] = -2.0f * yq[qi][c];
#pragma unroll
    for (int j = 0; j < K; ++j)
      best[qi][j] = (j < K - k) ? lowest_key() : empty_key();
    set_thresh(qi, kKnnSentinel);
    shared[qi] = kKnnSentinel;
    posted[qi] = kKnnSentinel;
    qcount[qi] = 0;
  }

  // ---- tile staging ---------------------------------------------------
  float stage[PT][DIM];

  auto load_tile = [&](int t) {
#pragma unroll
    for (int r = 0; r < PT; ++r) {
      const int pos = t * TX + r * kBlock + tid;
      const size_t g = (size_t)c_begin + pos;
#pragma unroll
      for (int c = 0; c < DIM; ++c) {
        // rows past the slice end become +inf: their distance is inf or
        // NaN and never passes a `<` test
        float v = __builtin_inff();
        if (pos < c_count)
          v = c < d_in ? p.x[g * d_in + c] : 0.0f;
        stage[r][c] = v;
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int r = 0; r < PT; ++r) {
      const int pt = r * kBlock + tid;
#pragma unroll
      for (int c = 0; c < DIM; ++c)
        xs[buf][c][pt] = stage[r][c];
      if (COSINE || FILTER) {
        float s = stage[r][0] * stage[r][0];
#pragma unroll
        for (int c = 1; c < DIM; ++c)
          s = __builtin_fmaf(stage[r][c], stage[r][c], s);
        if (COSINE) {
          s = __builtin_sqrtf(s);
        } else {
          // rows past the slice end (+inf) must never pass the filter; rows
          // whose squared norm is not a moderate finite number always pass
          // it and are judged by the exact distance alone
          if (stage[r][0] == __builtin_inff())
            s = __builtin_inff();
          else if (!(s <= kFilterNormLimit))
            s = -__builtin_inff();
          else
            s = s * kFilterDamp;
        }
        xs[buf][NC - 1][pt] = s;
      }
    }
  };

  // Drains the parked candidates of query slot qi: all 64 lanes resolve their
  // s-th parked candidate together -- exact distance from the tile in LDS,
  // test against the current worst kept distance, insertion network.
  auto flush_one = [&](int qi, int buf, int g_base) {
    for (int s = 0; s < QCAP; ++s) {
      const bool has = s < qcount[qi];
      if (!__any(has))
        break;
      const int j = has ? (int)queue[qi][s][tid] : 0;
      float d;
      if (COSINE) {
        d = xs[buf][0][j] * yq[qi][0];
#pragma unroll
        for (int c = 1; c < DIM; ++c)
          d = __builtin_fmaf(xs[buf][c][j], yq[qi][c], d);
        d = d / (xs[buf][NC - 1][j] * ynorm[qi]);
        d = 1.0f - d;
      } else {
        const float d0 = xs[buf][0][j] - yq[qi][0];
        d = d0 * d0;
#pragma unroll
        for (int c = 1; c < DIM; ++c) {
          const float dc = xs[buf][c][j] - yq[qi][c];
          d = __builtin_fmaf(dc, dc, d);
        }
      }
      // the worst kept distance may have dropped since this one was parked;
      // kept keys at that distance have lower rows, so `<` is exact
      const bool ok = has && d < thresh[qi];
      if (!__any(ok))
        continue;
      const double key = ok ? make_key(d, (uint32_t)(g_base + j)) : empty_key();
      sorted_insert<K>(best[qi], key);
      set_thresh(qi, __builtin_fminf(key_dist(best[qi][K - 1]), shared[qi]));
    }
    qcount[qi] = 0;
  };

  // exchange of pruning bounds between the slices of a query
  auto sync_bounds = [&]() {
#pragma unroll
    for (int qi = 0; qi < QPT; ++qi) {
      if (q[qi] < y_end) {
        // a (slightly) negative cosine distance is published as 0: still an
        // upper bound, and non-negative floats order like their bit patterns
        const float own = __builtin_fmaxf(key_dist(best[qi][K - 1]), 0.0f);
        const float seen = __hip_atomic_load(&p.tau[q[qi]], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
        if (own < seen && own < posted[qi]) {
          __hip_atomic_fetch_min(reinterpret_cast<int *>(&p.tau[q[qi]]),
                                 (int)__float_as_uint(own), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
          posted[qi] = own;
        } else if (seen < posted[qi]) {
          posted[qi] = seen;
          // another slice's k-th distance: equality must still pass
          shared[qi] = next_up_positive(seen);
          set_thresh(qi, __builtin_fminf(thresh[qi], shared[qi]));
        }
      }
    }
  };

  if (num_tiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();

  for (int t = 0; t < num_tiles; ++t) {
    const int buf = t & 1;
    const bool more = t + 1 < num_tiles;
    if (more)
      load_tile(t + 1); // global loads in flight while this tile is scanned
    if (p.tau)
      sync_bounds();

    const int g_base = c_begin + t * TX;
    // whole pairs of groups; rows between the slice end and the tile end are
    // +inf padding
    const int limit =
        min(TX, (c_count - t * TX + 2 * U - 1) & ~(2 * U - 1));

    // one group of U candidates (component-major in `grp`) against this
    // lane's queries
    auto scan_group = [&](const float4 (&grp)[NC], int j) {
      float cx[NC][U];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        cx[c][0] = grp[c].x;
        cx[c][1] = grp[c].y;
        cx[c][2] = grp[c].z;
        cx[c][3] = grp[c].w;
      }
      // score of every (query, candidate) pair of the group; per query the
      // smallest of them decides whether anything needs a closer look
      float score[QPT][U];
      uint64_t any_hit = 0;
#pragma unroll
      for (int qi = 0; qi < QPT; ++qi) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          float acc;
          if (COSINE) {
            acc = cx[0][u] * yq[qi][0];
#pragma unroll
            for (int c = 1; c < DIM; ++c)
              acc = __builtin_fmaf(cx[c][u], yq[qi][c], acc);
            acc = acc / (cx[NC - 1][u] * ynorm[qi]);
            acc = 1.0f - acc;
          } else if (FILTER) {
            // damped |x|^2 - 2 x.y: one FMA per component
            acc = cx[NC - 1][u];
#pragma unroll
            for (int c = DIM - 1; c >= 0; --c)
              acc = __builtin_fmaf(cx[c][u], ym2[qi][c], acc);
          } else {
            acc = exact_sqdist<DIM>(cx, u, yq[qi]);
          }
          score[qi][u] = acc;
        }
        const float lo = __builtin_fminf(
            min3f(score[qi][0], score[qi][1], score[qi][2]), score[qi][3]);
        any_hit |= __ballot(lo < bound[qi]);
      }
      // One scalar branch on the hot path.  On the rare path the lanes that
      // passed are collected per pair with a ballot into scalar registers, so
      // finding the pairs with work is scalar code; only a pair some lane
      // passed runs vector instructions, and those just park the candidate's
      // position -- the exact distance is taken when the queue is drained, by
      // all lanes together.
      if (any_hit != 0) {
#pragma unroll
        for (int qi = 0; qi < QPT; ++qi) {
          uint64_t hit[U];
#pragma unroll
          for (int u = 0; u < U; ++u)
            hit[u] = __ballot(score[qi][u] < bound[qi]);
#pragma unroll
          for (int u = 0; u < U; ++u) {
            if (hit[u] != 0 && score[qi][u] < bound[qi]) {
              queue[qi][qcount[qi]][tid] = (uint16_t)(j + u);
              ++qcount[qi];
            }
          }
          if (__any(qcount[qi] > QCAP - U))
            flush_one(qi, buf, g_base);
        }
      }
    };
    auto read_group = [&](float4 (&grp)[NC], int j) {
#pragma unroll
      for (int c = 0; c < NC; ++c)
        grp[c] = *reinterpret_cast<const float4 *>(&xs[buf][c][j]);
    };

    // two register sets take turns, so that the LDS reads of the next group
    // are in flight while the current group is evaluated, without copies
    float4 ga[NC], gb[NC];
    read_group(ga, 0);
    for (int j = 0; j < limit; j += 2 * U) {
      read_group(gb, j + U);
      scan_group(ga, j);
      read_group(ga, min(j + 2 * U, TX - U));
      scan_group(gb, j + U);
    }
    // parked positions refer to this tile: resolve them before it goes away
#pragma unroll
    for (int qi = 0; qi < QPT; ++qi)
      flush_one(qi, buf, g_base);

    if (more)
      store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- results --------------------------------------------------------
  if (p.num_chunks == 1) {
#pragma unroll
    for (int qi = 0; qi < QPT; ++qi)
      if (q[qi] < y_end)
        write_dense<K>(best[qi], k, q[qi], p.out_idx, p.out_dist,
                       p.out_count);
  } else {
    // sorted keys of this slice, [item][slot][query of the tile]
    double *dst = p.partial + (size_t)blockIdx.x * k * TQ;
#pragma unroll
    for (int qi = 0; qi < QPT; ++qi) {
#pragma unroll
      for (int j = 0; j < K; ++j) {
        const int e = j - (K - k);
        if (e >= 0)
          dst[(size_t)e * TQ + qi * kBlock + tid] = best[qi][j];
      }
    }
  }
}

// Merges the sorted key lists of every query of a tile of TQ queries (one
// workgroup per tile; list c of the tile's query at position `pos` starts at
// partial[((c * tiles + tile) * k) * TQ + pos], consecutive slots TQ apart).
// p.num_chunks is the number of lists per query.
template <int K, int TQ, bool NEAREST = false>
__global__ __launch_bounds__(kBlock) void knn_merge_kernel(KnnLowdParams p) {
  if (p.gate != nullptr && *p.gate == 0)
    return;
  const int tid = threadIdx.x;
  const int total_tiles = p.work_start[p.num_segments];
  const int tile = blockIdx.x;
  if (tile >= total_tiles)
    return;
  const int seg = find_segment(p.work_start, p.num_segments, tile);
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int q_base = y_begin + (tile - p.work_start[seg]) * TQ;
  const int k = p.k;

  // TQ is a multiple of the wave size, so a wave is either all in or all out
  for (int pos = tid; pos < TQ; pos += kBlock) {
    const int q = q_base + pos;
    double best[K];
#pragma unroll
    for (int j = 0; j < K; ++j)
      best[j] = (j < K - k) ? lowest_key() : SearchLimit<NEAREST>::empty();
    for (int c = 0; c < p.num_chunks; ++c) {
      const double *src =
          p.partial + (size_t)(c * total_tiles + tile) * k * TQ + pos;
      for (int e = 0; e < k; ++e) {
        const double key = src[(size_t)e * TQ];
        // lists are ascending: once no lane's entry beats its worst kept
        // key, the rest of this list cannot either
        if (!__any(key < best[K - 1]))
          break;
        sorted_insert<K>(best, key);
      }
    }
    if (q < y_end && (p.redo_q == nullptr || p.redo_q[q] != 0)) {
      if constexpr (NEAREST) // (k = 1: the one real slot is the last)
        write_nearest(best[K - 1], q, p.ptr_x ? (int)p.ptr_x[seg] : 0,
                      p.out_nearest);
      else
        note_edges<K>(best, k, q,
                      write_dense<K>(best, k, q, p.out_idx, p.out_dist,
                                     p.out_count),
                      p.edge_sums, p.self_pos, p.kept);
    }
  }
}

// One (DIM, COSINE) slice of the dispatch table; each slice is instantiated in
// its own translation unit so the slices build in parallel.
template <int DIM, bool COSINE>
hipError_t launch_knn_lowd_dim(const KnnLowdParams &p,
                               const KnnLowdConfig &cfg, int tiles_bound,
                               hipStream_t stream);

template <int DIM, int KB, int QPT, bool COSINE>
void launch_knn_lowd_one(const KnnLowdParams &p, int tiles_bound,
                         hipStream_t stream) {
  hipLaunchKernelGGL((knn_lowd_kernel<DIM, KB, QPT, COSINE>),
                     dim3(tiles_bound * p.num_chunks), dim3(kBlock), 0, stream,
                     p);
}

// Two queries per lane are built for the Euclidean lists of up to 32 entries
// only (register budget; the cosine distance is a rarely used path).
template <int DIM, int KB, bool COSINE>
void launch_knn_lowd_qpt(const KnnLowdParams &p, int queries_per_lane,
                         int tiles_bound, hipStream_t stream) {
  if constexpr (!COSINE && KB <= 32) {
    if (queries_per_lane == 2) {
      launch_knn_lowd_one<DIM, KB, 2, COSINE>(p, tiles_bound, stream);
      return;
    }
  }
  launch_knn_lowd_one<DIM, KB, 1, COSINE>(p, tiles_bound, stream);
}

#define PCA_LOWD_CASE(D, KB, C)                                                \
  case KB:                                                                     \
    launch_knn_lowd_qpt<D, KB, C>(p, cfg.queries_per_lane, tiles_bound,        \
                                  stream);                                     \
    break;

#define PCA_LOWD_DEFINE_SLICE(DIM_, COSINE_)                                   \
  template <>                                                                  \
  hipError_t launch_knn_lowd_dim<DIM_, COSINE_>(                               \
      const KnnLowdParams &p, const KnnLowdConfig &cfg, int tiles_bound,       \
      hipStream_t stream) {                                                    \
    switch (cfg.kbucket) {                                                     \
      PCA_LOWD_CASE(DIM_, 8, COSINE_)                                          \
      PCA_LOWD_CASE(DIM_, 16, COSINE_)                                         \
      PCA_LOWD_CASE(DIM_, 24, COSINE_)                                         \
      PCA_LOWD_CASE(DIM_, 32, COSINE_)                                         \
      PCA_LOWD_CASE(DIM_, 48, COSINE_)                                         \
      PCA_LOWD_CASE(DIM_, 64, COSINE_)                                         \
      PCA_LOWD_CASE(DIM_, 100, COSINE_)                                        \
    default:                                                                   \
      return hipErrorInvalidValue;                                             \
    }                                                                          \
    return hipGetLastError();                                                  \
  }

} // namespace pca
