// Brute-force kNN for low-dimensional fp32 points (d <= 8) on gfx950.
//
// Computes what knn_kernel of the reference computes
// (csrc/cuda/knn_cuda.cu:30-84: one thread per query, linear scan of the
// query's segment of x, sorted insertion list), with a different machine
// mapping:
//
//   * one workgroup (4 waves) owns a tile of 256 * QPT queries of ONE segment
//     (found from the work_start table, never crossing a segment boundary);
//     each lane owns QPT queries, their coordinates live in registers;
//   * the segment's x rows stream through LDS in tiles of TX points, staged
//     with coalesced global loads, double-buffered, stored component-major so
//     that the inner loop reads four candidates per ds_read_b128 and every
//     lane of the wave reads the same address (broadcast, no bank conflicts);
//   * distances use direct differences and one fused multiply-add per
//     dimension in ascending dimension order -- bit-identical to
//     `dist += (x - y) * (x - y)` as a GPU compiler contracts it;
//   * the running top-k of a query is a register-resident ascending list of K
//     64-bit (distance, row) keys (see device_utils.hpp), updated with a
//     branch-free min/max insertion network;
//   * candidates are pre-filtered against the list's current worst distance;
//     the few that pass are parked in a small per-lane LDS queue and the
//     insertion network runs only when some lane's queue is nearly full, so
//     the wave does not pay K slots of insertion for every lane that accepts
//     a candidate.
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
constexpr int kLowdQueueCap = 12;
constexpr int kLowdGroup = 4; // candidates per inner-loop step

template <int DIM, int K, int QPT, bool COSINE>
__global__ __launch_bounds__(kBlock) void knn_lowd_kernel(
    const float *__restrict__ x, const float *__restrict__ y,
    const int64_t *__restrict__ ptr_x, const int64_t *__restrict__ ptr_y,
    int n, int m, int d_in, int num_segments, int k,
    const int *__restrict__ work_start, int grid, int *__restrict__ out_idx,
    float *__restrict__ out_dist, int *__restrict__ out_count) {
  constexpr int TX = kLowdTileX;
  constexpr int QCAP = kLowdQueueCap;
  constexpr int U = kLowdGroup;
  constexpr int NC = COSINE ? DIM + 1 : DIM; // + |x| for the cosine distance
  constexpr int PT = TX / kBlock;            // points staged per thread
  constexpr int TQ = kBlock * QPT;

  __shared__ __attribute__((aligned(16))) float xs[2][NC][TX];
  __shared__ double queue[QPT][QCAP][kBlock];

  const int tid = threadIdx.x;
  const int tile = xcd_swizzle(blockIdx.x, grid);
  if (tile >= work_start[num_segments])
    return;
  const int seg = find_segment(work_start, num_segments, tile);
  const int x_begin = ptr_x ? (int)ptr_x[seg] : 0;
  const int x_end = ptr_x ? (int)ptr_x[seg + 1] : n;
  const int y_begin = ptr_y ? (int)ptr_y[seg] : 0;
  const int y_end = ptr_y ? (int)ptr_y[seg + 1] : m;
  const int q_base = y_begin + (tile - work_start[seg]) * TQ;

  // ---- per-lane query state -------------------------------------------
  int q[QPT];
  float yq[QPT][DIM];
  float ynorm[QPT];
  double best[QPT][K];
  float thresh[QPT];
  int qcount[QPT];
#pragma unroll
  for (int qi = 0; qi < QPT; ++qi) {
    q[qi] = q_base + qi * kBlock + tid;
    const bool valid = q[qi] < y_end;
#pragma unroll
    for (int c = 0; c < DIM; ++c)
      yq[qi][c] = (valid && c < d_in) ? y[(size_t)q[qi] * d_in + c] : 0.0f;
    if (COSINE) {
      float s = yq[qi][0] * yq[qi][0];
#pragma unroll
      for (int c = 1; c < DIM; ++c)
        s = __builtin_fmaf(yq[qi][c], yq[qi][c], s);
      ynorm[qi] = __builtin_sqrtf(s);
    }
#pragma unroll
    for (int j = 0; j < K; ++j)
      best[qi][j] = (j < K - k) ? lowest_key() : empty_key();
    thresh[qi] = kKnnSentinel;
    qcount[qi] = 0;
  }

  // ---- tile staging ---------------------------------------------------
  const int seg_len = x_end - x_begin;
  const int num_tiles = (seg_len + TX - 1) / TX;
  float stage[PT][DIM];

  auto load_tile = [&](int t) {
#pragma unroll
    for (int r = 0; r < PT; ++r) {
      const int g = x_begin + t * TX + r * kBlock + tid;
#pragma unroll
      for (int c = 0; c < DIM; ++c) {
        // rows past the segment end become +inf: their distance is inf or
        // NaN and never passes the `< thresh` filter
        float v = __builtin_inff();
        if (g < x_end)
          v = c < d_in ? x[(size_t)g * d_in + c] : 0.0f;
        stage[r][c] = v;
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int r = 0; r < PT; ++r) {
      const int p = r * kBlock + tid;
#pragma unroll
      for (int c = 0; c < DIM; ++c)
        xs[buf][c][p] = stage[r][c];
      if (COSINE) {
        float s = stage[r][0] * stage[r][0];
#pragma unroll
        for (int c = 1; c < DIM; ++c)
          s = __builtin_fmaf(stage[r][c], stage[r][c], s);
        xs[buf][NC - 1][p] = __builtin_sqrtf(s);
      }
    }
  };

  auto flush = [&]() {
#pragma unroll
    for (int qi = 0; qi < QPT; ++qi) {
      for (int s = 0; s < QCAP; ++s) {
        const bool has = s < qcount[qi];
        if (!__any(has))
          break;
        double key = empty_key();
        if (has)
          key = queue[qi][s][tid];
        // the worst kept key may have dropped since this one was parked
        if (!__any(key < best[qi][K - 1]))
          continue;
        sorted_insert<K>(best[qi], key);
      }
      thresh[qi] = key_dist(best[qi][K - 1]);
      qcount[qi] = 0;
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

    const int g_base = x_begin + t * TX;
    const int limit = min(TX, (x_end - g_base + U - 1) & ~(U - 1));
    for (int j = 0; j < limit; j += U) {
      float cx[NC][U];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const float4 v = *reinterpret_cast<const float4 *>(&xs[buf][c][j]);
        cx[c][0] = v.x;
        cx[c][1] = v.y;
        cx[c][2] = v.z;
        cx[c][3] = v.w;
      }
      float dist[QPT][U];
      bool pass = false;
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
          } else {
            const float d0 = cx[0][u] - yq[qi][0];
            acc = d0 * d0;
#pragma unroll
            for (int c = 1; c < DIM; ++c) {
              const float dc = cx[c][u] - yq[qi][c];
              acc = __builtin_fmaf(dc, dc, acc);
            }
          }
          dist[qi][u] = acc;
        }
        const float lo =
            __builtin_fminf(min3f(dist[qi][0], dist[qi][1], dist[qi][2]),
                            dist[qi][3]);
        pass |= lo < thresh[qi];
      }
      if (__any(pass)) {
        bool full = false;
#pragma unroll
        for (int qi = 0; qi < QPT; ++qi) {
#pragma unroll
          for (int u = 0; u < U; ++u) {
            if (dist[qi][u] < thresh[qi]) {
              queue[qi][qcount[qi]][tid] =
                  make_key(dist[qi][u], (uint32_t)(g_base + j + u));
              ++qcount[qi];
            }
          }
          full |= qcount[qi] > QCAP - U;
        }
        if (__any(full))
          flush();
      }
    }

    if (more)
      store_tile(buf ^ 1);
    __syncthreads();
  }
  flush();

  // ---- results --------------------------------------------------------
#pragma unroll
  for (int qi = 0; qi < QPT; ++qi) {
    if (q[qi] >= y_end)
      continue;
    const size_t row = (size_t)q[qi] * k;
    int found = 0;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int e = j - (K - k);
      if (e >= 0 && best[qi][j] < empty_key()) {
        out_idx[row + e] = key_row(best[qi][j]);
        if (out_dist)
          out_dist[row + e] = key_dist(best[qi][j]);
        ++found;
      }
    }
    out_count[q[qi]] = found;
  }
}

// One (DIM, COSINE) slice of the dispatch table; each slice is instantiated in
// its own translation unit so the slices build in parallel.
template <int DIM, bool COSINE>
hipError_t launch_knn_lowd_dim(const SearchInput &in, int k,
                               const KnnLowdConfig &cfg, const int *work_start,
                               int grid_bound, const DenseResult &out,
                               hipStream_t stream);

template <int DIM, int KB, int QPT, bool COSINE>
void launch_knn_lowd_one(const SearchInput &in, int k, const int *work_start,
                         int grid, const DenseResult &out,
                         hipStream_t stream) {
  hipLaunchKernelGGL((knn_lowd_kernel<DIM, KB, QPT, COSINE>), dim3(grid),
                     dim3(kBlock), 0, stream, (const float *)in.x,
                     (const float *)in.y, in.ptr_x, in.ptr_y, in.n, in.m, in.d,
                     in.num_segments, k, work_start, grid, out.idx, out.dist,
                     out.count);
}

// Two queries per lane are built for the Euclidean lists of up to 32 entries
// only (register budget; the cosine distance is a rarely used path).
template <int DIM, int KB, bool COSINE>
void launch_knn_lowd_qpt(const SearchInput &in, int k, int queries_per_lane,
                         const int *work_start, int grid,
                         const DenseResult &out, hipStream_t stream) {
  if constexpr (!COSINE && KB <= 32) {
    if (queries_per_lane == 2) {
      launch_knn_lowd_one<DIM, KB, 2, COSINE>(in, k, work_start, grid, out,
                                              stream);
      return;
    }
  }
  launch_knn_lowd_one<DIM, KB, 1, COSINE>(in, k, work_start, grid, out,
                                          stream);
}

#define PCA_LOWD_CASE(D, KB, C)                                                     \
  case KB:                                                                     \
    launch_knn_lowd_qpt<D, KB, C>(in, k, cfg.queries_per_lane, work_start,    \
                                  grid, out, stream);                          \
    break;

#define PCA_LOWD_DEFINE_SLICE(DIM_, COSINE_)                                   \
  template <>                                                                  \
  hipError_t launch_knn_lowd_dim<DIM_, COSINE_>(                               \
      const SearchInput &in, int k, const KnnLowdConfig &cfg,                  \
      const int *work_start, int grid_bound, const DenseResult &out,           \
      hipStream_t stream) {                                                    \
    const int grid = (grid_bound + 7) & ~7;                                    \
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
