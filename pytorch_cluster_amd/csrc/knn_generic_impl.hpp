// Brute-force kNN for fp32 points of any dimension (used for d > 8) on gfx950.
//
// Same result contract and the same selection machinery as the
// low-dimensional kernel (knn_lowd_impl.hpp): one query per lane, a sorted
// register list of K 64-bit (distance, row) keys, candidates pre-filtered
// against the current worst distance and parked in a per-lane LDS queue.
// What differs is the distance evaluation, because a query row no longer fits
// in registers:
//
//   * an x tile is TG candidates with all their components, row-major in LDS
//     (components are streamed in slabs of at most kSlab when d is larger);
//   * each lane keeps TG partial sums; for every chunk of 16 components it
//     loads that chunk of its query row once and walks the TG candidates,
//     reading their components as ds_read_b128 broadcasts;
//   * a partial sum receives one fused multiply-add per component, in
//     ascending component order, exactly like the reference's scalar loop
//     (csrc/cuda/knn_cuda.cu:55-64), so results are bit-identical to it.
//
// The cosine distance needs |x| of every candidate: the row norms of x are
// computed once by row_norm_kernel into the workspace.
#pragma once

#include "device_utils.hpp"
#include "launchers.hpp"

namespace pca {

constexpr int kGenTile = 32;    // candidates per LDS tile
constexpr int kGenChunk = 16;   // query components held in registers
constexpr int kGenSlab = 256;   // components of a tile resident in LDS
constexpr int kGenQueueCap = 12;

template <int K, bool COSINE>
__global__ __launch_bounds__(kBlock) void knn_generic_kernel(
    const float *__restrict__ x, const float *__restrict__ y,
    const int64_t *__restrict__ ptr_x, const int64_t *__restrict__ ptr_y,
    const float *__restrict__ x_norm, int n, int m, int d, int num_segments,
    int k, const int *__restrict__ work_start, int grid,
    int *__restrict__ out_idx, float *__restrict__ out_dist,
    int *__restrict__ out_count, const int *__restrict__ gate,
    const int *__restrict__ redo_q, int num_chunks,
    double *__restrict__ partial) {
  constexpr int TG = kGenTile;
  constexpr int CH = kGenChunk;
  constexpr int QCAP = kGenQueueCap;

  __shared__ __attribute__((aligned(16))) float xs[TG][kGenSlab];
  __shared__ float xn[TG];
  __shared__ double queue[QCAP][kBlock];

  // (second pass behind another search: only when that search flagged
  // queries, and only the flagged ones)
  if (gate != nullptr && *gate == 0)
    return;
  const int tid = threadIdx.x;
  // work item = (slice of the segment's x rows, tile of queries)
  const int item = PCA_TILE_OF_BLOCK(blockIdx.x, grid);
  const int total_tiles = work_start[num_segments];
  if (total_tiles == 0)
    return;
  const int chunk = item / total_tiles;
  const int tile = item - chunk * total_tiles;
  if (chunk >= num_chunks)
    return;
  const int seg = find_segment(work_start, num_segments, tile);
  const int x_begin = ptr_x ? (int)ptr_x[seg] : 0;
  const int x_end = ptr_x ? (int)ptr_x[seg + 1] : n;
  const int y_begin = ptr_y ? (int)ptr_y[seg] : 0;
  const int y_end = ptr_y ? (int)ptr_y[seg + 1] : m;
  const int q = y_begin + (tile - work_start[seg]) * kBlock + tid;
  bool valid = q < y_end;
  if (redo_q != nullptr) {
    valid = valid && redo_q[q] != 0;
    if (!__syncthreads_or(valid))
      return;
  }
  const float *yrow = y + (size_t)(valid ? q : y_begin) * d;
  const int seg_len = x_end - x_begin;
  const int chunk_len =
      ((seg_len + num_chunks - 1) / num_chunks + TG - 1) / TG * TG;
  const int c_begin = min(x_end, x_begin + chunk * chunk_len);
  const int c_end = min(x_end, c_begin + chunk_len);

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - k) ? lowest_key() : empty_key();
  float thresh = kKnnSentinel;
  int qcount = 0;

  float y_norm = 0.0f;
  if (COSINE) {
    float s = 0.0f;
    for (int c = 0; c < d; ++c)
      s = __builtin_fmaf(yrow[c], yrow[c], s);
    y_norm = __builtin_sqrtf(s);
  }

  auto flush = [&]() {
    for (int s = 0; s < QCAP; ++s) {
      const bool has = s < qcount;
      if (!__any(has))
        break;
      double key = empty_key();
      if (has)
        key = queue[s][tid];
      if (!__any(key < best[K - 1]))
        continue;
      sorted_insert<K>(best, key);
    }
    thresh = key_dist(best[K - 1]);
    qcount = 0;
  };

  for (int base = c_begin; base < c_end; base += TG) {
    const int rows = min(TG, c_end - base);
    float acc[TG];
#pragma unroll
    for (int j = 0; j < TG; ++j)
      acc[j] = 0.0f;

    for (int slab = 0; slab < d; slab += kGenSlab) {
      const int width = min(kGenSlab, d - slab);
      const int width4 = (width + 3) & ~3;
      __syncthreads(); // previous slab / tile fully consumed
      // stage rows [base, base+rows) x components [slab, slab+width); pad
      // missing rows with +inf and the tail of the last float4 with zeros
      for (int i = tid; i < TG * width4; i += kBlock) {
        const int r = i / width4;
        const int c = i - r * width4;
        float v = 0.0f;
        if (c < width)
          v = r < rows ? x[(size_t)(base + r) * d + slab + c]
                       : __builtin_inff();
        xs[r][c] = v;
      }
      if (COSINE && slab == 0 && tid < TG)
        xn[tid] = tid < rows ? x_norm[base + tid] : __builtin_inff();
      __syncthreads();

      for (int c0 = 0; c0 < width; c0 += CH) {
        float yv[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c)
          yv[c] = (c0 + c < width) ? yrow[slab + c0 + c] : 0.0f;
        // number of float4 groups of this chunk that hold real components
        const int groups = min(CH / 4, (width4 - c0) / 4);
#pragma unroll
        for (int j = 0; j < TG; ++j) {
#pragma unroll
          for (int g = 0; g < CH / 4; ++g) {
            if (g < groups) {
              const float4 v =
                  *reinterpret_cast<const float4 *>(&xs[j][c0 + 4 * g]);
              const float xv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                if (COSINE) {
                  acc[j] = __builtin_fmaf(xv[e], yv[4 * g + e], acc[j]);
                } else {
                  const float dc = xv[e] - yv[4 * g + e];
                  acc[j] = __builtin_fmaf(dc, dc, acc[j]);
                }
              }
            }
          }
        }
      }
    }

    // distances of this tile -> filter -> queue
    bool pass = false;
#pragma unroll
    for (int j = 0; j < TG; ++j) {
      if (COSINE) {
        acc[j] = acc[j] / (xn[j] * y_norm);
        acc[j] = 1.0f - acc[j];
      }
      pass |= acc[j] < thresh;
    }
    if (__any(pass)) {
#pragma unroll
      for (int j0 = 0; j0 < TG; j0 += 4) {
        bool full = false;
#pragma unroll
        for (int j = j0; j < j0 + 4; ++j) {
          if (acc[j] < thresh) {
            queue[qcount][tid] = make_key(acc[j], (uint32_t)(base + j));
            ++qcount;
          }
        }
        full = qcount > QCAP - 4;
        if (__any(full))
          flush();
      }
    }
  }
  flush();

  if (num_chunks > 1) {
    // sorted keys of this slice, [item][slot][query of the tile]; the merge
    // (knn_merge_kernel) unites the slices
    double *dst = partial + (size_t)(chunk * total_tiles + tile) * k * kBlock + tid;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int e = j - (K - k);
      if (e >= 0)
        dst[(size_t)e * kBlock] = best[j];
    }
    return;
  }
  if (valid) {
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
  }
}

template <bool COSINE>
hipError_t launch_knn_generic_metric(const SearchInput &in, int k, int kbucket,
                                     const float *x_norm,
                                     const int *work_start, int grid_bound,
                                     const DenseResult &out,
                                     hipStream_t stream, const int *gate,
                                     const int *redo_q, int num_chunks,
                                     double *partial);

#define PCA_GENERIC_CASE(KB, C)                                                \
  case KB:                                                                     \
    hipLaunchKernelGGL((knn_generic_kernel<KB, C>), dim3(grid), dim3(kBlock),  \
                       0, stream, (const float *)in.x, (const float *)in.y,    \
                       in.ptr_x, in.ptr_y, x_norm, in.n, in.m, in.d,           \
                       in.num_segments, k, work_start, grid, out.idx,          \
                       out.dist, out.count, gate, redo_q, num_chunks,          \
                       partial);                                               \
    break;

#define PCA_GENERIC_DEFINE(C)                                                  \
  template <>                                                                  \
  hipError_t launch_knn_generic_metric<C>(                                     \
      const SearchInput &in, int k, int kbucket, const float *x_norm,          \
      const int *work_start, int grid_bound, const DenseResult &out,           \
      hipStream_t stream, const int *gate, const int *redo_q,                  \
      int num_chunks, double *partial) {                                       \
    const int grid = (grid_bound * num_chunks + 7) & ~7;                       \
    switch (kbucket) {                                                         \
      PCA_GENERIC_CASE(8, C)                                                   \
      PCA_GENERIC_CASE(16, C)                                                  \
      PCA_GENERIC_CASE(24, C)                                                  \
      PCA_GENERIC_CASE(32, C)                                                  \
      PCA_GENERIC_CASE(48, C)                                                  \
      PCA_GENERIC_CASE(64, C)                                                  \
      PCA_GENERIC_CASE(100, C)                                                 \
    default:                                                                   \
      return hipErrorInvalidValue;                                             \
    }                                                                          \
    return hipGetLastError();                                                  \
  }

} // namespace pca
