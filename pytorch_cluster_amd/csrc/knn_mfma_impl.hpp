// Feature-space kNN (8 < d <= 128, k <= 32, Euclidean or cosine) on the gfx950
// matrix cores, with results bit-identical to the reference's scalar loop
// (csrc/cuda/knn_cuda.cu:52-78).
//
// The distance of a (query, candidate) pair is |x|^2 + |y|^2 - 2 x.y.  The
// x.y of 32 candidates x 32 queries is one chain of v_mfma_f32_32x32x2_f32
// (fp32 in, fp32 accumulate) over the components -- a dense contraction, the
// one place on this path where the matrix cores apply.  The expanded form is
// not accurate enough to rank neighbours by itself (|x - y| can be far below
// |x|), so, exactly as in the low-dimensional kernel, it only REJECTS:
//
//     t   = fl(|x|^2) * (1 - eps) - 2 * mfma_dot(x, y)
//     cut = thresh * (1 + eps) - fl(|y|^2) * (1 - eps)      (rounded up)
//     eps = (d + 32) * 2^-22
//
// With the matrix-core dot product within 2 u |x||y| per accumulated term of
// the true one (u = 2^-24), norms accumulated with one FMA per component and
// the exact distance d_exact >= |x-y|^2 (1 - (d+2) u), a candidate with
// d_exact < thresh always has t < cut.  Candidates with t >= cut are dropped
// after one FMA and their share of a min/compare; the rest (true neighbours
// plus a sliver) are parked, and before the tile leaves LDS all 64 lanes take
// the exact distance of their parked candidates -- direct differences, one
// FMA per component in ascending order, the candidate's components from the
// tile in LDS, the query's from the B-operand registers of the lane and of
// its partner lane (v_permlane32_swap) -- and feed the usual (distance, row)
// key lists.  No memory latency is involved, and the vector work of one wave
// overlaps the matrix-core chain of the other wave on the same SIMD.
//
// The cosine distance 1 - x.y / (|x| |y|) uses the same matrix-core dot
// product: the filter value is 1 - mfma_dot * (1/|x|) * (1/|y|), within
// (3d + 40) u of the exactly evaluated distance, and is tested against
// thresh + (4d + 64) u; the exact value divides the sequentially accumulated
// dot product by the product of the two norms like the reference does
// (csrc/cuda/knn_cuda.cu:9-28,55-59).
//
// Mapping: a workgroup owns 128 queries of one segment (4 waves x 32) and one
// slice of the segment's x rows.  A = 32 candidates (rows i), B = 32 queries
// (columns j): lane l supplies A[l%32][2s + l/32] and B[2s + l/32][l%32] for
// step s, and receives, in 16 accumulator registers, the dot products of
// query l%32 with the 16 candidate rows 8*(v/4) + 4*(l/32) + v%4.  So the two
// lanes l and l+32 share a query and split its candidates; they hand each
// other every key they accept (v_permlane32_swap) and so keep one identical
// list.  The lists of a query's slices are merged by knn_merge_kernel and
// exchange their pruning bound through `tau` like the slices of the
// low-dimensional kernel do.
//
// The query operands stay in registers for the whole scan (d/2 per lane);
// candidate tiles stream through LDS, double-buffered, with the even and odd
// components of a row stored as two contiguous halves so that a lane's
// operands for 4 consecutive steps are one ds_read_b128.
#pragma once

#include "device_utils.hpp"
#include "knn_lowd_impl.hpp"
#include "launchers.hpp"

namespace pca {

constexpr int kMfmaQueries = 128; // queries per workgroup
constexpr int kMfmaRows = 32;     // candidates per tile
constexpr int kMfmaSyncTiles = 8; // tiles between exchanges of bounds

typedef float mfma_acc_t __attribute__((ext_vector_type(16)));

struct KnnMfmaParams {
  const float *x;
  const float *y;
  const int64_t *ptr_x;
  const int64_t *ptr_y;
  const float *x_sq; // [n] squared norms of the x rows (cosine: norms)
  int n, m, d, num_segments, k;
  const int *work_start; // [num_segments + 1] first 128-query tile per segment
  int num_chunks;        // slices of every segment's x rows
  float *tau;            // [m] shared pruning bounds
  double *partial;       // [num_chunks * tiles][k][128] keys
};

// Squared row norms, one FMA per component in ascending order.
__global__ __launch_bounds__(kBlock) void row_sqnorm_kernel(
    const float *__restrict__ x, int n, int d, float *__restrict__ out);

__device__ __forceinline__ float mfma_filter_cut(float thresh, float ysq,
                                                 double eps) {
  if (!(ysq <= kFilterNormLimit))
    return __builtin_inff(); // examine everything exactly
  const double c =
      (double)thresh * (1.0 + eps) - (double)ysq * (1.0 - eps) + 1e-30;
  float f = (float)c;
  if ((double)f < c) // round towards +inf
    f = __uint_as_float(f >= 0.0f ? __float_as_uint(f) + 1u
                                  : __float_as_uint(f) - 1u);
  return f;
}

// STEPS = padded d / 2: matrix-core steps per tile.
template <int STEPS, int K, bool COSINE>
__global__ __launch_bounds__(kBlock) void knn_mfma_kernel(KnnMfmaParams p) {
  constexpr int DP = 2 * STEPS;  // padded number of components
  constexpr int RS = DP + 4;     // LDS row stride (floats), keeps b128 reads
                                 // of 8 neighbouring rows on distinct banks
  constexpr int TR = kMfmaRows;
  constexpr int TQ = kMfmaQueries;
  constexpr int PER_THREAD = TR * DP / kBlock; // floats staged per thread

  __shared__ __attribute__((aligned(16))) float xs[2][TR][RS];
  // per row: damped squared norm (Euclidean) or 1 / norm (cosine) ...
  __shared__ __attribute__((aligned(16))) float wn[2][TR];
  // ... and, for the cosine distance, the norm itself
  __shared__ float xnorm[2][COSINE ? TR : 1];
  __shared__ uint8_t queue[16][kBlock]; // parked rows of the current tile

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int half = lane >> 5; // which components (parity) / which rows
  const int col = lane & 31;  // query column of B, candidate row of A

  const int total_tiles = p.work_start[p.num_segments];
  if (total_tiles == 0)
    return;
  const int chunk = blockIdx.x / total_tiles;
  const int tile = blockIdx.x - chunk * total_tiles;
  if (chunk >= p.num_chunks)
    return;
  const int seg = find_segment(p.work_start, p.num_segments, tile);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int q = y_begin + (tile - p.work_start[seg]) * TQ + wave * 32 + col;
  const bool valid = q < y_end;
  const int d = p.d;
  const int k = p.k;
  const float *yrow = p.y + (size_t)(valid ? q : y_begin) * d;

  const int seg_len = x_end - x_begin;
  const int chunk_len =
      ((seg_len + p.num_chunks - 1) / p.num_chunks + TR - 1) / TR * TR;
  const int c_begin = min(x_end, x_begin + chunk * chunk_len);
  const int c_end = min(x_end, c_begin + chunk_len);
  const int num_tiles = (c_end - c_begin + TR - 1) / TR;

  const double eps = (double)(d + 32) * (1.0 / 4194304.0); // (d+32) * 2^-22
  const float damp = (float)(1.0 - eps);

  // ---- per-lane state ---------------------------------------------------
  float yb[STEPS]; // B operands: this lane's parity of the query's components
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int c = 2 * s + half;
    yb[s] = (valid && c < d) ? yrow[c] : 0.0f;
  }
  float ysq = 0.0f;
  for (int c = 0; c < d; ++c)
    ysq = __builtin_fmaf(yrow[c], yrow[c], ysq);
  const float ynorm = __builtin_sqrtf(ysq);
  const float yrinv = 1.0f / ynorm;
  const float cos_margin = (float)(4 * d + 64) * 5.9604644775390625e-08f;

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - k) ? lowest_key() : empty_key();
  float thresh = kKnnSentinel;
  float bound =
      COSINE ? thresh + cos_margin : mfma_filter_cut(thresh, ysq, eps);
  float shared = kKnnSentinel;
  float posted = kKnnSentinel;

  auto set_thresh = [&](float v) {
    thresh = v;
    bound = COSINE ? v + cos_margin : mfma_filter_cut(v, ysq, eps);
  };

  // ---- tile staging -------------------------------------------------------
  // thread -> row tid / 8, components [seg8 * DP/8, (seg8 + 1) * DP/8)
  const int st_row = tid >> 3;
  const int st_c0 = (tid & 7) * (DP / 8);
  float stage[PER_THREAD];
  float stage_w = 0.0f;
  float stage_norm = 0.0f;

  auto load_tile = [&](int t) {
    const int g = c_begin + t * TR + st_row;
#pragma unroll
    for (int e = 0; e < PER_THREAD; ++e) {
      const int c = st_c0 + e;
      // rows past the slice end and padding components are zero; such rows
      // get w = +inf below and never pass the filter
      stage[e] = (g < c_end && c < d) ? p.x[(size_t)g * d + c] : 0.0f;
    }
    if (tid < TR) {
      const int gr = c_begin + t * TR + tid;
      float w = __builtin_inff();
      if (COSINE) {
        // filter value = 1 - dot * w * (1 / |y|); padding rows: w = 0 and
        // |x| = NaN, so that neither the filter (bound < 1 once a list is
        // full) nor the exact distance (NaN) can accept them
        float nx = __builtin_nanf("");
        w = 0.0f;
        if (gr < c_end) {
          nx = p.x_sq[gr];
          w = 1.0f / nx;
        }
        stage_norm = nx;
      } else if (gr < c_end) {
        const float s = p.x_sq[gr];
        // norms that are not moderate finite numbers always pass the filter
        w = (s <= kFilterNormLimit) ? s * damp : -__builtin_inff();
      }
      stage_w = w;
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int e = 0; e < PER_THREAD; ++e) {
      const int c = st_c0 + e;
      xs[buf][st_row][(c & 1) * STEPS + (c >> 1)] = stage[e];
    }
    if (tid < TR) {
      wn[buf][tid] = stage_w;
      if (COSINE)
        xnorm[buf][tid] = stage_norm;
    }
  };

  // Exchange of pruning bounds between the slices of a query: the k-th best
  // distance any slice has reached bounds the final k-th distance from above.
  auto sync_bounds = [&]() {
    if (valid) {
      // a (slightly) negative cosine distance is published as 0: still an
      // upper bound, and non-negative floats order like their bit patterns
      const float own = __builtin_fmaxf(key_dist(best[K - 1]), 0.0f);
      const float seen = __hip_atomic_load(&p.tau[q], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
      if (own < seen && own < posted) {
        __hip_atomic_fetch_min(reinterpret_cast<int *>(&p.tau[q]),
                               (int)__float_as_uint(own), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        posted = own;
      } else if (seen < posted) {
        posted = seen;
        // another slice's k-th distance: equality must still pass
        shared = next_up_positive(seen);
        set_thresh(__builtin_fminf(thresh, shared));
      }
    }
  };

  // Exact distances of the rows parked from the current tile, slot by slot
  // for all lanes together.
  int parked = 0;
  auto drain = [&](int buf, int g_base) {
    for (int s = 0; s < 16; ++s) {
      const bool has = s < parked;
      if (!__any(has))
        break;
      const int row = has ? (int)queue[s][tid] : 0;
      const float *xr = &xs[buf][row][0];
      float dist = 0.0f;
#pragma unroll
      for (int s4 = 0; s4 < STEPS / 4; ++s4) {
        const float4 xe = *reinterpret_cast<const float4 *>(xr + 4 * s4);
        const float4 xo =
            *reinterpret_cast<const float4 *>(xr + STEPS + 4 * s4);
        const float xev[4] = {xe.x, xe.y, xe.z, xe.w};
        const float xov[4] = {xo.x, xo.y, xo.z, xo.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // lanes 0-31 hold the even components of their query, lanes 32-63
          // the odd ones: the swap hands every lane both
          const auto both = __builtin_amdgcn_permlane32_swap(
              __float_as_uint(yb[4 * s4 + e]), __float_as_uint(yb[4 * s4 + e]),
              false, false);
          if (COSINE) {
            dist = __builtin_fmaf(xev[e], __uint_as_float(both[0]), dist);
            dist = __builtin_fmaf(xov[e], __uint_as_float(both[1]), dist);
          } else {
            const float d0 = xev[e] - __uint_as_float(both[0]);
            dist = __builtin_fmaf(d0, d0, dist);
            const float d1 = xov[e] - __uint_as_float(both[1]);
            dist = __builtin_fmaf(d1, d1, dist);
          }
        }
      }
      if (COSINE) {
        dist = dist / (xnorm[buf][row] * ynorm);
        dist = 1.0f - dist;
      }
      // The two lanes that share a query keep ONE list between them: each
      // hands its key to the other, both insert both, so the lists stay
      // identical and the pruning bound is the k-th distance over all 32 rows
      // of a tile, not over a lane's 16.  Rows of one lane reach its list in
      // ascending order but the partner's rows interleave, so equality with
      // the worst kept distance must pass (`<=`): the key order settles ties.
      const bool ok = has && valid && dist <= thresh;
      if (!__any(ok))
        continue;
      const double key =
          ok ? make_key(dist, (uint32_t)(g_base + row)) : empty_key();
      const auto hi = __builtin_amdgcn_permlane32_swap(
          (unsigned)__double2hiint(key), (unsigned)__double2hiint(key), false,
          false);
      const auto lo = __builtin_amdgcn_permlane32_swap(
          (unsigned)__double2loint(key), (unsigned)__double2loint(key), false,
          false);
      // element 0 = the lower lane's key, element 1 = the upper lane's
      const double key_a = __hiloint2double((int)hi[0], (int)lo[0]);
      const double key_b = __hiloint2double((int)hi[1], (int)lo[1]);
      sorted_insert<K>(best, key_a);
      sorted_insert<K>(best, key_b);
      set_thresh(__builtin_fminf(key_dist(best[K - 1]), shared));
    }
    parked = 0;
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
      load_tile(t + 1);
    if ((t % kMfmaSyncTiles) == 0)
      sync_bounds();
    const int g_base = c_begin + t * TR;

    // ---- 32 x 32 dot products on the matrix cores -----------------------
    mfma_acc_t acc = {0};
    const float *arow = &xs[buf][col][half * STEPS];
#pragma unroll
    for (int s4 = 0; s4 < STEPS / 4; ++s4) {
      const float4 a = *reinterpret_cast<const float4 *>(arow + 4 * s4);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, yb[4 * s4 + 0], acc, 0,
                                                 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, yb[4 * s4 + 1], acc, 0,
                                                 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, yb[4 * s4 + 2], acc, 0,
                                                 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, yb[4 * s4 + 3], acc, 0,
                                                 0, 0);
    }

    // ---- filter ---------------------------------------------------------
    // accumulator v holds candidate row 8 * (v / 4) + 4 * half + v % 4
    float score[16];
    float lo = __builtin_inff();
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const float4 w =
          *reinterpret_cast<const float4 *>(&wn[buf][8 * v4 + 4 * half]);
      if (COSINE) {
        score[4 * v4 + 0] = __builtin_fmaf(-acc[4 * v4 + 0], w.x * yrinv, 1.0f);
        score[4 * v4 + 1] = __builtin_fmaf(-acc[4 * v4 + 1], w.y * yrinv, 1.0f);
        score[4 * v4 + 2] = __builtin_fmaf(-acc[4 * v4 + 2], w.z * yrinv, 1.0f);
        score[4 * v4 + 3] = __builtin_fmaf(-acc[4 * v4 + 3], w.w * yrinv, 1.0f);
      } else {
        score[4 * v4 + 0] = __builtin_fmaf(-2.0f, acc[4 * v4 + 0], w.x);
        score[4 * v4 + 1] = __builtin_fmaf(-2.0f, acc[4 * v4 + 1], w.y);
        score[4 * v4 + 2] = __builtin_fmaf(-2.0f, acc[4 * v4 + 2], w.z);
        score[4 * v4 + 3] = __builtin_fmaf(-2.0f, acc[4 * v4 + 3], w.w);
      }
      lo = __builtin_fminf(
          lo, __builtin_fminf(min3f(score[4 * v4], score[4 * v4 + 1],
                                    score[4 * v4 + 2]),
                              score[4 * v4 + 3]));
    }

    if (__ballot(lo < bound) != 0) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        if (__ballot(score[v] < bound) != 0 && score[v] < bound) {
          queue[parked][tid] = (uint8_t)(8 * (v / 4) + 4 * half + (v % 4));
          ++parked;
        }
      }
      drain(buf, g_base);
    }

    if (more)
      store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- sorted keys of this slice (both lanes of a pair hold the same list)
  if (half == 0) {
    const size_t list = (size_t)chunk * total_tiles + tile;
    double *dst = p.partial + list * k * TQ + wave * 32 + col;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int e = j - (K - k);
      if (e >= 0)
        dst[(size_t)e * TQ] = best[j];
    }
  }
}

} // namespace pca
