// Feature-space kNN (8 < d <= 134, k <= 32, Euclidean or cosine) on the gfx950
// matrix cores, with results bit-identical to the reference's scalar loop
// (csrc/cuda/knn_cuda.cu:52-78).
//
// Filter.  The matrix cores decide which candidates are LOOKED AT; every
// distance that is kept is evaluated exactly as the reference does.  For the
// Euclidean metric the filter value of a (query, candidate) pair is
//     t = w - 2 x.y,      w = fl(|x|^2) (1 - eps),
// the dot product of the augmented rows (x, w) and (-2 y, 1): one chain of
// v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate) over the components for 32
// candidates x 32 queries.  The last component carries (1) . (-cut),
//     cut = thresh (1 + eps) - fl(|y|^2) (1 - eps)   (rounded up),
//     eps = (d + 32) 2^-22,
// so the SIGN of a result says whether the candidate can still have an exact
// distance below thresh: with the accumulated products within 2 u |x||y| per
// term of the true ones (u = 2^-24), norms accumulated with one FMA per
// component and the exact chain d_exact >= |x-y|^2 (1 - (d + 2) u), a
// candidate with d_exact < thresh always has t - cut < 0.  Rows whose squared
// norm is not a moderate finite number enter with zero coordinates and
// w = -inf (always looked at), padding rows with w = NaN (never), queries with
// such a norm use cut = +inf with zero coordinates (look at every real row).
//
// The cosine distance 1 - x.y / (|x| |y|) uses the same chain on normalised
// rows: (x / |x|, 1) . (-y / |y|, 1) = 1 - cos, within (4 d + 72) u of the
// exactly evaluated distance; the cut is thresh + that margin.
// Rows of norm 0 or NaN have a NaN distance in the reference and are padding
// here; a row or query of infinite norm is looked at / looks at everything.
//
// Selection.  A lane gathers the 16 sign bits of a 32-row step with funnel
// shifts and, if any is set, parks (step, mask) in its LDS queue -- one write.
// Every kMfmaDrainSteps steps a wave resolves what its lanes have parked,
// densely: the parked (query, row) pairs of all 64 lanes are compacted into
// one list, lane i takes pair i, 64 + i, ... and evaluates its exact distance
// -- direct differences, one FMA per component in ascending order
// (csrc/cuda/knn_cuda.cu:9-28,55-66), both rows streamed from global memory
// (they are L2 resident) -- and hands the (distance, row) key back through
// LDS to the lane that owns the query, which runs the insertion network.  An
// exact distance costs ~2 d vector instructions for the whole wave whether 1
// or 64 lanes have work, so the dense list is what keeps the re-rank a few
// percent of the matrix-core time even when a handful of queries collect most
// of the candidates.
//
// Mapping: a workgroup owns 128 queries of one segment (4 waves x 32) and one
// slice of the segment's x rows.  A = 32 candidates (rows i), B = 32 queries
// (columns j): lane l supplies A[l%32][2s + l/32] and B[2s + l/32][l%32] for
// step s, and receives, in 16 accumulator registers, the results of query
// l%32 against the 16 candidate rows 8*(v/4) + 4*(l/32) + v%4.  So lanes l and
// l+32 share a query and split its candidates; the lower lane keeps the
// query's list and collects the keys of both lanes' rows in ascending row
// order (so the list's k-th distance is a strict bound), the upper lane
// filters with the same bound.  The lists of a query's slices are merged by
// knn_merge_kernel and exchange their pruning bound through `tau` like the
// slices of the low-dimensional kernels do.
//
// The query operands stay in registers for the whole scan (d/2 + 1 per lane);
// candidate tiles stream through LDS, double-buffered, with the even and odd
// components of a row stored as two contiguous halves so that a lane's
// operands for 4 consecutive steps are one ds_read_b128.
#pragma once

#include "device_utils.hpp"
#include "knn_lowd_impl.hpp"
#include "launchers.hpp"

namespace pca {

constexpr int kMfmaQueries = 128;   // queries per workgroup
constexpr int kMfmaRows = 32;       // candidates per step
constexpr int kMfmaDrainSteps = 16; // steps between drains (= queue entries)
constexpr int kMfmaPassPairs = 256; // pairs a wave evaluates per pass

typedef float mfma_acc_t __attribute__((ext_vector_type(16)));

struct KnnMfmaParams {
  const float *x;
  const float *y;
  const int64_t *ptr_x;
  const int64_t *ptr_y;
  const float *x_sq;   // [n] squared norms of the x rows (cosine: norms)
  const float *y_norm; // [m] norms of the y rows (cosine only)
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

// A lane's walk over the rows it has parked, in ascending order.
struct MfmaWalk {
  int taken;        // queue entries started
  uint32_t pending; // rows of the current entry still to visit
  int base;         // the lane's first row of that entry's step
};

// STEPS = matrix-core steps per 32 rows: 2 STEPS >= d + 2 components (the
// coordinates, w, and the last one for the cut).
template <int STEPS, int K, bool COSINE>
__global__ __launch_bounds__(kBlock) void knn_mfma_kernel(KnnMfmaParams p) {
  constexpr int DP = 2 * STEPS; // padded number of components (with w)
  constexpr int RS = DP + 4;    // LDS row stride (floats), keeps b128 reads
                                // of 8 neighbouring rows on distinct banks
  constexpr int TR = kMfmaRows;
  constexpr int TQ = kMfmaQueries;
  constexpr int PER_THREAD = TR * DP / kBlock; // floats staged per thread
  constexpr int QCAP = kMfmaDrainSteps;
  constexpr int CAP = kMfmaPassPairs;
  static_assert(STEPS % 4 == 0 && (TR * DP) % kBlock == 0, "tile shape");

  __shared__ __attribute__((aligned(16))) float xs[2][TR][RS];
  // parked steps: (step within the batch << 16) | mask of the lane's rows
  __shared__ uint32_t queue[QCAP][kBlock];
  // dense re-rank, per wave: (query, row) pairs and their keys
  __shared__ int2 pairs[kBlock / kWave][CAP];
  __shared__ double results[kBlock / kWave][CAP];

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
  // the slice: rows c_begin + position, position < c_count
  const int c_begin = min(x_end, x_begin + chunk * chunk_len);
  const int c_count = min(x_end, c_begin + chunk_len) - c_begin;
  const int num_steps = (c_count + TR - 1) / TR;

  const double eps = (double)(d + 32) * (1.0 / 4194304.0); // (d+32) * 2^-22
  const float damp = (float)(1.0 - eps);
  const float cos_margin = (float)(4 * d + 72) * 5.9604644775390625e-08f;

  // ---- per-lane query state ---------------------------------------------
  float ysq = 0.0f;
  for (int c = 0; c < d; ++c)
    ysq = __builtin_fmaf(yrow[c], yrow[c], ysq);
  const float ynorm = __builtin_sqrtf(ysq);
  // what the query contributes to the filter: coordinates (scaled), or
  // nothing when the filter is switched off for it
  bool y_filtered; // false: coordinates enter as zeros
  bool y_blind;    // true: the query can have no neighbours at all
  float y_scale;
  if (COSINE) {
    y_blind = !(ynorm > 0.0f); // 0 or NaN: every distance is NaN
    y_filtered = !y_blind && ynorm < __builtin_inff();
    y_scale = y_filtered ? -1.0f / ynorm : 0.0f;
  } else {
    y_blind = false;
    y_filtered = ysq <= kFilterNormLimit;
    y_scale = -2.0f;
  }
  const bool active = valid && !y_blind;
  float yb[STEPS]; // B operands: this lane's parity of the augmented query
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int c = 2 * s + half;
    float v = 0.0f;
    if (active) {
      if (c < d)
        v = y_filtered ? yrow[c] * y_scale : 0.0f;
      else if (c == d)
        v = 1.0f;
    }
    yb[s] = v;
  }

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - k) ? lowest_key() : empty_key();
  // exact distances must be strictly below thresh
  float thresh = active ? kKnnSentinel : -__builtin_inff();
  float shared = kKnnSentinel; // bound inherited from other slices / partner
  float posted = kKnnSentinel;
  // the last component of the rows (odd: upper lanes) is 1; the upper lanes
  // hold -cut there (a lane without a query holds zeros everywhere and never
  // parks)
  auto set_thresh = [&](float v) {
    if (!active)
      return;
    thresh = v;
    float cut;
    if (COSINE)
      cut = y_filtered ? v + cos_margin : __builtin_inff();
    else
      cut = mfma_filter_cut(v, ysq, eps);
    if (half)
      yb[STEPS - 1] = -cut;
  };
  set_thresh(thresh);

  // ---- tile staging -------------------------------------------------------
  // thread -> row tid / 8, components tid % 8, tid % 8 + 8, ...
  const int st_row = tid >> 3;
  const int st_c0 = tid & 7;
  // load_tile only issues the global loads (they are in flight during the
  // matrix-core chain of the current tile); store_tile turns what arrived
  // into filter operands
  float raw[PER_THREAD];
  float raw_norm = 0.0f;
  bool raw_real = false;

  auto load_tile = [&](int t) {
    const int pos = t * TR + st_row;
    const size_t g = (size_t)c_begin + pos;
    raw_real = pos < c_count;
    // (rows past the end and padding components read a clamped address and
    // are masked out later)
    const size_t gl = raw_real ? g : (size_t)c_begin;
    raw_norm = p.x_sq[gl];
    const float *src = p.x + gl * d + st_c0;
#pragma unroll
    for (int e = 0; e < PER_THREAD; ++e)
      raw[e] = (st_c0 + 8 * e < d) ? src[8 * e] : 0.0f;
  };
  auto store_tile = [&](int buf) {
    const float nv = raw_norm;
    // coordinates enter the filter scaled by `scale` (0: not at all); `aug`
    // is the augmented component
    float scale, aug;
    if (COSINE) {
      if (!raw_real || !(nv > 0.0f)) { // padding, or a NaN distance anyway
        scale = 0.0f;
        aug = __builtin_nanf("");
      } else if (nv == __builtin_inff()) { // always looked at
        scale = 0.0f;
        aug = -__builtin_inff();
      } else {
        scale = 1.0f / nv;
        aug = 1.0f;
      }
    } else {
      if (!raw_real) {
        scale = 0.0f;
        aug = __builtin_nanf("");
      } else if (!(nv <= kFilterNormLimit)) {
        scale = 0.0f;
        aug = -__builtin_inff();
      } else {
        scale = 1.0f;
        aug = nv * damp;
      }
    }
#pragma unroll
    for (int e = 0; e < PER_THREAD; ++e) {
      const int c = st_c0 + 8 * e;
      float v = (scale != 0.0f && c < d) ? raw[e] * scale : 0.0f;
      v = (c == d) ? aug : v;
      v = (c == DP - 1) ? 1.0f : v; // times -cut
      xs[buf][st_row][(c & 1) * STEPS + (c >> 1)] = v;
    }
  };

  // Exchange of pruning bounds between the slices of a query: the k-th best
  // distance any slice has reached bounds the final k-th distance from above.
  auto sync_bounds = [&]() {
    if (active) {
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
        shared = __builtin_fminf(shared, next_up_positive(seen));
        if (shared < thresh)
          set_thresh(shared);
      }
    }
  };

  // ---- dense re-rank ------------------------------------------------------
  int qn = 0; // parked steps of this lane: queue[0 .. qn)[tid]

  // The next parked row of queue column `column` (relative to the batch's
  // first row; row0 = first row of that lane within a step), or kNoRow.
  constexpr int kNoRow = 1 << 30;
  auto peek = [&](MfmaWalk &w, int column, int entries, int row0) {
    if (w.pending == 0 && w.taken < entries) {
      const uint32_t word = queue[w.taken][column];
      ++w.taken;
      w.pending = word & 0xffffu;
      w.base = (int)(word >> 16) * TR + row0;
    }
    if (w.pending == 0)
      return kNoRow;
    // bit 15 - v of the mask stands for accumulator v = row
    // 8 (v / 4) + v % 4 of the lane's rows: highest bit first
    const int v = 15 - (31 - __builtin_clz(w.pending));
    return w.base + 2 * (v & 12) + (v & 3);
  };
  auto pop = [&](MfmaWalk &w) { // (only after a successful peek)
    w.pending &= ~(1u << (31 - __builtin_clz(w.pending)));
  };

  auto exact_distance = [&](int qq, int g) {
    const float *xr = p.x + (size_t)g * d;
    const float *yr = p.y + (size_t)qq * d;
    float acc = 0.0f;
    if ((d & 3) == 0) {
      const float4 *x4 = reinterpret_cast<const float4 *>(xr);
      const float4 *y4 = reinterpret_cast<const float4 *>(yr);
#pragma unroll 4
      for (int c = 0; c < d / 4; ++c) {
        const float4 a = x4[c];
        const float4 b = y4[c];
        if (COSINE) {
          acc = __builtin_fmaf(a.x, b.x, acc);
          acc = __builtin_fmaf(a.y, b.y, acc);
          acc = __builtin_fmaf(a.z, b.z, acc);
          acc = __builtin_fmaf(a.w, b.w, acc);
        } else {
          const float d0 = a.x - b.x, d1 = a.y - b.y;
          const float d2 = a.z - b.z, d3 = a.w - b.w;
          acc = __builtin_fmaf(d0, d0, acc);
          acc = __builtin_fmaf(d1, d1, acc);
          acc = __builtin_fmaf(d2, d2, acc);
          acc = __builtin_fmaf(d3, d3, acc);
        }
      }
    } else {
      for (int c = 0; c < d; ++c) {
        if (COSINE) {
          acc = __builtin_fmaf(xr[c], yr[c], acc);
        } else {
          const float dc = xr[c] - yr[c];
          acc = __builtin_fmaf(dc, dc, acc);
        }
      }
    }
    if (COSINE) {
      acc = acc / (p.x_sq[g] * p.y_norm[qq]);
      acc = 1.0f - acc;
    }
    return acc;
  };

  // Resolves everything parked since the last drain; pos0 = position of the
  // batch's first row in the slice.
  auto drain = [&](int pos0) {
    // how many rows has each lane parked, and where do they go in the list
    int count = 0;
    for (int e = 0; e < QCAP; ++e)
      if (e < qn)
        count += __builtin_popcount(queue[e][tid] & 0xffffu);
    int offset = count; // inclusive prefix sum over the wave
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1) {
      const int up = __shfl_up(offset, sh);
      if (lane >= sh)
        offset += up;
    }
    const int total = __shfl(offset, kWave - 1);
    offset -= count;
    // the lower lane of a pair collects the keys of both lanes
    const auto qn_both = __builtin_amdgcn_permlane32_swap(
        (unsigned)qn, (unsigned)qn, false, false);
    const auto off_both = __builtin_amdgcn_permlane32_swap(
        (unsigned)offset, (unsigned)offset, false, false);
    const int qn_upper = (int)qn_both[1];
    const int offset_upper = (int)off_both[1];
    const bool owner = half == 0 && active;
    bool changed = false; // wave-uniform

    for (int pass0 = 0; pass0 < total; pass0 += CAP) {
      // 1. the pairs of this pass, compacted
      {
        MfmaWalk w{0, 0u, 0};
        int idx = offset;
        for (;;) {
          const int row = peek(w, tid, qn, 4 * half);
          const bool has = row != kNoRow;
          if (!__any(has))
            break;
          if (has) {
            pop(w);
            if (idx >= pass0 && idx < pass0 + CAP)
              pairs[wave][idx - pass0] =
                  make_int2(q, pos0 + row < c_count ? c_begin + pos0 + row
                                                    : -1);
            ++idx;
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      // 2. exact distances, one pair per lane and round
      const int in_pass = min(CAP, total - pass0);
      for (int i = lane; i < in_pass; i += kWave) {
        const int2 pr = pairs[wave][i];
        float dist = __builtin_nanf("");
        if (pr.y >= 0) // (a padding row is never a candidate)
          dist = exact_distance(pr.x, pr.y);
        results[wave][i] = make_key(dist, (uint32_t)pr.y);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      // 3. the lower lane of every pair takes the keys of both lanes' rows,
      // in ascending row order
      {
        MfmaWalk lo{0, 0u, 0}, hi{0, 0u, 0};
        int idx_lo = offset, idx_hi = offset_upper;
        for (;;) {
          int idx = -1;
          bool has = false;
          if (owner) {
            const int a = peek(lo, tid, qn, 0);
            const int b = peek(hi, tid + 32, qn_upper, 4);
            has = min(a, b) != kNoRow;
            if (has) {
              if (a <= b) {
                pop(lo);
                idx = idx_lo++;
              } else {
                pop(hi);
                idx = idx_hi++;
              }
            }
          }
          if (!__any(has))
            break;
          const bool mine = has && idx >= pass0 && idx < pass0 + CAP;
          const double key = mine ? results[wave][idx - pass0] : empty_key();
          // NaN and sentinel distances fail the compare like in the
          // reference (csrc/cuda/knn_cuda.cu:48,68).  Equality passes: a
          // pass boundary can separate the two lanes' rows, so a row may
          // arrive after higher rows of its partner -- the key order
          // settles ties.
          const bool ok = mine && key_dist(key) <= thresh &&
                          key_dist(key) < kKnnSentinel;
          if (!__any(ok))
            continue;
          sorted_insert<K>(best, ok ? key : empty_key());
          if (owner)
            thresh = __builtin_fminf(key_dist(best[K - 1]), shared);
          changed = true;
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    qn = 0;
    sync_bounds();
    // both lanes of a pair filter with the list's bound
    const auto t_both = __builtin_amdgcn_permlane32_swap(
        __float_as_uint(thresh), __float_as_uint(thresh), false, false);
    const float pair_thresh = __uint_as_float(t_both[0]);
    if (changed || pair_thresh < thresh)
      set_thresh(__builtin_fminf(thresh, pair_thresh));
  };

  if (num_steps > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();
  sync_bounds(); // what other slices already know

  // steps [batch_t0, t] are parked and not yet resolved; the first drains
  // come early (after steps 0, 1 and 3), while the lists are still empty and
  // every row passes
  int batch_t0 = 0;
  for (int t = 0; t < num_steps; ++t) {
    const int buf = t & 1;
    const bool more = t + 1 < num_steps;
    if (more)
      load_tile(t + 1);

    // ---- 32 x 32 filter values on the matrix cores ----------------------
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

    // accumulator v belongs to candidate row 8 (v / 4) + 4 half + v % 4; its
    // sign bit says "look at this row" (bit 15 - v of the mask)
    uint32_t mask = 0;
#pragma unroll
    for (int v = 0; v < 16; ++v)
      mask = __builtin_amdgcn_alignbit(mask, __float_as_uint(acc[v]), 31);
    if (active && mask != 0) {
      queue[qn][tid] = ((uint32_t)(t - batch_t0) << 16) | mask;
      ++qn;
    }
    if (t - batch_t0 == QCAP - 1 || !more || t <= 1 || t == 3) {
      drain(batch_t0 * TR);
      batch_t0 = t + 1;
    }

    if (more)
      store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- results ------------------------------------------------------------
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
