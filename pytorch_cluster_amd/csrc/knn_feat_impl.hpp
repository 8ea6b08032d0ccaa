// Feature-space kNN (8 < d <= 512, k <= 100, Euclidean or cosine) on the gfx950
// matrix cores: ONE fp16 product per pair and component picks a short list of
// candidates per query, a second kernel evaluates those exactly.  Results are
// bit-identical to the reference's scalar loop (csrc/cuda/knn_cuda.cu:52-78).
//
// Stage 1, knn_feat_kernel: a lower bound of every distance on the matrix
// cores.  All rows are scaled by one power of two (chosen per call so that the
// largest component lies in [2^10, 2^11)) and rounded to fp16, X = x / sigma,
// h(X) = fp16(X), components below 2^-14 flushed to zero.  For a row x and a
// query y
//     s = W + sum_c h(X_c) h(-2 Y_c),      W <= |X|^2 (1 - rho),
// is one chain of v_mfma_f32_32x32x16_f16 over the blocks of 16 components
// plus one block that carries W (three fp16 parts times 2^15, 2^4, 2^-7).
// With rho = 2^-9 (2^-8 beyond 256 components, feat_rho) and C0 = 2^-12 d
// the value
//     l = s + |Y|^2 (1 - rho) - C0
// is a LOWER bound of the distance e' = e / sigma^2 the reference computes,
// and e' <= F(l) = (l + 6 rho |Y|^2 + 2 C0) (1 + 4.1 rho):
//   * fp16 rounding: |h(v) - v| <= 2^-11 |v| + 2^-14, so the sum of products is
//     within (2^-10 + 2^-11) (|X|^2 + |Y|^2) + 2^-13 d of -2 X.Y (the absolute
//     parts folded in with a b <= (a^2 + b^2) / 2);
//   * accumulation in the matrix cores: d + 16 terms, each step within 2^-22 of
//     the running magnitude (<= 2.01 (|X|^2 + |Y|^2)): 0.13 x 2^-10 at d = 256;
//   * the fp32 chains of |x|^2 and of the reference's distance: (d + 2) 2^-24
//     relative each;
//   together below 1.5 x 2^-10 (|X|^2 + |Y|^2) + C0 / 2, and rho = 2 x 2^-10.
//   F follows with |X|^2 <= 2 |X - Y|^2 + 2 |Y|^2.
//   Where the reference's own squares underflow (tiny rows) each loses up to
//   2^-149: C0 grows by d 2^-149 / sigma^2.
// The cosine distance 1 - x.y / (|x| |y|) runs the same chain on rows
// normalised to length 2^10 (W = 2^20 exactly): |s - e'| <= Ec = 2^-9 2^20
// (rounding 2^-10, accumulation, normalisation and the exact chain
// (4 d + 72) 2^-24), so l = s - Ec and F(l) = l + 2 Ec.  Rows and queries of
// norm below 1e-18, whose products underflow in the reference's chain, are
// left to the other kernel.
//
// Every query keeps the k + 16 smallest (s, row) of its slice of x in a
// sorted register list; the k-th of them bounds the query's final k-th
// distance by U = F(l_k), and a row is looked at only if l <= U, i.e.
// s < cut.  The 16 values a lane gets from a chain are tested against its cut
// with a minimum tree; lanes that hold a value below it park (s, row) in LDS,
// and the lists take the parked values in rounds, all queries of a wave
// together.  No global memory is read for any of this.
//
// Stage 2, feat_refine_kernel (one wave per query): the exact distance --
// direct differences, one FMA per component in ascending order
// (csrc/cuda/knn_cuda.cu:9-28,55-66) -- of the listed rows that can matter,
// sorted by (distance, row).  The list provably holds the k nearest rows when
// it is not full or when its last entry's lower bound lies above the k-th
// exact distance found (every row outside the list has a lower bound at
// least as large).  Queries for which neither holds (more than 16 rows within
// the rounding margin of the k-th distance: near-duplicates) are flagged and
// searched again by the kernel that evaluates every candidate exactly in the
// loop (knn_mfma_impl.hpp), as is everything when x holds rows whose squared
// norm overflows.
//
// Mapping: a workgroup owns 128 queries of one segment (4 waves x 32) and one
// slice of the segment's x rows; lanes l and l + 32 share a query and split
// its candidates (the 32 x 32 result layout), the lower lane keeps the list.
// Candidate tiles (64 packed rows; 32 from 129 components on) go from global
// memory straight into a ring of three LDS buffers with LDS-direct loads, two
// tiles ahead.  Slices share their bounds through `tau` (atomic minimum).
#pragma once

#include "device_utils.hpp"
#include "knn_lowd_impl.hpp"
#include "launchers.hpp"

namespace pca {

constexpr int kFeatQueries = 128; // queries per workgroup
constexpr int kFeatStep = 32;     // candidates per chain of matrix instructions
constexpr int kFeatQueue = 8;     // parked rows per lane
constexpr int kFeatSlack = 16;    // list entries beyond k
constexpr int kFeatDrainEvery = 64;
constexpr int kFeatRoundPeriod = 8; // tiles between scheduled rounds
constexpr int kFeatMaxDim = 512;    // components this path takes
constexpr int kFeatRedoGroup = 32;  // queued queries per workgroup of the scan
constexpr int kFeatMaxHits = 256;   // most rows the scan holds per query
constexpr int kFeatRedoSlices = 32; // workgroups that share a group's rows

typedef _Float16 feat_f16x8_t __attribute__((ext_vector_type(8)));
typedef float feat_acc_t __attribute__((ext_vector_type(16)));

// Per-call values the kernels share through device memory.
struct FeatGlobals {
  unsigned max_bits; // largest finite |component| of x and y (float bits)
  int odd_rows;      // rows of x the filter cannot represent
  int any_redo;      // queries whose list could not be shown complete
  int unresolved;    // ... of them, those left to the full second pass
  int queued;        // ... and those queued for the threshold scan
  int pad[3];
  // event counts of the filter kernel, written only by builds with
  // -DPCA_FEAT_STATS (steps, flagged steps, parked singles, lane-by-lane
  // values, drains, list rounds, direct steps, direct rounds)
  unsigned long long stats[8];
  // Rows far larger than the rest do not set the scale.  hist_x / hist_y: rows
  // per binary exponent of their largest finite |component| (kFeatHistCopies
  // copies that the workgroups spread their counts over: thousands of adds to
  // one word take turns in the L2, 10 ns each); out_limit: float
  // bits of the largest |component| the scale was made for (rows of x beyond
  // it, at most kFeatMaxOutliers, stay out of the filter and are evaluated
  // exactly for every query: out_rows; queries beyond it take the second
  // pass)
  unsigned out_limit;
  int n_out;
  int out_rows[8];
  unsigned hist_x[32 * 256];
  unsigned hist_y[32 * 256];
};
constexpr int kFeatMaxOutliers = 8;
constexpr int kFeatHistCopies = 32;

// ---- constants of the error analysis (see the header) ----------------------
// rho: 2^-9 up to 256 components, 2^-8 beyond (the accumulation error of the
// longer chains no longer fits under 2^-9)
__host__ __device__ __forceinline__ double feat_rho(int d) {
  return d <= 256 ? 1.0 / 512.0 : 1.0 / 256.0;
}
__host__ __device__ __forceinline__ double feat_grow(int d) {
  return 1.0 + 4.1 * feat_rho(d);
}
constexpr double kFeatCosScale = 1048576.0; // 2^20
// Ec = rho x 2^20
__host__ __device__ __forceinline__ double feat_cos_err(int d) {
  return feat_rho(d) * kFeatCosScale;
}
// smallest norm the cosine filter takes
constexpr float kFeatCosTiny = kCosTinyNorm;

__host__ __device__ __forceinline__ double feat_c0(int d) {
  return (double)d * (1.0 / 4096.0);
}

// 1 / sigma: the power of two that brings `max_bits` into [2^10, 2^11).
__device__ __forceinline__ float feat_inv_sigma(unsigned max_bits) {
  if (max_bits == 0)
    return 1.0f;
  const int biased = (int)((max_bits >> 23) & 0xffu);
  int e = 137 - biased;
  e = e > 100 ? 100 : (e < -100 ? -100 : e);
  return __uint_as_float((uint32_t)(e + 127) << 23);
}

// fp16 nearest-even with small values flushed to zero, as bits.
__device__ __forceinline__ uint32_t feat_h(float v) {
  if (!(__builtin_fabsf(v) >= 6.103515625e-05f)) // 2^-14 (NaN: zero)
    return 0u;
  const _Float16 h = (_Float16)v;
  return (uint32_t)__builtin_bit_cast(unsigned short, h);
}

// Largest fp16 (flushed like feat_h) that is <= v, for v >= 0.
__device__ __forceinline__ uint32_t feat_h_down(double v) {
  if (!(v >= 6.103515625e-05))
    return 0u;
  if (v >= 65504.0)
    return 0x7bffu;
  _Float16 h = (_Float16)(float)v;
  unsigned short bits = __builtin_bit_cast(unsigned short, h);
  if ((double)(float)h > v)
    --bits; // positive values: the previous fp16
  if (bits < 0x0400u) // below the normal range
    return 0u;
  return bits;
}

__device__ __forceinline__ double feat_h_value(uint32_t bits) {
  return (double)(float)__builtin_bit_cast(_Float16, (unsigned short)bits);
}

// Smallest float above v, twice over (a strict `<` test against the result
// admits everything <= v).
__device__ __forceinline__ float feat_float_above(double v) {
  float f = (float)v;
  if (!(f == f))
    return __builtin_inff();
  if (f == __builtin_inff())
    return f;
  if (f == -__builtin_inff())
    f = -3.4028234663852886e38f;
  auto up = [](float a) {
    if (a == 0.0f)
      return 1.401298464324817e-45f;
    const uint32_t u = __float_as_uint(a);
    return __uint_as_float(a > 0.0f ? u + 1u : u - 1u);
  };
  if ((double)f < v)
    f = up(f);
  return up(f);
}

// What a query contributes to the bounds.
struct FeatQuery {
  bool dead;    // no row can be a neighbour (NaN components, zero norm)
  bool odd;     // the filter cannot represent it: searched by the other kernel
  double shift; // l = s + shift
  double widen; // F(l) = (l + widen) * grow
  double grow;
};

// Classification and bound constants of query row `yrow`.
//   Euclid: `norm_in` unused.  cosine: the row's norm.
//   R16 = 1 / 2: the row takes part in the filter with every component times
//   chain_keep<R16> (device_utils.hpp), as the rows of x were packed.
template <bool COSINE, int R16 = 0>
__device__ __forceinline__ FeatQuery feat_query(const float *yrow, int d,
                                                float inv_sigma,
                                                float norm_in) {
  FeatQuery fq;
  if (COSINE) {
    // A query of zeros has no neighbours (0 / 0).  A norm of zero over
    // components that are not all zero -- their squares underflowed -- still
    // divides a dot product that need not be zero: the reference returns the
    // rows with a positive one at distance -inf.  That query is left to the
    // exact evaluation of every row, like the other norms the filter cannot
    // take.
    bool nonzero = false;
    if (norm_in == 0.0f)
      for (int c = 0; c < d; ++c)
        nonzero = nonzero || yrow[c] != 0.0f;
    fq.dead = !(norm_in > 0.0f) && !nonzero;
    // (below kFeatCosTiny the reference's own products underflow too much
    // for the margin Ec)
    fq.odd = !fq.dead &&
             !(norm_in < __builtin_inff() && norm_in >= kFeatCosTiny);
    fq.shift = -feat_cos_err(d);
    fq.widen = 2.0 * feat_cos_err(d);
    fq.grow = 1.0;
    return fq;
  }
  float chain = 0.0f; // classification as the old kernel does it
  double ysq = 0.0;
  float top = 0.0f;
  for (int c = 0; c < d; ++c) {
    const float v = yrow[c] * chain_keep<R16>(d, c);
    chain = __builtin_fmaf(v, v, chain);
    const float scaled = v * inv_sigma;
    top = __builtin_fmaxf(top, __builtin_fabsf(scaled));
    const double s = (double)scaled;
    ysq += s * s;
  }
  fq.dead = chain != chain;
  // (a component beyond the range the scale was made for -- a query far
  // larger than the other rows -- would overflow the fp16 operand)
  fq.odd = !fq.dead && !(chain < __builtin_inff() && top < 2048.0f);
  // (the reference's squares lose up to 2^-149 each where they underflow)
  const double c0 =
      feat_c0(d) + (double)d * 1.4012984643248171e-45 * (double)inv_sigma *
                       (double)inv_sigma;
  fq.shift = ysq * (1.0 - feat_rho(d)) - c0;
  fq.widen = 6.0 * feat_rho(d) * ysq + 2.0 * c0;
  fq.grow = feat_grow(d);
  return fq;
}

// Key of an empty list slot: above every (s, row).
__device__ __forceinline__ double feat_empty_key() {
  return __hiloint2double((int)(0x7f800000u + kKeyBias), -1);
}

struct KnnFeatParams {
  const float *x;
  const float *y;
  const int64_t *ptr_x;
  const int64_t *ptr_y;
  const float *x_norm; // [n] squared norms of x (cosine: norms)
  const float *y_norm; // [m] norms of y (cosine only)
  const uint4 *x_pack; // packed fp16 rows (feat_pack_kernel)
  FeatGlobals *globals;
  int n, m, d, num_segments, k;
  const int *work_start; // [num_segments + 1] first 128-query tile per segment
  int num_chunks;        // slices of every segment's x rows
  int round_period;       // tiles between scheduled rounds
  float *tau;            // [m] shared bounds U (scaled units, float bits)
  double *partial;       // [num_chunks * tiles][k + 16][128] keys
  double *cand;          // [m][k + 16] merged keys
  int *redo_q;           // [m] 1: search this query again (full second pass)
  // threshold scan of the flagged queries (feat_redo_scan_kernel)
  int *redo_list;        // [redo_cap] queued queries
  float *redo_tau;       // [redo_cap] their k-th distance among the listed rows
  int *hit_count;        // [redo_cap] rows found at or below it
  double *hits;          // [redo_cap][hit_cap] their (distance, row) keys
  int redo_cap;
  int hit_cap;
  const int *overflow;   // [m] or null: 1 = the first stage lost candidates
  int *out_idx;
  float *out_dist;
  int *out_count;
  // the compaction's block sums and self slots (DenseResult; the one-kernel
  // search fills them, NULL otherwise)
  unsigned long long *edge_sums = nullptr;
  int *self_pos = nullptr;
  int *kept = nullptr;
  // the radius search of the one-kernel search (k: max_num_neighbors)
  float r2 = 0.0f;
  int ignore_same = 0;
};

// Packed row: 2 units of 16 bytes (8 fp16) per block of 16 components, NB
// blocks (the last one carries W), one unit of padding (odd stride: the reads
// of neighbouring rows fall on distinct LDS banks).
template <int NB> struct FeatShape {
  static constexpr int UNITS = 2 * NB;
  static constexpr int RSU = UNITS + 1;
  static constexpr int MAX_D = 16 * (NB - 1);
  static constexpr int TILE = NB <= 9 ? 64 : 32; // rows per LDS tile
  // LDS buffers the tiles rotate through (160 KB per CU)
  static constexpr int RING = 3;
};

// Workgroups per CU the filter kernel is compiled for: two (256 registers per
// lane) while the query operands (4 NB registers) and the list (KP registers)
// leave room for the rest, one (512 registers) beyond.
constexpr int feat_resident_groups(int nb, int kp) {
  return (nb > 17 || kp > 64) ? 1 : 2;
}

// ---- preparation ------------------------------------------------------------

// Packs the rows of x: one thread per 16-byte unit, `spare` zero rows behind
// the last one (the last tile of a slice is read in full).
template <int NB, bool COSINE>
__global__ __launch_bounds__(kBlock) void feat_pack_kernel(
    const float *__restrict__ x, const float *__restrict__ norms,
    const float *__restrict__ cls, const unsigned *__restrict__ big, int n,
    int d, int spare, FeatGlobals *g, uint4 *__restrict__ out) {
  typedef FeatShape<NB> S;
  const size_t id = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (id >= (size_t)(n + spare) * S::RSU)
    return;
  const int row = (int)(id / S::RSU);
  const int unit = (int)(id - (size_t)row * S::RSU);
  uint32_t part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (row < n && unit < S::UNITS) {
    const float nv = norms[row];
    // squared norm by another summation, NaN when a component is not finite
    // (such a row is nobody's neighbour); infinite: finite components whose
    // squares overflow -- the one kind of row this path cannot search
    const float cv = cls[row];
    // usable: the row takes part in the filter; otherwise it is padding that
    // no cut ever reaches
    bool usable;
    float scale;
    if (COSINE) {
      usable = nv >= kFeatCosTiny && nv < __builtin_inff() &&
               cv < __builtin_inff();
      scale = usable ? 1024.0f / nv : 0.0f;
    } else {
      usable = nv < __builtin_inff(); // (false for NaN too)
      scale = feat_inv_sigma(g->max_bits);
      // a row far larger than the others: left out here (the scale was made
      // without it), listed for the exact stage
      if (usable && big != nullptr && big[row] > g->out_limit) {
        usable = false;
        if (unit == 0) {
          const int slot = atomicAdd(&g->n_out, 1);
          if (slot < kFeatMaxOutliers)
            g->out_rows[slot] = row;
        }
      }
    }
    // (cosine: also a row whose norm underflowed to zero over components
    // that are not all zero -- its dot products need not be zero, and the
    // reference divides them by that zero)
    bool lost_norm = false;
    if (COSINE && unit == 0 && nv == 0.0f)
      for (int c = 0; c < d; ++c)
        lost_norm = lost_norm || x[(size_t)row * d + c] != 0.0f;
    if (unit == 0 &&
        (cv == __builtin_inff() || (cv == cv && nv == __builtin_inff()) ||
         (COSINE && nv > 0.0f && nv < kFeatCosTiny) || lost_norm))
      atomicAdd(&g->odd_rows, 1);
    if (unit < S::UNITS - 2) {
      if (usable) {
        const int c0 = 8 * unit;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int c = c0 + e;
          part[e] = c < d ? feat_h(x[(size_t)row * d + c] * scale) : 0u;
        }
      }
    } else if (unit == S::UNITS - 2) {
      // W in three parts (times 2^15, 2^4, 2^-7 on the query side), each
      // rounded towards zero
      if (!usable) {
        part[0] = 0x7bffu; // 65504 x 2^15: above every cut
      } else {
        double w;
        if (COSINE) {
          w = kFeatCosScale;
        } else {
          const double inv = (double)scale;
          w = (double)nv * inv * inv * (1.0 - feat_rho(d));
        }
        const uint32_t a1 = feat_h_down(w * (1.0 / 32768.0));
        const double r1 = w - feat_h_value(a1) * 32768.0;
        const uint32_t a2 = feat_h_down(r1 * (1.0 / 16.0));
        const double r2 = r1 - feat_h_value(a2) * 16.0;
        const uint32_t a3 = feat_h_down(r2 * 128.0);
        part[0] = a1;
        part[1] = a2;
        part[2] = a3;
      }
      // powers of two for a cut carried by the query's operand
      // (knn_feat_wide_impl.hpp; queries without one hold zeros there)
      part[3] = 0x7800u; // 2^15
      part[4] = 0x5000u; // 2^5
      part[5] = 0x2800u; // 2^-5
    } else {
      part[0] = 0x7800u;
      part[1] = 0x5000u;
      part[2] = 0x2800u;
    }
  }
  out[id] = make_uint4(part[0] | (part[1] << 16), part[2] | (part[3] << 16),
                       part[4] | (part[5] << 16), part[6] | (part[7] << 16));
}

// ---- stage 1 ----------------------------------------------------------------

// Value v of the 16 * SUBS accumulator registers of a tile, for a wave-uniform
// v.
template <int SUBS>
__device__ __forceinline__ float feat_pick(const feat_acc_t (&a)[SUBS], int v) {
  float r = 0.0f;
#pragma unroll
  for (int sub = 0; sub < SUBS; ++sub) {
    if ((v >> 4) == sub)
      r = a[sub][v & 15]; // (a uniform index: register-relative read)
  }
  return r;
}

// KP: list width (>= k + 16).  The first KP - (k + 16) slots hold keys below
// every real one, so the k-th smallest real key is always slot KP - 17 and the
// last one slot KP - 1.  The two lanes of a query hold half of its list each:
// the lower lane slots 0 .. KP/2 - 1, the upper lane the rest.  A key enters
// the lower half; what that half pushes out enters the upper half one
// insertion later (both lanes run the same network of KP/2 slots, each on its
// own key), so the upper half may lag by one key -- its entries are then too
// large, never too small, which keeps every bound read from it valid.
template <int NB, int KP, bool COSINE>
__global__ __launch_bounds__(kBlock, feat_resident_groups(NB, KP)) void
knn_feat_kernel(KnnFeatParams p) {
  typedef FeatShape<NB> S;
  constexpr int RSU = S::RSU;
  constexpr int TILE = S::TILE;
  constexpr int SUBS = TILE / kFeatStep;
  constexpr int TILE_UNITS = TILE * RSU;
  constexpr int PIECES = (TILE_UNITS + kWave - 1) / kWave;
  constexpr int MAX_PIECES_PER_WAVE = (PIECES + 3) / 4;
  constexpr int RING = S::RING;
  constexpr int QCAP = kFeatQueue;
  static_assert((QCAP & (QCAP - 1)) == 0, "the queue is a ring");
  constexpr int TQ = kFeatQueries;
  constexpr int H = KP / 2;
  constexpr int KTH = KP - 1 - kFeatSlack; // slot of the k-th smallest key

  __shared__ __attribute__((aligned(16))) uint4 xs[RING][TILE_UNITS];
  __shared__ uint2 queue[QCAP][kBlock]; // (s bits, row)

  if (p.globals->odd_rows != 0)
    return; // everything is searched by the other kernel

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int half = lane >> 5;
  const int col = lane & 31;

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
  const int kk = p.k + kFeatSlack; // real list entries
  const float *yrow = p.y + (size_t)(valid ? q : y_begin) * d;

  const int seg_len = x_end - x_begin;
  const int chunk_len =
      ((seg_len + p.num_chunks - 1) / p.num_chunks + TILE - 1) / TILE * TILE;
  const int c_begin = min(x_end, x_begin + chunk * chunk_len);
  const int c_count = min(x_end, c_begin + chunk_len) - c_begin;
  const int num_tiles = (c_count + TILE - 1) / TILE;

  // ---- per-lane query state ---------------------------------------------
  const float inv_sigma = COSINE ? 1.0f : feat_inv_sigma(p.globals->max_bits);
  const float ynorm = COSINE && valid ? p.y_norm[q] : 1.0f;
  const FeatQuery fq = feat_query<COSINE>(yrow, d, inv_sigma, ynorm);
  const bool active = valid && !fq.dead && !fq.odd;
  const float y_scale =
      COSINE ? (active ? -1024.0f / ynorm : 0.0f) : -2.0f * inv_sigma;

  // B operands: this lane's 8 components of every block; the last block
  // holds the powers of two that W's parts are multiplied by (lower lanes)
  feat_f16x8_t yh[NB];
  const bool vec4 = (d & 3) == 0;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    uint32_t hb[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (i < NB - 1) {
      const int cb = 16 * i + 8 * half;
      float comp[8];
      if (vec4) {
        const float4 a =
            *reinterpret_cast<const float4 *>(yrow + min(cb, d - 4));
        const float4 b =
            *reinterpret_cast<const float4 *>(yrow + min(cb + 4, d - 4));
        comp[0] = a.x, comp[1] = a.y, comp[2] = a.z, comp[3] = a.w;
        comp[4] = b.x, comp[5] = b.y, comp[6] = b.z, comp[7] = b.w;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          comp[e] = yrow[min(cb + e, d - 1)];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e)
        hb[e] = (active && cb + e < d) ? feat_h(comp[e] * y_scale) : 0u;
    } else if (half == 0 && active) {
      hb[0] = 0x7800u; // 2^15
      hb[1] = 0x4c00u; // 2^4
      hb[2] = 0x2000u; // 2^-7
    }
    yh[i] = __builtin_bit_cast(
        feat_f16x8_t,
        make_uint4(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16),
                   hb[4] | (hb[5] << 16), hb[6] | (hb[7] << 16)));
  }

  // this lane's half of the query's list
  double best[H];
#pragma unroll
  for (int j = 0; j < H; ++j)
    best[j] = (half * H + j < KP - kk) ? lowest_key() : feat_empty_key();
  // (upper lanes) what the lower half pushed out last, not yet taken in
  double carry = feat_empty_key();

  // a row is looked at when its s is below cut (+inf: no bound yet; -inf: a
  // lane without a query)
  float cut = active ? __builtin_inff() : -__builtin_inff();
  double bound = __builtin_inf(); // U: upper bound of the final k-th distance
  float posted = __builtin_inff();
  // what the other slices of the query have published (read every few tiles)
  float tau_seen = valid ? __hip_atomic_load(&p.tau[q], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT)
                         : __builtin_inff();

  // U from the list's k-th entry and from the other slices of the query
  auto update_bound = [&](bool publish_all) __attribute__((always_inline)) {
    // the k-th smallest key, wherever it lives, in the lower lane
    double kth;
    if (KTH < H) {
      kth = best[KTH < H ? KTH : 0];
    } else {
      const double mine = best[KTH >= H ? KTH - H : 0];
      const auto hi = __builtin_amdgcn_permlane32_swap(
          (unsigned)__double2hiint(mine), (unsigned)__double2hiint(mine),
          false, false);
      const auto lo = __builtin_amdgcn_permlane32_swap(
          (unsigned)__double2loint(mine), (unsigned)__double2loint(mine),
          false, false);
      kth = __hiloint2double((int)hi[1], (int)lo[1]);
    }
    if (half == 0 && active) {
      if (kth < feat_empty_key()) {
        const double l = (double)key_dist(kth) + fq.shift;
        const double u = (l + fq.widen) * fq.grow;
        bound = u < bound ? u : bound;
      }
      // published as a non-negative float, rounded up (non-negative floats
      // order like their bit patterns)
      float own = bound < 3.0e38 ? feat_float_above(bound) : __builtin_inff();
      own = __builtin_fmaxf(own, 0.0f);
      const float seen = tau_seen;
      if (own < seen &&
          (own < posted * 0.999f || (publish_all && own < posted))) {
        __hip_atomic_fetch_min(reinterpret_cast<int *>(&p.tau[q]),
                               (int)__float_as_uint(own), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        posted = own;
      } else if (seen < posted) {
        posted = seen;
        bound = (double)seen < bound ? (double)seen : bound;
      }
      if (bound < __builtin_inf())
        cut = feat_float_above(bound - fq.shift);
    }
    // both lanes of a query filter with the same cut
    const auto both = __builtin_amdgcn_permlane32_swap(
        __float_as_uint(cut), __float_as_uint(cut), false, false);
    if (half && active)
      cut = __uint_as_float(both[0]);
  };

  // ---- tile staging -------------------------------------------------------
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto request_tile = [&](int t) {
    const uint4 *src = p.x_pack + ((size_t)c_begin + (size_t)t * TILE) * RSU;
    const uint32_t dst = (uint32_t)(uintptr_t)&xs[t % RING][0];
#pragma unroll
    for (int e = 0; e < MAX_PIECES_PER_WAVE; ++e) {
      const int piece = wave_u + 4 * e;
      const int u = piece * kWave + lane;
      // (a tile of 64 rows of an odd number of units is a whole number of
      // pieces)
      if (piece < PIECES && (TILE_UNITS % kWave == 0 || u < TILE_UNITS)) {
        const uint4 *g = src + u;
        const uint32_t base = dst + (uint32_t)piece * (kWave * 16);
        asm volatile("s_mov_b32 m0, %1\n\t"
                     "s_nop 0\n\t"
                     "global_load_lds_dwordx4 %0, off"
                     :
                     : "v"(g), "s"(base)
                     : "memory");
      }
    }
  };
  // all but the newest tile's requests of this wave have completed
  auto await_tile = [&](bool newer_in_flight) {
    if (newer_in_flight)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(MAX_PIECES_PER_WAVE - 1)
                   : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };

  // parked rows of this lane: a ring, entries qh .. qt - 1 at slot % QCAP
  int qh = 0, qt = 0;
#ifdef PCA_FEAT_STATS
  unsigned long long st[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#define PCA_STAT(i, n) st[i] += (n)
#else
#define PCA_STAT(i, n)
#endif

  if (num_tiles > 0)
    request_tile(0);
  if (num_tiles > 1)
    request_tile(1);
  if (RING > 2 && num_tiles > 2)
    request_tile(2);
  update_bound(false); // what other slices already know
  if (num_tiles > 0) {
    await_tile(num_tiles > 1); // (tiles 1 and 2 count as one newer tile here:
                               // at worst the wait is longer than needed)
  }

  // One pass per tile, software-pipelined: pass t issues the chains of matrix
  // instructions of tile t (into `cur`) and, in their shadow -- a matrix
  // instruction occupies the issue port for one of its eight passes --, takes
  // the minimum and the flags of tile t - 1's results (`old`).  Then the
  // workgroup's part of tile t + 1 is awaited, and what tile t - 1 flagged is
  // parked.  A pass ends with the rounds in which the lists take rows: the
  // ONLY place per pass body where the insertion network is instantiated.
  // Either the flagged values straight from the accumulators (`direct`: a
  // lane has more of them than free queue slots, or the tile reaches past the
  // slice's end), or the oldest parked row of every lane.  Two more passes at
  // the end look at the last tile and empty the queues.  The body exists
  // twice, with the two sets of accumulators in either role.
  auto pass = [&](feat_acc_t (&cur)[SUBS], feat_acc_t (&old)[SUBS],
                  int t) __attribute__((always_inline)) {
    const bool finish = t == num_tiles + 1;
    const int pos0 = (t - 1) * TILE; // position of `old`'s tile in the slice
    const bool look = t >= 1 && t <= num_tiles;
    uint32_t mask[SUBS];
    float lo[SUBS];
#pragma unroll
    for (int sub = 0; sub < SUBS; ++sub) {
      mask[sub] = 0;
      lo[sub] = 0.0f;
    }
    bool direct = false;
    if (!finish) {
      // this wave's pieces of tile t have arrived (awaited at the end of the
      // previous pass); after the barrier so have everybody's, and everybody
      // is done with tile t - 1
      __syncthreads();
      if (t >= 1 && t + RING - 1 < num_tiles)
        request_tile(t + RING - 1); // into the buffer of tile t - 1
      // the tile's SUBS * NB operands, read AHEAD operands before they are
      // used (LDS latency is several matrix instructions long); pass
      // num_tiles has no tile: it computes on what the buffer holds and
      // nobody looks at the result
      const uint4 *arow = &xs[t % RING][col * RSU + half];
      constexpr int OPS = SUBS * NB;
      constexpr int AHEAD = 4;
      uint4 window[AHEAD];
#pragma unroll
      for (int o = 0; o < AHEAD && o < OPS; ++o)
        window[o] = arow[(o / NB) * kFeatStep * RSU + 2 * (o % NB)];
#pragma unroll
      for (int sub = 0; sub < SUBS; ++sub)
        cur[sub] = feat_acc_t{0};
      __builtin_amdgcn_sched_barrier(0); // (the reads above stay above)
      // smallest of the lane's 16 values of every step of the previous tile,
      // and which of the 16 are below the cut: bit 15 - v of the mask for
      // accumulator v (the sign of the difference; a cut of +inf flags
      // everything, -inf nothing)
#pragma unroll
      for (int sub = 0; sub < SUBS; ++sub) {
        const feat_acc_t &a = old[sub];
        float m0 = min3f(a[0], a[1], a[2]);
        float m1 = min3f(a[3], a[4], a[5]);
        float m2 = min3f(a[6], a[7], a[8]);
        float m3 = min3f(a[9], a[10], a[11]);
        float m4 = min3f(a[12], a[13], a[14]);
        m0 = min3f(m0, m1, m2);
        m3 = min3f(m3, m4, a[15]);
        lo[sub] = __builtin_fminf(m0, m3);
        uint32_t part[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          uint32_t mk = __float_as_uint(a[4 * g] - cut) >> 31;
#pragma unroll
          for (int v = 1; v < 4; ++v)
            mk = __builtin_amdgcn_alignbit(
                mk, __float_as_uint(a[4 * g + v] - cut), 31);
          part[g] = mk & 15u;
        }
        mask[sub] = (part[0] << 12) | (part[1] << 8) | (part[2] << 4) | part[3];
      }
#pragma unroll
      for (int o = 0; o < OPS; ++o) {
        const feat_f16x8_t a =
            __builtin_bit_cast(feat_f16x8_t, window[o % AHEAD]);
        if (o + AHEAD < OPS) {
          const int n = o + AHEAD;
          window[o % AHEAD] = arow[(n / NB) * kFeatStep * RSU + 2 * (n % NB)];
        }
        cur[o / NB] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
            a, yh[o % NB], cur[o / NB], 0, 0, 0);
        // one matrix instruction, one LDS read, a few of the vector
        // instructions above, in this order
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
      }
      // (keeps the minimum and the flags up here instead of next to their
      // first use further down)
#pragma unroll
      for (int sub = 0; sub < SUBS; ++sub)
        asm volatile("" : "+v"(mask[sub]), "+v"(lo[sub]));
      __builtin_amdgcn_sched_barrier(0);
      // the next tile's pieces of this wave, so that the next pass starts with
      // the barrier
      if (t + 1 < num_tiles)
        await_tile(RING > 2 && t + 2 < num_tiles);
      // (consumed inside the branch, so that the wait for it stays there)
      if ((t & 63) == 63) {
        const float now = __hip_atomic_load(&p.tau[valid ? q : y_begin],
                                            __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
        tau_seen = __builtin_fminf(tau_seen, now);
      }

      bool any_low = false;
#pragma unroll
      for (int sub = 0; sub < SUBS; ++sub)
        any_low |= mask[sub] != 0;
      PCA_STAT(0, look ? SUBS : 0);
      if (look && __any(any_low)) {
        PCA_STAT(1, 1);
        const bool tail = pos0 + TILE > c_count;
        int cnt = 0;
#pragma unroll
        for (int sub = 0; sub < SUBS; ++sub) {
          // the slice's last tile may reach past its end
          if (tail) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
              if (pos0 + sub * kFeatStep + 8 * (v / 4) + 4 * half + (v % 4) >=
                  c_count)
                mask[sub] &= ~(1u << (15 - v));
          }
          cnt += __builtin_popcount(mask[sub]);
        }
        direct = tail || __any(qt - qh + cnt > QCAP);
        if (!direct) {
#pragma unroll
          for (int sub = 0; sub < SUBS; ++sub) {
            const uint32_t mk = mask[sub];
            const int c1 = __builtin_popcount(mk);
            const int row0 = c_begin + pos0 + sub * kFeatStep;
            // one value below the cut: it is the step's minimum
            PCA_STAT(2, __builtin_popcountll(__ballot(c1 == 1)));
            if (c1 == 1) {
              const int v = __builtin_clz(mk) - 16;
              queue[qt & (QCAP - 1)][tid] = make_uint2(
                  __float_as_uint(lo[sub]),
                  (uint32_t)(row0 + 8 * (v >> 2) + 4 * half + (v & 3)));
              ++qt;
            }
            // several: lane by lane
            uint64_t pend = __ballot(c1 > 1);
            while (pend != 0) {
              const int src = __builtin_ctzll(pend);
              pend &= pend - 1;
              uint32_t bits = __builtin_amdgcn_readlane(mk, src);
              const int src_half = src >> 5;
              while (bits != 0) {
                const int hb = 31 - __builtin_clz(bits);
                bits &= ~(1u << hb);
                const int v = 15 - hb;
                const float s = feat_pick<SUBS>(old, 16 * sub + v);
                PCA_STAT(3, 1);
                if (lane == src) {
                  queue[qt & (QCAP - 1)][tid] = make_uint2(
                      __float_as_uint(s),
                      (uint32_t)(row0 + 8 * (v / 4) + 4 * src_half + (v % 4)));
                  ++qt;
                }
              }
            }
          }
        } else {
          PCA_STAT(6, 1);
        }
      }
    }

    // ---- rounds ---------------------------------------------------------
    bool changed = false;
    uint32_t mask_upper[SUBS];
#pragma unroll
    for (int sub = 0; sub < SUBS; ++sub) {
      mask_upper[sub] = 0;
      if (direct) {
        const auto mboth = __builtin_amdgcn_permlane32_swap(
            mask[sub], mask[sub], false, false);
        mask_upper[sub] = mboth[1];
      }
    }
    int dv = direct ? 0 : 32 * SUBS; // (accumulator, lane of the pair) to take
    int turn = 0; // 0: the lower lanes' turn, 1: the upper lanes', 2: done
    bool flushed = false;
    // (most passes have nothing to do here)
    const bool rounds_due = direct || finish ||
                            (t % p.round_period) == p.round_period - 1 ||
                            __any(qt - qh >= QCAP - 2);
#pragma unroll 1
    for (; rounds_due;) {
      double key = feat_empty_key();
      bool has = false;
      if (dv < 32 * SUBS) {
        // accumulator v of the lower (dv even) or upper (dv odd) lanes
        const int v = (dv >> 1) & 15, sub = dv >> 5, upper = dv & 1;
        ++dv;
        const uint32_t bit = 1u << (15 - v);
        uint32_t mk = 0;
#pragma unroll
        for (int s2 = 0; s2 < SUBS; ++s2)
          if (s2 == sub)
            mk = upper ? mask_upper[s2] : mask[s2];
        has = half == 0 && (mk & bit) != 0;
        if (!__any(has))
          continue;
        const float mine = feat_pick<SUBS>(old, 16 * sub + v);
        const auto vboth = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(mine), __float_as_uint(mine), false, false);
        const int r = c_begin + pos0 + sub * kFeatStep + 8 * (v / 4) +
                      4 * upper + (v % 4);
        if (has)
          key = make_key(upper ? __uint_as_float(vboth[1]) : mine,
                         (uint32_t)r);
        PCA_STAT(7, 1);
      } else {
        // the oldest parked row of the lower lanes, then of the upper lanes:
        // every few tiles (the same in all four waves of the workgroup, which
        // meet at the barrier), when a queue is nearly full, and everything
        // at the end
        const uint64_t waiting = __ballot(qh < qt);
        if (waiting == 0) {
          if (!finish || flushed)
            break;
          flushed = true; // one last insertion takes the carry in
        } else {
          const bool must = finish || __any(qt - qh >= QCAP - 2);
          if (turn >= 2) {
            if (!must)
              break;
            turn = 0;
          }
          if (turn == 0 && !must &&
              (t % p.round_period) != p.round_period - 1)
            break;
          const bool lower_turn = turn == 0;
          ++turn;
          if ((waiting & (lower_turn ? 0xffffffffull : ~0xffffffffull)) == 0)
            continue; // nobody on this side
          const bool mine = qh < qt && (half == 0) == lower_turn;
          const int slot = qh & (QCAP - 1);
          const auto slots = __builtin_amdgcn_permlane32_swap(
              (unsigned)(mine ? slot : QCAP), (unsigned)(mine ? slot : QCAP),
              false, false);
          if (lower_turn) {
            has = half == 0 && mine;
            if (has) {
              const uint2 w = queue[slot][tid];
              key = make_key(__uint_as_float(w.x), w.y);
            }
          } else {
            const int slot_upper = (int)slots[1];
            has = half == 0 && slot_upper < QCAP;
            if (has) {
              const uint2 w = queue[slot_upper][tid + 32];
              key = make_key(__uint_as_float(w.x), w.y);
            }
          }
          qh += mine ? 1 : 0;
          PCA_STAT(5, 1);
        }
      }
      // the key enters the lower half; what that half pushes out enters the
      // upper half with the next insertion
      const double out = key_max(best[H - 1], key);
      sorted_insert<H>(best, half ? carry : key);
      const auto ohi = __builtin_amdgcn_permlane32_swap(
          (unsigned)__double2hiint(out), (unsigned)__double2hiint(out), false,
          false);
      const auto olo = __builtin_amdgcn_permlane32_swap(
          (unsigned)__double2loint(out), (unsigned)__double2loint(out), false,
          false);
      if (half)
        carry = __hiloint2double((int)ohi[0], (int)olo[0]);
      changed = true;
    }
    if (changed || finish)
      update_bound(finish);
  };

  {
    feat_acc_t acc_a[SUBS], acc_b[SUBS];
#pragma unroll
    for (int sub = 0; sub < SUBS; ++sub) {
      acc_a[sub] = feat_acc_t{0};
      acc_b[sub] = feat_acc_t{0};
    }
#pragma unroll 1
    for (int t = 0; t <= num_tiles + 1; t += 2) {
      pass(acc_a, acc_b, t);
      if (t + 1 <= num_tiles + 1)
        pass(acc_b, acc_a, t + 1);
    }
  }
#ifdef PCA_FEAT_STATS
  if (lane == 0)
    for (int i = 0; i < 8; ++i)
      atomicAdd(&p.globals->stats[i], st[i]);
#endif

  // ---- the slice's list ----------------------------------------------------
  {
    const size_t list = (size_t)chunk * total_tiles + tile;
    double *dst = p.partial + list * kk * TQ + wave * 32 + col;
#pragma unroll
    for (int j = 0; j < H; ++j) {
      const int e = half * H + j - (KP - kk);
      if (e >= 0)
        dst[(size_t)e * TQ] = best[j];
    }
  }
}

// ---- stage 2 ----------------------------------------------------------------

// One lane per query: the k + 16 smallest keys of the query's slices, to
// cand[q][0 .. k + 16).
template <int KP>
__global__ __launch_bounds__(kBlock) void feat_merge_kernel(KnnFeatParams p) {
  constexpr int TQ = kFeatQueries;
  if (p.globals->odd_rows != 0)
    return;
  const int tid = threadIdx.x;
  const int total_tiles = p.work_start[p.num_segments];
  const int tile = blockIdx.x;
  if (tile >= total_tiles)
    return;
  const int seg = find_segment(p.work_start, p.num_segments, tile);
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int kk = p.k + kFeatSlack;
  if (tid >= TQ)
    return;
  const int pos = tid;
  const int q = y_begin + (tile - p.work_start[seg]) * TQ + pos;
  double best[KP];
#pragma unroll
  for (int j = 0; j < KP; ++j)
    best[j] = (j < KP - kk) ? lowest_key() : feat_empty_key();
  for (int c = 0; c < p.num_chunks; ++c) {
    const double *src =
        p.partial + (size_t)(c * total_tiles + tile) * kk * TQ + pos;
    for (int e = 0; e < kk; ++e) {
      const double key = src[(size_t)e * TQ];
      if (!__any(key < best[KP - 1]))
        break;
      sorted_insert<KP>(best, key);
    }
  }
  if (q < y_end) {
    double *dst = p.cand + (size_t)q * kk;
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const int e = j - (KP - kk);
      if (e >= 0)
        dst[e] = best[j];
    }
  }
}

// Segment of query q: the last b with ptr[b] <= q (segments may be empty).
__device__ __forceinline__ int feat_segment_of(const int64_t *__restrict__ ptr,
                                               int num_segments, int q) {
  int lo = 0, hi = num_segments;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (ptr[mid] <= (int64_t)q)
      lo = mid;
    else
      hi = mid;
  }
  return lo;
}

// One wave per query: exact distances of the listed rows that can matter,
// sorted; flags the query when the list cannot be shown to hold its k nearest
// rows.
template <bool COSINE>
__global__ __launch_bounds__(kBlock) void feat_refine_kernel(KnnFeatParams p) {
  constexpr int WAVES = kBlock / kWave;
  __shared__ __attribute__((aligned(16))) float ys[WAVES][kFeatMaxDim];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int q = blockIdx.x * WAVES + wave;
  if (q >= p.m)
    return;
  const int k = p.k;
  const int kk = k + kFeatSlack;
  const int d = p.d;
  const size_t slot0 = (size_t)q * k;
  // a query the filter cannot serve at all: left to the full second pass
  auto unresolved = [&]() {
    p.redo_q[q] = 1;
    atomicAdd(&p.globals->any_redo, 1);
    atomicAdd(&p.globals->unresolved, 1);
  };
  if (p.globals->odd_rows != 0) {
    if (lane == 0)
      unresolved();
    return;
  }
  const float *yrow = p.y + (size_t)q * d;
  const float inv_sigma = COSINE ? 1.0f : feat_inv_sigma(p.globals->max_bits);
  const float ynorm = COSINE ? p.y_norm[q] : 1.0f;
  // (every lane computes the same values)
  const FeatQuery fq = feat_query<COSINE>(yrow, d, inv_sigma, ynorm);
  if (fq.dead || fq.odd) {
    if (lane == 0) {
      p.out_count[q] = 0;
      p.redo_q[q] = 0;
      if (fq.odd)
        unresolved();
    }
    return;
  }
  // a candidate buffer of the query overflowed: its list may lack rows
  if (p.overflow != nullptr && p.overflow[q] != 0) {
    if (lane == 0) {
      p.out_count[q] = 0;
      unresolved();
    }
    return;
  }
  for (int c = lane; c < d; c += kWave)
    ys[wave][c] = yrow[c];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  const double scale2 =
      COSINE ? kFeatCosScale : (double)inv_sigma * (double)inv_sigma;
  // a lane looks after the list entries lane and lane + 64 (lists of up to
  // 116 entries)
  constexpr int PER = 2;
  double key[PER], lower[PER];
  bool listed[PER];
  int row[PER];
  int listed_count = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = lane + kWave * i;
    key[i] = c < kk ? p.cand[(size_t)q * kk + c] : feat_empty_key();
    listed[i] = key[i] < feat_empty_key();
    row[i] = key_row(key[i]);
    lower[i] = (double)key_dist(key[i]) + fq.shift; // l of the row
    listed_count += __builtin_popcountll(__ballot(listed[i]));
  }

  auto exact = [&](int g) {
    const float *xr = p.x + (size_t)g * d;
    float acc = 0.0f;
    if ((d & 3) == 0) {
      const float4 *x4 = reinterpret_cast<const float4 *>(xr);
      const float4 *y4 = reinterpret_cast<const float4 *>(&ys[wave][0]);
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
          acc = __builtin_fmaf(xr[c], ys[wave][c], acc);
        } else {
          const float dc = xr[c] - ys[wave][c];
          acc = __builtin_fmaf(dc, dc, acc);
        }
      }
    }
    if (COSINE) {
      acc = acc / (p.x_norm[g] * ynorm);
      acc = 1.0f - acc;
    }
    return acc;
  };

  // the first k listed rows, then those whose lower bound does not exceed
  // the largest distance found among them
  float dist[PER];
  bool done[PER];
  auto usable = [&](float v) { return v < kKnnSentinel; }; // (false for NaN)
  int first_good = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    dist[i] = __builtin_nanf("");
    done[i] = false;
    if (listed[i] && lane + kWave * i < k) {
      dist[i] = exact(row[i]);
      done[i] = true;
    }
    first_good += __builtin_popcountll(__ballot(done[i] && usable(dist[i])));
  }
  {
    double reach = __builtin_inf(); // scaled distance rows must stay below
    if (first_good >= k) {
      // the k-th smallest of k values is their largest
      double mine = 0.0;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const double v = done[i] ? (double)dist[i] * scale2 : 0.0;
        mine = v > mine ? v : mine;
      }
#pragma unroll
      for (int sh = 32; sh >= 1; sh >>= 1) {
        const double o = __shfl_xor(mine, sh);
        mine = o > mine ? o : mine;
      }
      reach = mine;
    }
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (listed[i] && !done[i] && lower[i] <= reach) {
        dist[i] = exact(row[i]);
        done[i] = true;
      }
  }
  bool good[PER];
  double ekey[PER];
  int good_count = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    good[i] = done[i] && usable(dist[i]);
    ekey[i] = good[i] ? make_key(dist[i], (uint32_t)row[i]) : empty_key();
    good_count += __builtin_popcountll(__ballot(good[i]));
  }
  // rank among the evaluated rows (keys differ: rows differ)
  int rank[PER] = {0, 0};
  const bool second_half = kk > kWave; // (uniform)
  for (int j = 0; j < kWave; ++j) {
    const double o0 = __shfl(ekey[0], j);
    rank[0] += o0 < ekey[0] ? 1 : 0;
    if (second_half) {
      const double o1 = __shfl(ekey[1], j);
      rank[0] += o1 < ekey[0] ? 1 : 0;
      rank[1] += (o0 < ekey[1] ? 1 : 0) + (o1 < ekey[1] ? 1 : 0);
    }
  }
  // is the list provably complete?  k-th exact distance found, scaled
  double kth = __builtin_inf();
  float kth_plain = __builtin_inff();
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    if (good[i] && rank[i] < k) {
      p.out_idx[slot0 + rank[i]] = row[i];
      if (p.out_dist)
        p.out_dist[slot0 + rank[i]] = dist[i];
    }
    const uint64_t who = __ballot(good[i] && rank[i] == k - 1);
    if (who != 0) {
      kth_plain = __shfl(dist[i], __builtin_ctzll(who));
      kth = (double)kth_plain * scale2;
    }
  }
  // lower bound of every row outside the list: that of the list's last entry
  const double last_lower = kk > kWave ? __shfl(lower[1], kk - 1 - kWave)
                                       : __shfl(lower[0], kk - 1);
  const bool full = listed_count == kk;
  // rows of x that were left out of the filter (far larger than the rest):
  // one lane each evaluates them; one that belongs among the k nearest sends
  // the query to the scans that look at every row
  bool outlier_in_reach = false;
  if (!COSINE && p.globals->n_out > 0) {
    const int n_out = min(p.globals->n_out, kFeatMaxOutliers);
    const int seg = p.ptr_y ? feat_segment_of(p.ptr_y, p.num_segments, q) : 0;
    const int xb = p.ptr_x ? (int)p.ptr_x[seg] : 0;
    const int xe = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
    bool mine = false;
    if (lane < n_out) {
      const int g = p.globals->out_rows[lane];
      if (g >= xb && g < xe) {
        const float e = exact(g);
        mine = usable(e) && (good_count < k || !(e > kth_plain));
      }
    }
    outlier_in_reach = __any(mine);
  }
  // rows that were listed but not evaluated have lower > reach >= kth
  const bool complete = (!full || last_lower > kth) && !outlier_in_reach;
  if (lane == 0) {
    p.out_count[q] = good_count < k ? good_count : k;
    p.redo_q[q] = 0;
    if (!complete) {
      // The k nearest rows all lie at or below the k-th distance found among
      // the listed ones: queue the query for the scan that collects exactly
      // those rows; the full second pass takes what the queue cannot hold.
      const int slot = kth_plain < kKnnSentinel
                           ? atomicAdd(&p.globals->queued, 1)
                           : p.redo_cap;
      if (slot < p.redo_cap) {
        p.redo_list[slot] = q;
        p.redo_tau[slot] = kth_plain;
        atomicAdd(&p.globals->any_redo, 1);
      } else {
        unresolved();
      }
    }
  }
}

// Threshold scan of the queued queries.  A workgroup takes 32 of them (8 per
// wave) and one slice of their segment's rows; a lane evaluates the exact
// distance of one row per step against each of its wave's queries -- the
// reference's chain, one fused multiply-add per component in ascending order
// (csrc/cuda/knn_cuda.cu:55-66) -- and rows at or below a query's threshold
// are appended to that query's hit list.  Rows and query components reach the
// lanes through LDS, 64 rows x 32 components per step, read from global
// memory in full 128-byte pieces; missing rows and components are zeros,
// which leave a chain as it is.  Queries of different segments in one group
// are served one segment after the other.
template <bool COSINE>
__global__ __launch_bounds__(kBlock) void feat_redo_scan_kernel(
    KnnFeatParams p) {
  constexpr int SLAB = 32;   // components per step
  constexpr int STRIDE = 36; // floats per staged row: 16-byte reads of
                             // neighbouring rows fall on distinct banks
  constexpr int G = kFeatRedoGroup;
  constexpr int Q = G / (kBlock / kWave);
  __shared__ __attribute__((aligned(16))) float tile[kWave][STRIDE];
  __shared__ __attribute__((aligned(16))) float ysl[G][SLAB];
  __shared__ int s_q[G], s_xb[G], s_xe[G];
  __shared__ float s_tau[G], s_yn[G];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int group = blockIdx.x / kFeatRedoSlices;
  const int slice = blockIdx.x - group * kFeatRedoSlices;
  const int queued = min(p.globals->queued, p.redo_cap);
  if (group * G >= queued)
    return;
  const int d = p.d;
  if (tid < G) {
    const int j = group * G + tid;
    int q = -1, xb = 0, xe = 0;
    float tau = -__builtin_inff(), yn = 1.0f;
    if (j < queued) {
      q = p.redo_list[j];
      tau = p.redo_tau[j];
      const int seg = p.ptr_y ? feat_segment_of(p.ptr_y, p.num_segments, q) : 0;
      xb = p.ptr_x ? (int)p.ptr_x[seg] : 0;
      xe = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
      if (COSINE)
        yn = p.y_norm[q];
    }
    s_q[tid] = q;
    s_xb[tid] = xb;
    s_xe[tid] = xe;
    s_tau[tid] = tau;
    s_yn[tid] = yn;
  }
  __syncthreads();
  const bool vector_rows = (d & 3) == 0;

  // (everything that decides about a barrier below is the same in all lanes
  // of the workgroup)
  for (int lead = 0; lead < G; ++lead) {
    if (s_q[lead] < 0)
      continue;
    const int xb = s_xb[lead], xe = s_xe[lead];
    bool seen = false;
    for (int e = 0; e < lead; ++e)
      seen |= s_q[e] >= 0 && s_xb[e] == xb && s_xe[e] == xe;
    if (seen)
      continue; // served together with an earlier query of the segment
    const int per_slice =
        ((xe - xb + kFeatRedoSlices - 1) / kFeatRedoSlices + kWave - 1) /
        kWave * kWave;
    const int r0 = min(xe, xb + slice * per_slice);
    const int r1 = min(xe, r0 + per_slice);
    if (r0 >= r1)
      continue;
    bool act[Q];
#pragma unroll
    for (int i = 0; i < Q; ++i) {
      const int e = wave * Q + i;
      act[i] = s_q[e] >= 0 && s_xb[e] == xb && s_xe[e] == xe;
    }

    for (int base = r0; base < r1; base += kWave) {
      float acc[Q];
#pragma unroll
      for (int i = 0; i < Q; ++i)
        acc[i] = 0.0f;
      for (int c0 = 0; c0 < d; c0 += SLAB) {
        __syncthreads(); // the previous step's tile has been read
        if (vector_rows) {
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int idx = tid + kBlock * i;
            const int r = idx >> 3, part = (idx & 7) * 4;
            float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (base + r < r1 && c0 + part < d)
              v = *reinterpret_cast<const float4 *>(
                  p.x + (size_t)(base + r) * d + c0 + part);
            *reinterpret_cast<float4 *>(&tile[r][part]) = v;
          }
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int idx = tid + kBlock * i;
            const int r = idx >> 5, c = idx & 31;
            float v = 0.0f;
            if (base + r < r1 && c0 + c < d)
              v = p.x[(size_t)(base + r) * d + c0 + c];
            tile[r][c] = v;
          }
        }
#pragma unroll
        for (int i = 0; i < G * SLAB / kBlock; ++i) {
          const int idx = tid + kBlock * i;
          const int e = idx >> 5, c = idx & 31;
          const int q = s_q[e];
          float v = 0.0f;
          if (q >= 0 && c0 + c < d)
            v = p.y[(size_t)q * d + c0 + c];
          ysl[e][c] = v;
        }
        __syncthreads();
        float4 xr[SLAB / 4];
#pragma unroll
        for (int g = 0; g < SLAB / 4; ++g)
          xr[g] = *reinterpret_cast<const float4 *>(&tile[lane][4 * g]);
#pragma unroll
        for (int i = 0; i < Q; ++i) {
          if (!act[i])
            continue;
#pragma unroll
          for (int g = 0; g < SLAB / 4; ++g) {
            const float4 a = xr[g];
            const float4 b =
                *reinterpret_cast<const float4 *>(&ysl[wave * Q + i][4 * g]);
            float v = acc[i];
            if (COSINE) {
              v = __builtin_fmaf(a.x, b.x, v);
              v = __builtin_fmaf(a.y, b.y, v);
              v = __builtin_fmaf(a.z, b.z, v);
              v = __builtin_fmaf(a.w, b.w, v);
            } else {
              const float d0 = a.x - b.x, d1 = a.y - b.y;
              const float d2 = a.z - b.z, d3 = a.w - b.w;
              v = __builtin_fmaf(d0, d0, v);
              v = __builtin_fmaf(d1, d1, v);
              v = __builtin_fmaf(d2, d2, v);
              v = __builtin_fmaf(d3, d3, v);
            }
            acc[i] = v;
          }
        }
      }
      const int row = base + lane;
      const float xn = COSINE ? p.x_norm[row < r1 ? row : r0] : 1.0f;
#pragma unroll
      for (int i = 0; i < Q; ++i) {
        if (!act[i])
          continue;
        const int e = wave * Q + i;
        float dist = acc[i];
        if (COSINE) {
          dist = dist / (xn * s_yn[e]);
          dist = 1.0f - dist;
        }
        const bool hit = row < r1 && dist <= s_tau[e]; // (false for NaN)
        const uint64_t hits = __ballot(hit);
        if (hits == 0)
          continue;
        const int j = group * G + e;
        int first = 0;
        if (lane == 0)
          first = atomicAdd(&p.hit_count[j], __builtin_popcountll(hits));
        first = __shfl(first, 0);
        const int at =
            first + __builtin_popcountll(hits & ((1ull << lane) - 1ull));
        if (hit && at < p.hit_cap)
          p.hits[(size_t)j * p.hit_cap + at] = make_key(dist, (uint32_t)row);
      }
    }
  }
}

// Everything for one number of blocks (instantiated in its own translation
// unit so that the sizes build in parallel).
template <int NB>
hipError_t launch_knn_feat_blocks(const KnnFeatParams &p, int kp, bool cosine,
                                  int grid, hipStream_t stream);
template <int NB>
hipError_t launch_feat_pack(const float *x, const float *norms,
                            const float *cls, const unsigned *big, int n,
                            int d, bool cosine, FeatGlobals *g, uint4 *out,
                            hipStream_t stream);

#define PCA_KNN_FEAT_DEFINE(NB_)                                               \
  template <int KP>                                                            \
  static void launch_feat_one_##NB_(const KnnFeatParams &p, bool cosine,       \
                                    int grid, hipStream_t stream) {            \
    if (cosine)                                                                \
      hipLaunchKernelGGL((knn_feat_kernel<NB_, KP, true>), dim3(grid),         \
                         dim3(kBlock), 0, stream, p);                          \
    else                                                                       \
      hipLaunchKernelGGL((knn_feat_kernel<NB_, KP, false>), dim3(grid),        \
                         dim3(kBlock), 0, stream, p);                          \
  }                                                                            \
  template <>                                                                  \
  hipError_t launch_knn_feat_blocks<NB_>(const KnnFeatParams &p, int kp,       \
                                         bool cosine, int grid,                \
                                         hipStream_t stream) {                 \
    switch (kp) {                                                              \
    case 24:                                                                   \
      launch_feat_one_##NB_<24>(p, cosine, grid, stream);                      \
      break;                                                                   \
    case 32:                                                                   \
      launch_feat_one_##NB_<32>(p, cosine, grid, stream);                      \
      break;                                                                   \
    case 48:                                                                   \
      launch_feat_one_##NB_<48>(p, cosine, grid, stream);                      \
      break;                                                                   \
    case 64:                                                                   \
      launch_feat_one_##NB_<64>(p, cosine, grid, stream);                      \
      break;                                                                   \
    case 80:                                                                   \
      launch_feat_one_##NB_<80>(p, cosine, grid, stream);                      \
      break;                                                                   \
    case 116:                                                                  \
      launch_feat_one_##NB_<116>(p, cosine, grid, stream);                     \
      break;                                                                   \
    default:                                                                   \
      return hipErrorInvalidValue;                                             \
    }                                                                          \
    return hipGetLastError();                                                  \
  }                                                                            \
  template <>                                                                  \
  hipError_t launch_feat_pack<NB_>(const float *x, const float *norms,         \
                                   const float *cls, const unsigned *big,      \
                                   int n, int d, bool cosine, FeatGlobals *g,  \
                                   uint4 *out, hipStream_t stream) {           \
    const int spare = FeatShape<NB_>::TILE;                                    \
    const size_t units = (size_t)(n + spare) * FeatShape<NB_>::RSU;            \
    const unsigned grid = (unsigned)((units + kBlock - 1) / kBlock);           \
    if (cosine)                                                                \
      hipLaunchKernelGGL((feat_pack_kernel<NB_, true>), dim3(grid),            \
                         dim3(kBlock), 0, stream, x, norms, cls, nullptr, n,   \
                         d, spare, g, out);                                    \
    else                                                                       \
      hipLaunchKernelGGL((feat_pack_kernel<NB_, false>), dim3(grid),           \
                         dim3(kBlock), 0, stream, x, norms, cls, big, n, d,    \
                         spare, g, out);                                       \
    return hipGetLastError();                                                  \
  }

} // namespace pca
