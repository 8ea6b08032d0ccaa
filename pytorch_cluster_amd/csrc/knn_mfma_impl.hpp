// Feature-space kNN (8 < d <= 128, k <= 64, Euclidean or cosine) on the gfx950
// matrix cores, with results bit-identical to the reference's scalar loop
// (csrc/cuda/knn_cuda.cu:52-78).
//
// Filter.  The matrix cores decide which candidates are LOOKED AT; every
// distance that is kept is evaluated exactly as the reference does.  For the
// Euclidean metric the filter value of a (query, candidate) pair is
//     t = w - 2 x.y,      w = fl(|x|^2) (1 - eps),
// the dot product of the augmented rows (x, w) and (-2 y, 1).  Every fp32
// operand v is split into two bf16 numbers, v = hi + lo + r with
// |lo| <= 2^-8 |v| and |r| <= 2^-17 |v| (the worst cases over all 2^23
// mantissas; bf16 keeps the exponent range of fp32), and the products
// hi*hi + hi*lo + lo*hi of 16 components at a time are one
// v_mfma_f32_32x32x16_bf16 each (exact products, fp32 accumulation): 32
// candidates x 32 queries x 16 components in 8 passes, where the fp32 matrix
// instruction needs 16 passes for 2 components.  A last block of components
// holds w (two parts, times 1) and 1 (twice, times the two parts of -cut),
//     cut = thresh (1 + eps) - fl(|y|^2) (1 - eps)   (rounded up),
// so the SIGN of a result says whether the candidate can still have an exact
// distance below thresh.  Error budget, relative to |x|^2 + |y|^2 + thresh:
// a product x_c y_c misses lo*lo (2^-16 |x_c y_c|) and the residuals
// (2 x 2^-17), all of one sign when y is close to x: 2^-15 |x_c y_c| each,
// 2^-15 (|x|^2 + |y|^2) for -2 x.y, and 2^-17 |x|^2 for w; accumulating
// 3 d + 4 terms, each step within 2^-23 of the running magnitude (which stays
// below 2 (|x|^2 + |y|^2) + thresh), (3 d + 4) 2^-22; norms and the exact
// chain (d + 2) 2^-24 each: 2^-15 + 2^-17 + (3 d + 4) 2^-22 + (d + 2) 2^-23.
// eps = 2^-14 + (3 d + 8) 2^-21 is 1.6 times that or more for every d
// (tests/test_filter_bounds.py holds the inequality against rows whose
// mantissas maximise the split's error, y equal to x).
// Rows whose squared norm is not a moderate finite number enter with zero
// coordinates and w = -1e38 (always looked at; an infinity would meet a zero
// part of another operand and turn into NaN), padding rows with a huge
// positive w and are never candidates whatever the filter says, queries with
// such a norm use the largest finite cut with zero coordinates (look at every
// real row).
//
// The cosine distance 1 - x.y / (|x| |y|) uses the same chain on normalised
// rows: (x / |x|, 1) . (-y / |y|, 1) = 1 - cos, within (4 d + 72) 2^-24 (the
// normalisations) + eps (split and accumulation, magnitudes below 4) of the
// exactly evaluated distance; the cut is thresh + that margin.
// Rows of norm 0 or NaN have a NaN distance in the reference and are padding
// here; a row or query of infinite norm is looked at / looks at everything.
//
// Selection.  A lane gathers the 16 sign bits of a 32-row step with funnel
// shifts and, if any is set, parks (step, mask) in its LDS queue -- one write.
// When a lane runs out of queue entries (and every kMfmaMaxBatch steps at the
// latest) a wave resolves what its lanes have parked, densely: the parked (query, row) pairs of all 64 lanes are compacted into
// one list, lane i takes pair i, 64 + i, ... and evaluates its exact distance
// -- direct differences, one FMA per component in ascending order
// (csrc/cuda/knn_cuda.cu:9-28,55-66), both rows streamed from global memory
// (they are L2 resident) -- and hands the (distance, row) key back through
// LDS to the lane that owns the query, which runs the insertion network.  An
// exact distance costs ~2 d vector instructions for the whole wave whether 1
// or 64 lanes have work, so the dense list is what keeps the re-rank cheap
// even when a handful of queries collect most of the candidates.
//
// Mapping: a workgroup owns 128 queries of one segment (4 waves x 32) and one
// slice of the segment's x rows.  A = 32 candidates (rows i), B = 32 queries
// (columns j): for the block of components 16 b .. 16 b + 15 lane l supplies
// the 8 components 16 b + 8 (l / 32) + 0..7 of candidate l % 32 and of query
// l % 32, and receives, in 16 accumulator registers, the results of query
// l%32 against the 16 candidate rows 8*(v/4) + 4*(l/32) + v%4.  So lanes l and
// l+32 share a query and split its candidates; the lower lane keeps the
// query's list and collects the keys of both lanes' rows in ascending row
// order (so the list's k-th distance is a strict bound), the upper lane
// filters with the same bound.  The lists of a query's slices are merged by
// knn_merge_kernel and exchange their pruning bound through `tau` like the
// slices of the low-dimensional kernels do.
//
// The query operands stay in registers for the whole scan; the candidate rows
// are split once per call (mfma_pack_rows_kernel: per row the hi parts of all
// blocks, then the lo parts of the coordinate blocks, 16 bytes per lane and
// block, rows an odd number of 16-byte units apart so that the reads of
// neighbouring rows fall on distinct LDS banks) and go to a ring of three LDS
// buffers as they are, by LDS-direct loads issued two steps ahead.
#pragma once

#include "device_utils.hpp"
#include "knn_lowd_impl.hpp"
#include "launchers.hpp"

namespace pca {

constexpr int kMfmaQueries = 128;   // queries per workgroup
constexpr int kMfmaEarlySteps = 128; // drains after steps 0, 1, 3, 7, ... below this
constexpr int kMfmaRows = 32;       // candidates per step
constexpr int kMfmaDrainSteps = 8;  // queue entries (parked steps) per lane
constexpr int kMfmaMaxBatch = 128;  // steps between drains at most
// pairs a wave evaluates per pass (248, not 256: with five blocks of
// components the workgroup then needs 53,512 bytes of LDS, and three fit the
// CU's 160 KB, which is handed out in pieces of 1,280 bytes)
constexpr int kMfmaPassPairs = 248;

typedef float mfma_acc_t __attribute__((ext_vector_type(16)));

struct KnnMfmaParams {
  const float *x;
  const float *y;
  const int64_t *ptr_x;
  const int64_t *ptr_y;
  const float *x_sq;   // [n] squared norms of the x rows (cosine: norms)
  const float *y_norm; // [m] norms of the y rows (cosine only)
  const uint4 *x_pack; // [n] packed filter operands (mfma_pack_rows_kernel)
  int n, m, d, num_segments, k;
  const int *work_start; // [num_segments + 1] first 128-query tile per segment
  int num_chunks;        // slices of every segment's x rows
  float *tau;            // [m] shared pruning bounds
  double *partial;       // [num_chunks * tiles][k][128] keys
  // second pass behind another search: nothing runs while *gate is 0, and
  // only tiles with a query whose redo_q entry is non-zero are searched
  const int *gate = nullptr;
  const int *redo_q = nullptr;
};

// Squared row norms, one FMA per component in ascending order.
__global__ __launch_bounds__(kBlock) void row_sqnorm_kernel(
    const float *__restrict__ x, int n, int d, float *__restrict__ out);

// Shape of a packed row for NB blocks of 16 components (the last block holds
// the augmented components): 16-byte units of 8 bf16 numbers.
template <int NB> struct MfmaShape {
  static constexpr int P = 16 * NB;          // components with the padding
  static constexpr int HI = 2 * NB;          // units of hi parts
  static constexpr int LO = 2 * (NB - 1);    // units of lo parts (coordinates)
  static constexpr int UNITS = HI + LO;      // units of a row that hold data
  static constexpr int RSU = UNITS + 1;      // row stride, in memory and in LDS
                                             // (odd: see the header)
  static constexpr int MAX_D = 16 * (NB - 1);
};

__host__ __device__ __forceinline__ double mfma_filter_eps(int d) {
  return 1.0 / 16384.0 + (double)(3 * d + 8) * (1.0 / 2097152.0);
}

__device__ __forceinline__ float mfma_filter_cut(float thresh, float ysq,
                                                 double eps) {
  if (!(ysq <= kFilterNormLimit))
    return __builtin_inff(); // examine everything exactly
  // (1e-20: operands below the bf16 normal range may be flushed to zero by
  // the matrix cores, 400 terms of at most 2^-126 * 2e15 each)
  const double c =
      (double)thresh * (1.0 + eps) - (double)ysq * (1.0 - eps) + 1e-20;
  float f = (float)c;
  if ((double)f < c) // round towards +inf
    f = __uint_as_float(f >= 0.0f ? __float_as_uint(f) + 1u
                                  : __float_as_uint(f) - 1u);
  return f;
}

// Packs the filter operands of the x rows: one thread per 16-byte unit.
// norms: squared norms (Euclidean) or norms (cosine) of the rows.
template <int NB, bool COSINE>
__global__ __launch_bounds__(kBlock) void mfma_pack_rows_kernel(
    const float *__restrict__ x, const float *__restrict__ norms, int n, int d,
    uint4 *__restrict__ out, const int *__restrict__ gate) {
  typedef MfmaShape<NB> S;
  if (gate != nullptr && *gate == 0)
    return;
  const size_t id = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (id >= (size_t)n * S::UNITS)
    return;
  const int row = (int)(id / S::UNITS);
  const int unit = (int)(id - (size_t)row * S::UNITS);
  const bool lo_part = unit >= S::HI;
  const int c0 = 8 * (lo_part ? unit - S::HI : unit);
  const float nv = norms[row];
  // coordinates enter scaled by `scale` (0: not at all); `aug` is w
  float scale, aug;
  if (COSINE) {
    // (a norm of zero over components that are not all zero: their squares
    // underflowed, the dot products need not be zero, and the reference
    // divides them by that zero)
    bool lost_norm = false;
    if (nv == 0.0f)
      for (int c = 0; c < d; ++c)
        lost_norm = lost_norm || x[(size_t)row * d + c] != 0.0f;
    if (lost_norm || (nv > 0.0f && nv < kCosTinyNorm)) { // always looked at
      scale = 0.0f;
      aug = -1e38f;
    } else if (!(nv > 0.0f)) { // a NaN distance anyway: never a candidate
      scale = 0.0f;
      aug = 1.7e38f;
    } else if (nv == __builtin_inff()) { // always looked at
      scale = 0.0f;
      aug = -1e38f;
    } else {
      scale = 1.0f / nv;
      aug = 1.0f;
    }
  } else {
    if (!(nv <= kFilterNormLimit)) {
      scale = 0.0f;
      aug = -1e38f;
    } else {
      scale = 1.0f;
      aug = nv * (float)(1.0 - mfma_filter_eps(d));
    }
  }
  uint32_t part[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int c = c0 + e;
    float v = 0.0f;
    if (c < d)
      v = scale != 0.0f ? x[(size_t)row * d + c] * scale : 0.0f;
    uint32_t hi, lo;
    mc_split(v, hi, lo);
    if (!lo_part) {
      // the augmented components: w in two parts, then 1 twice
      if (c == S::P - 4 || c == S::P - 3) {
        uint32_t whi, wlo = 0;
        if (__builtin_fabsf(aug) < 1e37f)
          mc_split(aug, whi, wlo);
        else
          whi = __float_as_uint(aug) >> 16;
        hi = (c == S::P - 4) ? whi : wlo;
      } else if (c >= S::P - 2) {
        hi = 0x3f80u;
      }
    }
    part[e] = lo_part ? lo : hi;
  }
  // (rows are RSU units apart, like in LDS: a tile is copied as it is)
  out[(size_t)row * S::RSU + unit] =
      make_uint4(part[0] | (part[1] << 16), part[2] | (part[3] << 16),
                 part[4] | (part[5] << 16), part[6] | (part[7] << 16));
}

// A lane's walk over the rows it has parked, in ascending order.
struct MfmaWalk {
  int taken;        // queue entries started
  uint32_t pending; // rows of the current entry still to visit
  int base;         // the lane's first row of that entry's step
};

// NB = blocks of 16 components per row: the coordinates (d <= 16 (NB - 1)) and
// one block with the augmented components.
// NEAREST: the search of the `nearest` operator (one neighbour, limit 1e38,
// the reference's order among equal distances: see device_utils.hpp); the
// lists go through knn_merge_kernel like those of the kNN.
template <int NB, int K, bool COSINE, bool NEAREST = false>
__global__ __launch_bounds__(kBlock, K > 48 ? 2 : 1) void knn_mfma_kernel(KnnMfmaParams p) {
  static_assert(!NEAREST || !COSINE, "nearest is Euclidean");
  constexpr float kLimit = SearchLimit<NEAREST>::value;
  typedef MfmaShape<NB> S;
  constexpr int RSU = S::RSU;
  constexpr int TR = kMfmaRows;
  constexpr int TQ = kMfmaQueries;
  constexpr int TILE_UNITS = TR * RSU; // a tile in global memory and in LDS
  // 1 KB pieces of a tile (one LDS-direct load of a wave each), dealt to the
  // four waves in turn
  constexpr int PIECES = (TILE_UNITS + kWave - 1) / kWave;
  constexpr int MAX_PIECES_PER_WAVE = (PIECES + 3) / 4;
  constexpr int RING = 3; // tile buffers
  constexpr int QCAP = kMfmaDrainSteps;
  constexpr int CAP = kMfmaPassPairs;

  __shared__ __attribute__((aligned(16))) uint4 xs[RING][TR * RSU];
  // parked steps: (step within the batch << 16) | mask of the lane's rows
  __shared__ uint32_t queue[QCAP][kBlock];
  // the step after which every wave of the workgroup drains: written by
  // lanes that are about to run out of queue entries (waves that drain
  // together also wait for memory together).  Entry t & 1 is read during
  // step t and written (for step t + 2) during step t + 1, a barrier later.
  __shared__ int drain_at[2];
  // dense re-rank, per wave: (query, row) pairs and their keys
  __shared__ int2 pairs[kBlock / kWave][CAP];
  __shared__ double results[kBlock / kWave][CAP];

  if (p.gate != nullptr && *p.gate == 0)
    return;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int half = lane >> 5; // which 8 components of a block / which rows
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
  if (p.redo_q != nullptr &&
      !__syncthreads_or(valid && p.redo_q[q] != 0))
    return;
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

  const double eps = mfma_filter_eps(d);
  const float cos_margin =
      (float)(4 * d + 72) * 5.9604644775390625e-08f + (float)eps;

  // ---- per-lane query state ---------------------------------------------
  // (rows of a multiple of four components are read in 16-byte pieces, many
  // at a time: one dependent load per component would cost a memory round
  // trip each)
  const bool vec4 = (d & 3) == 0;
  float ysq = 0.0f;
  if (vec4) {
    const float4 *y4 = reinterpret_cast<const float4 *>(yrow);
#pragma unroll 8
    for (int c = 0; c < d / 4; ++c) {
      const float4 v = y4[c];
      ysq = __builtin_fmaf(v.x, v.x, ysq);
      ysq = __builtin_fmaf(v.y, v.y, ysq);
      ysq = __builtin_fmaf(v.z, v.z, ysq);
      ysq = __builtin_fmaf(v.w, v.w, ysq);
    }
  } else {
#pragma unroll 8
    for (int c = 0; c < d; ++c)
      ysq = __builtin_fmaf(yrow[c], yrow[c], ysq);
  }
  const float ynorm = __builtin_sqrtf(ysq);
  // what the query contributes to the filter: coordinates (scaled), or
  // nothing when the filter is switched off for it
  bool y_filtered; // false: coordinates enter as zeros
  bool y_blind;    // true: the query can have no neighbours at all
  float y_scale;
  if (COSINE) {
    // 0 or NaN: every distance is NaN -- unless the norm is zero only
    // because the squares underflowed: then the dot products still count
    bool lost_norm = false;
    if (ynorm == 0.0f)
      for (int c = 0; c < d; ++c)
        lost_norm = lost_norm || yrow[c] != 0.0f;
    y_blind = !(ynorm > 0.0f) && !lost_norm;
    y_filtered = !y_blind && ynorm < __builtin_inff() && ynorm >= kCosTinyNorm;
    y_scale = y_filtered ? -1.0f / ynorm : 0.0f;
  } else {
    y_blind = false;
    y_filtered = ysq <= kFilterNormLimit;
    y_scale = -2.0f;
  }
  const bool active = valid && !y_blind;
  // B operands: this lane's 8 components of every block of the augmented
  // query, hi parts (all blocks) and lo parts (coordinate blocks).  In the
  // last block the upper lanes hold (0, 0, 0, 0, 1, 1, -cut_hi, -cut_lo); its
  // last word is kept apart (cut_word) and put in place at the instruction.
  mc_bf16x8_t yh[NB];
  mc_bf16x8_t yl[NB - 1];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    // the lane's 8 components of this block, read from clamped addresses
    // (no load depends on a branch) and masked afterwards
    const int cb = 16 * i + 8 * half;
    float comp[8];
    if (i < NB - 1) {
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
    }
    uint32_t hi[8], lo[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int c = cb + e;
      float v = 0.0f;
      if (active) {
        if (i < NB - 1 && c < d)
          v = y_filtered ? comp[e] * y_scale : 0.0f;
        else if (c == S::P - 4 || c == S::P - 3)
          v = 1.0f;
      }
      mc_split(v, hi[e], lo[e]);
    }
    yh[i] = __builtin_bit_cast(
        mc_bf16x8_t, make_uint4(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16),
                                hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16)));
    if (i < NB - 1)
      yl[i < NB - 1 ? i : 0] = __builtin_bit_cast(
          mc_bf16x8_t,
          make_uint4(lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16),
                     lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16)));
  }
  uint32_t cut_word = 0; // (-cut_hi, -cut_lo) of the upper lanes

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - k) ? lowest_key() : SearchLimit<NEAREST>::empty();
  // exact distances must be strictly below thresh
  float thresh = active ? kLimit : -__builtin_inff();
  float shared = kLimit; // bound inherited from other slices / partner
  float posted = kLimit;
  // the rows' last two components are 1; the upper lanes hold the two parts
  // of -cut', cut' = cut + 2^-15 |cut| (what the split may lose never lowers
  // the cut), there; an infinite cut enters as the largest finite bf16 (a
  // lane without a query holds zeros everywhere and never parks)
  auto set_thresh = [&](float v) {
    if (!active)
      return;
    thresh = v;
    float cut;
    if (COSINE)
      cut = y_filtered ? v + cos_margin : __builtin_inff();
    else // (`nearest`: a later row of EQUAL distance can still win the tie)
      cut = mfma_filter_cut(
          NEAREST && v < kLimit ? next_up_positive(v) : v, ysq, eps);
    if (half) {
      const float neg =
          -__builtin_fmaf(__builtin_fabsf(cut), 3.0517578125e-05f, cut);
      uint32_t hi, lo;
      if (__builtin_fabsf(neg) < 1e38f) {
        mc_split(neg, hi, lo);
      } else {
        hi = neg < 0.0f ? 0xff7fu : 0x7f7fu;
        lo = 0;
      }
      cut_word = hi | (lo << 16);
    }
  };
  set_thresh(thresh);

  // ---- tile staging -------------------------------------------------------
  // A tile is TR packed rows, contiguous in global memory, and goes to LDS as
  // it is: LDS-direct loads (16 bytes per lane, a wave fills 1 KB from the
  // address in M0 on), no registers in between.  Tiles are requested two
  // steps ahead; a wave's requests complete in order, so "at most the
  // requests of one tile outstanding" means the older tile has arrived.
  // Rows past the end of the slice are whatever follows in memory (the packed
  // array has TR spare rows); the drain never takes them for candidates.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto request_tile = [&](int t) {
    const uint4 *src = p.x_pack + ((size_t)c_begin + (size_t)t * TR) * RSU;
    const uint32_t dst =
        (uint32_t)(uintptr_t)&xs[t % RING][0]; // byte offset within LDS
#pragma unroll
    for (int e = 0; e < MAX_PIECES_PER_WAVE; ++e) {
      const int piece = wave_u + 4 * e;
      const int u = piece * kWave + lane;
      if (piece < PIECES && u < TILE_UNITS) {
        const uint4 *g = src + u;
        const uint32_t base = dst + (uint32_t)piece * (kWave * 16);
        // (M0 is written and used inside one statement; the compiler keeps
        // nothing in it across statements)
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
#pragma unroll 8
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
        results[wave][i] = make_key(
            dist, NEAREST ? nearest_tie((uint32_t)(pr.y - x_begin))
                          : (uint32_t)pr.y);
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
          const double key = mine ? results[wave][idx - pass0]
                                  : SearchLimit<NEAREST>::empty();
          // NaN and sentinel distances fail the compare like in the
          // reference (csrc/cuda/knn_cuda.cu:48,68).  Equality passes: a
          // pass boundary can separate the two lanes' rows, so a row may
          // arrive after higher rows of its partner -- the key order
          // settles ties.
          const bool ok = mine && key_dist(key) <= thresh &&
                          key_dist(key) < kLimit;
          if (!__any(ok))
            continue;
          sorted_insert<K>(best, ok ? key : SearchLimit<NEAREST>::empty());
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

  if (num_steps > 0)
    request_tile(0);
  if (num_steps > 1)
    request_tile(1);
  if (tid == 0)
    drain_at[0] = drain_at[1] = -1;
  sync_bounds(); // what other slices already know

  // steps [batch_t0, t] are parked and not yet resolved; the first drains
  // come early (after steps 0, 1, 3, 7, ... of the slice), while the lists
  // are empty or their bounds still loose and many rows pass
  int batch_t0 = 0;
  for (int t = 0; t < num_steps; ++t) {
    const int buf = t % RING;
    const bool more = t + 1 < num_steps;
    // this wave's pieces of tile t have arrived; after the barrier so have
    // everybody's, and everybody is done with tile t - 1, whose buffer tile
    // t + 2 may now overwrite
    await_tile(more);
    __syncthreads();
    if (t + 2 < num_steps)
      request_tile(t + 2);

    const uint4 *arow = &xs[buf][col * RSU + half];
    if (NEAREST && t == 0) {
      // `nearest` starts without a bound, and without one every row of the
      // first step would pass the filter (32 exact distances per query, when
      // the whole slice needs about ten).  First bound: the filter values of
      // this step with a cut of zero are |x|^2 - 2 x.y, which orders a
      // query's rows like their distances; every lane takes its smallest one
      // and that row's exact distance, the smaller of a pair's two is the
      // query's bound.  The row itself passes the filter again below and
      // enters the list there.
      mfma_acc_t probe = {0};
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const mc_bf16x8_t ah = __builtin_bit_cast(mc_bf16x8_t, arow[2 * i]);
        if (i < NB - 1) {
          const mc_bf16x8_t al =
              __builtin_bit_cast(mc_bf16x8_t, arow[S::HI + 2 * i]);
          probe = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, yh[i], probe, 0, 0, 0);
          probe = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              ah, yl[i < NB - 1 ? i : 0], probe, 0, 0, 0);
          probe = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, yh[i], probe, 0, 0, 0);
        } else {
          uint4 b = __builtin_bit_cast(uint4, yh[i]);
          b.w = 0;
          probe = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              ah, __builtin_bit_cast(mc_bf16x8_t, b), probe, 0, 0, 0);
        }
      }
      float least = __builtin_inff();
      int least_row = -1;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = 8 * (v / 4) + 4 * half + (v % 4);
        if (row < c_count && probe[v] < least) {
          least = probe[v];
          least_row = row;
        }
      }
      float first = __builtin_inff();
      if (active && least_row >= 0)
        first = exact_distance(q, c_begin + least_row);
      const auto both = __builtin_amdgcn_permlane32_swap(
          __float_as_uint(first), __float_as_uint(first), false, false);
      // (fminf drops a NaN; what is left may be +inf: no bound yet)
      first = __builtin_fminf(__uint_as_float(both[0]),
                              __uint_as_float(both[1]));
      if (first < thresh)
        set_thresh(first);
    }

    // ---- 32 x 32 filter values on the matrix cores ----------------------
    mfma_acc_t acc = {0};
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const mc_bf16x8_t ah = __builtin_bit_cast(mc_bf16x8_t, arow[2 * i]);
      if (i < NB - 1) {
        const mc_bf16x8_t al =
            __builtin_bit_cast(mc_bf16x8_t, arow[S::HI + 2 * i]);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, yh[i], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            ah, yl[i < NB - 1 ? i : 0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, yh[i], acc, 0, 0, 0);
      } else {
        uint4 b = __builtin_bit_cast(uint4, yh[i]);
        b.w = cut_word;
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            ah, __builtin_bit_cast(mc_bf16x8_t, b), acc, 0, 0, 0);
      }
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
      // one entry left: everybody drains after the next step
      if (qn == QCAP - 1)
        drain_at[(t + 1) & 1] = t + 1;
    }
    // Parked steps are resolved when a lane of this wave has no entry left,
    // when some lane of the workgroup announced it one step ago, after
    // kMfmaMaxBatch steps, and at the end.  While lists fill, that is every
    // few steps; later, when hits are rare, a drain (four memory round trips
    // whether it holds 1 pair or 64) comes only every kMfmaMaxBatch steps.
    // (read here, behind the operand reads, not straight after the barrier)
    const bool drain_ordered = drain_at[t & 1] == t;
    if (__any(qn == QCAP) || drain_ordered ||
        t - batch_t0 == kMfmaMaxBatch - 1 || !more ||
        (t < kMfmaEarlySteps && (t & (t + 1)) == 0)) {
      drain(batch_t0 * TR);
      batch_t0 = t + 1;
    }

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

// Everything for one number of blocks (instantiated in its own translation
// unit so the sizes build in parallel).
#define PCA_KNN_MFMA_DEFINE(NB_)                                               \
  template <int KB>                                                            \
  static void launch_one_##NB_(const KnnMfmaParams &p, bool cosine, int grid,  \
                               hipStream_t stream) {                           \
    if (cosine)                                                                \
      hipLaunchKernelGGL((knn_mfma_kernel<NB_, KB, true>), dim3(grid),         \
                         dim3(kBlock), 0, stream, p);                          \
    else                                                                       \
      hipLaunchKernelGGL((knn_mfma_kernel<NB_, KB, false>), dim3(grid),        \
                         dim3(kBlock), 0, stream, p);                          \
  }                                                                            \
  template <>                                                                  \
  hipError_t launch_knn_mfma_blocks<NB_>(const KnnMfmaParams &p, int kbucket,  \
                                         bool cosine, int grid,                \
                                         hipStream_t stream) {                 \
    switch (kbucket) {                                                         \
    case 1: /* the `nearest` search: one entry of an 8-wide list */            \
      hipLaunchKernelGGL((knn_mfma_kernel<NB_, 8, false, true>), dim3(grid),   \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 8:                                                                    \
      launch_one_##NB_<8>(p, cosine, grid, stream);                            \
      break;                                                                   \
    case 16:                                                                   \
      launch_one_##NB_<16>(p, cosine, grid, stream);                           \
      break;                                                                   \
    case 24:                                                                   \
      launch_one_##NB_<24>(p, cosine, grid, stream);                           \
      break;                                                                   \
    case 32:                                                                   \
      launch_one_##NB_<32>(p, cosine, grid, stream);                           \
      break;                                                                   \
    case 48:                                                                   \
      launch_one_##NB_<48>(p, cosine, grid, stream);                           \
      break;                                                                   \
    case 64: /* (one wave per SIMD: the list takes 128 registers) */           \
      launch_one_##NB_<64>(p, cosine, grid, stream);                           \
      break;                                                                   \
    default:                                                                   \
      return hipErrorInvalidValue;                                             \
    }                                                                          \
    return hipGetLastError();                                                  \
  }                                                                            \
  template <>                                                                  \
  hipError_t launch_mfma_pack_rows<NB_>(const float *x, const float *norms,    \
                                        int n, int d, bool cosine, uint4 *out, \
                                        hipStream_t stream,                    \
                                        const int *gate) {                     \
    const size_t units = (size_t)n * MfmaShape<NB_>::UNITS;                    \
    const unsigned grid = (unsigned)((units + kBlock - 1) / kBlock);           \
    if (cosine)                                                                \
      hipLaunchKernelGGL((mfma_pack_rows_kernel<NB_, true>), dim3(grid),       \
                         dim3(kBlock), 0, stream, x, norms, n, d, out, gate);  \
    else                                                                       \
      hipLaunchKernelGGL((mfma_pack_rows_kernel<NB_, false>), dim3(grid),      \
                         dim3(kBlock), 0, stream, x, norms, n, d, out, gate);  \
    return hipGetLastError();                                                  \
  }

} // namespace pca
