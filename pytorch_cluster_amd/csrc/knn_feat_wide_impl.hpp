// Feature-space kNN, first stage, for rows of up to 128 components: the fp16
// filter of knn_feat_impl.hpp (same packed rows, same bounds l and F(l), same
// second stage) in a loop that leaves the matrix cores little to wait for.
// Reference loop: csrc/cuda/knn_cuda.cu:52-78.
//
// What the loop is built around (stripped-loop measurements on the device):
//   * the matrix instructions themselves, their A operands read from LDS, the
//     sign masks and a barrier per tile run at the matrix cores' own rate;
//   * bringing the tiles of packed rows from the L2 into LDS does not -- its
//     cost is proportional to the bytes staged per matrix instruction.  So a
//     workgroup is eight waves that share one tile, and a wave multiplies
//     every A operand it reads with the operands of TWO blocks of 32 queries
//     (512 queries per staged tile: a quarter of the bytes of four waves with
//     one block each);
//   * the sorted lists of the other kernel cost registers (one workgroup of
//     four waves had to hold 128 lists) and issue slots in the loop.  Here a
//     lane that finds a value below the cut parks (value, row) in a small
//     LDS queue of its own; the queues are written to the queries' candidate
//     buffers in global memory one tile later (stores that have just been
//     issued would be waited for together with the tile loads: one counter
//     covers both); and only at checkpoints --
//     after 64, 128, 256, ... rows of the piece, or when a buffer fills up --
//     the lane that owns a query runs the new candidates through a sorted
//     list of the k smallest VALUES (fp32, one v_med3_f32 per slot and
//     insertion; kept in global memory between checkpoints), takes the new
//     bound U = F(l_k) from it and drops the buffer entries above it.
//
// The cut inside the matrix product.  The filter's test is s < cut with
// s = W + sum_c h(X_c) h(-2 Y_c).  The block that carries W has thirteen
// unused components; the packed rows hold the powers of two 2^15, 2^5, 2^-5
// in components 3..5 and 8..10 of it, and the lane that owns a query puts
// -c_rep, split into three fp16 numbers (c_rep = p0 2^15 + p1 2^5 + p2 2^-5,
// 33 bits: any float of the range is represented exactly or rounded up), into
// the matching components of the query's operand.  The chain then delivers
// acc = s - c_rep up to its own rounding, and a lane only has to gather sign
// bits (16 v_alignbit_b32 per 16 values) where the other kernel subtracts
// first.  Budget: the chain has d + 22 terms instead of d + 16 and its
// running magnitude grows by |c_rep|, so
//     |acc - (S - c_rep)| <= (d + 22) 2^-22 (2.01 (|X|^2 + |Y|^2) + |c_rep|)
// (S: the exact sum of the terms of s).  The first part is inside what the
// error analysis of knn_feat_impl.hpp leaves to accumulation (0.15 x 2^-10
// (|X|^2 + |Y|^2); 0.074 are used at 128 components); the second part,
// D(c) = (d + 23) 2^-22 |c_rep| (one unit for the float additions below), is
// made up for explicitly:
//   * c_rep >= cut + D(c_rep): a row with l <= U has a negative acc;
//   * the value kept for a flagged row is acc + float_below(c_rep - D), which
//     lies in [S - room - 2 D, S + room]: still a lower bound of the row's
//     distance once the shift is added, and F(l + 2 D) an upper bound.
// While a query's list is not full there is no cut: its operand carries
// zeros there, every row counts as flagged and acc is s itself.
//
// Work: the (tile of 512 queries, 64-row unit of the tile's segment) pairs of
// a call form one line; workgroup w takes the w-th of `grid` equal stretches
// of it, piece by piece (a piece: one tile of queries, a contiguous range of
// units).  Pieces of a tile share their bounds through `tau` as the slices of
// the other kernel do; a gather kernel unites their buffers into the same
// list of k + 16 (value, row) keys per query that feat_refine_kernel reads.
#pragma once

#include "knn_feat_impl.hpp"

#ifndef PCA_WIDE_EXP
#define PCA_WIDE_EXP 0 // (timing experiments: parts of the loop switched off)
#endif

namespace pca {

constexpr int kWideWaves = 8;
constexpr int kWideThreads = kWideWaves * kWave; // 512
constexpr int kWideQueries = kWideThreads;       // one owned query per lane
constexpr int kWideTileRows = 64;                // rows per staged tile (unit)
constexpr int kWideRing = 4;                     // LDS buffers of the tile ring
constexpr int kWideMaxDim = 128;
constexpr int kWideQueue = 8;                    // parked values per lane

// the cut's three fp16 parts are multiplied by these (fp16 bit patterns)
constexpr uint32_t kWideScale0 = 0x7800u; // 2^15
constexpr uint32_t kWideScale1 = 0x5000u; // 2^5
constexpr uint32_t kWideScale2 = 0x2800u; // 2^-5

struct KnnFeatWideParams {
  KnnFeatParams base;
  const int *tile_start;        // [num_segments + 1] first 512-query tile
  const long long *unit_start;  // [num_segments + 1] first (tile, unit) pair
  int cap;                      // buffer entries per (piece, query, half)
  int ckpt_growth;              // next checkpoint at tile t * this / 16 (> 16)
  // candidate buffers: one per query and half of the wave that found the
  // values (the two lanes that share a query's values write their own)
  uint2 *buf;                   // [pieces][8 waves][2][cap][64] (value, row)
  int *buf_count;               // [pieces][2][512] entries at the piece's end
  float *lists;                 // [grid][K][512] the owners' sorted values
  struct WideOwner *owners;     // [grid][512] the owners' state
  int *overflow;                // [m] 1: a buffer of the query overflowed
};

// State of the lane that owns a query, kept in global memory between
// checkpoints (the loop itself has no use for it, and registers are what the
// loop is short of).
struct WideOwner {
  double bound;    // U: upper bound of the query's final k-th distance
  double fold_err; // largest D of the piece's cuts so far
  double shift;    // l = value + shift
  double widen;    // F(l) = (l + widen) * grow
  float posted;    // what this piece has published to `tau`
  float tau_seen;  // what the query's other pieces have
  int seen[2];     // buffer entries the list has taken, per half
  int flags;       // 1: the list exists, 2: a buffer overflowed
  int pad;
};

// What a checkpoint hands back to the loop.
struct WideCut {
  uint32_t part01, part2; // the three fp16 parts of -c_rep
  float recon;            // what is added to a flagged value
  int fill;               // no cut: every row counts
  int kept[2];            // entries left in the two buffers
  int rounds;             // insertions the wave ran (statistics)
};

// D(c) of the header.
__device__ __forceinline__ double wide_fold_err(int d, double c_rep) {
  return (double)(d + 23) * (1.0 / 4194304.0) * __builtin_fabs(c_rep);
}

// Splits c into three fp16 numbers (bit patterns, sign included) with
// rep = p0 2^15 + p1 2^5 + p2 2^-5 >= c and returns rep; false when c is
// beyond the range (the caller then works without a cut).
__device__ __forceinline__ bool wide_cut_parts(double c, uint32_t (&p)[3],
                                               double &rep) {
  const bool neg = c < 0.0;
  const double a = neg ? -c : c;
  if (!(a < 2.0e9))
    return false;
  // magnitudes, each part truncated towards zero
  const uint32_t a0 = feat_h_down(a * (1.0 / 32768.0));
  const double r0 = a - feat_h_value(a0) * 32768.0;
  const uint32_t a1 = feat_h_down(r0 * (1.0 / 32.0));
  const double r1 = r0 - feat_h_value(a1) * 32.0;
  uint32_t a2 = feat_h_down(r1 * 32.0);
  double r2 = r1 - feat_h_value(a2) * (1.0 / 32.0);
  if (!neg && r2 > 0.0) {
    // what is left would make rep < c: the next fp16 above (from zero: the
    // smallest normal number)
    a2 = a2 == 0 ? 0x0400u : a2 + 1u;
    if (a2 > 0x7bffu)
      return false;
    r2 = r1 - feat_h_value(a2) * (1.0 / 32.0);
  }
  const double mag = a - r2;
  rep = neg ? -mag : mag;
  const uint32_t sign = neg ? 0x8000u : 0u;
  p[0] = a0 ? (a0 | sign) : 0u;
  p[1] = a1 ? (a1 | sign) : 0u;
  p[2] = a2 ? (a2 | sign) : 0u;
  return true;
}

// Largest float that is <= v.
__device__ __forceinline__ float wide_float_below(double v) {
  float f = (float)v;
  if ((double)f > v) {
    const uint32_t u = __float_as_uint(f);
    if (f > 0.0f)
      f = __uint_as_float(u - 1u);
    else if (f < 0.0f)
      f = __uint_as_float(u + 1u);
    else
      f = -1.401298464324817e-45f;
  }
  return f;
}

// Segment s with unit_start[s] <= pos < unit_start[s + 1].
__device__ __forceinline__ int wide_segment_of(
    const long long *__restrict__ unit_start, int num_segments,
    long long pos) {
  int lo = 0, hi = num_segments;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (unit_start[mid] <= pos)
      lo = mid;
    else
      hi = mid;
  }
  return lo;
}

// The stretch of the line a workgroup takes.
__device__ __forceinline__ long long wide_stretch(long long total, int grid) {
  return (total + grid - 1) / grid;
}

// A checkpoint of the lane that owns a query (all lanes of a wave together).
// The entries the query's two buffers have got since the last checkpoint go
// through the sorted list of the k smallest values (`list`, [K] floats 512
// apart); the list's k-th value and what the query's other pieces have
// published give the bound U; entries above the new cut leave the buffers
// when one is half full (always at the piece's end, where the counts are
// written to count_out[0] and count_out[512]).  col_buf: the query's column
// of the first buffer (entries 64 apart; the second buffer cap entries on).
template <int K, bool COSINE>
__device__ __attribute__((noinline)) WideCut wide_checkpoint(
    WideOwner *o_mem, uint2 *col_buf, float *list, int cap, int count0,
    int count1, int d, int k, float *tau_q, bool own_active, bool last,
    int *count_out, int *overflow_q) {
  // this wave's appends have reached the L2 (the loads below are device-scope
  // atomics: they see them there; no cache is written back or invalidated)
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  WideOwner o = *o_mem;
  double bound = o.bound, fold_err = o.fold_err;
  float posted = o.posted, tau_seen = o.tau_seen;
  const bool have_list = (o.flags & 1) != 0;
  bool over = (o.flags & 2) != 0;
  WideCut out;
  out.rounds = 0;
  int n[2] = {count0, count1};
#pragma unroll
  for (int h = 0; h < 2; ++h)
    if (n[h] > cap) {
      over = true;
      n[h] = cap;
    }
  float best[K];
  if (have_list) {
#pragma unroll
    for (int j = 0; j < K; ++j)
      best[j] = list[(unsigned)(j * kWideQueries)];
  } else {
#pragma unroll
    for (int j = 0; j < K; ++j)
      best[j] = j < K - k ? -__builtin_inff() : __builtin_inff();
  }
  int most[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    uint2 *src = col_buf + (size_t)h * cap * kWave;
    most[h] = n[h];
#pragma unroll
    for (int sh = 32; sh >= 1; sh >>= 1)
      most[h] = max(most[h], __shfl_xor(most[h], sh));
    const int first = o.seen[h];
    int least = first;
#pragma unroll
    for (int sh = 32; sh >= 1; sh >>= 1)
      least = min(least, __shfl_xor(least, sh));
    // (CHUNK loads in flight at a time: one after the other, each would
    // wait a full trip to the L2)
    constexpr int CHUNK = 16;
#pragma unroll 1
    for (int e0 = least; e0 < most[h]; e0 += CHUNK) {
      float keys[CHUNK];
#pragma unroll
      for (int i = 0; i < CHUNK; ++i) {
        const int e = e0 + i;
        keys[i] = __builtin_inff();
        if (e >= first && e < n[h])
          keys[i] = __uint_as_float(__hip_atomic_load(
              reinterpret_cast<const uint32_t *>(src + (size_t)e * kWave),
              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      }
#pragma unroll
      for (int i = 0; i < CHUNK; ++i) {
        const float key = keys[i];
        if (!__any(key < best[K - 1]))
          continue;
        ++out.rounds;
#pragma unroll
        for (int j = K - 1; j >= 1; --j)
          best[j] = __builtin_amdgcn_fmed3f(best[j - 1], best[j], key);
        best[0] = __builtin_fminf(best[0], key);
      }
    }
    o.seen[h] = n[h];
  }
#pragma unroll
  for (int j = 0; j < K; ++j)
    list[(unsigned)(j * kWideQueries)] = best[j];

  // the bound: from the list's k-th value and from the query's other pieces
  const float kth = best[K - 1];
  float cut_plain = __builtin_inff(); // s < cut_plain: the row can matter
  if (own_active) {
    if (kth < __builtin_inff()) {
      const double l = (double)kth + o.shift;
      const double u = (l + o.widen + 2.0 * fold_err) *
                       (COSINE ? 1.0 : feat_grow(d));
      bound = u < bound ? u : bound;
    }
    float own = bound < 3.0e38 ? feat_float_above(bound) : __builtin_inff();
    own = __builtin_fmaxf(own, 0.0f);
    const float now = __hip_atomic_load(tau_q, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
    tau_seen = __builtin_fminf(tau_seen, now);
    if (own < tau_seen && (own < posted * 0.999f || (last && own < posted))) {
      __hip_atomic_fetch_min(reinterpret_cast<int *>(tau_q),
                             (int)__float_as_uint(own), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      posted = own;
    } else if (tau_seen < posted) {
      posted = tau_seen;
      bound = (double)tau_seen < bound ? (double)tau_seen : bound;
    }
    if (bound < __builtin_inf())
      cut_plain = feat_float_above(bound - o.shift);
  } else {
    cut_plain = -__builtin_inff();
  }

  // entries above the new cut leave the buffers
  const bool tidy = __any(n[0] > cap / 2 || n[1] > cap / 2) || last;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if (tidy) {
      uint2 *src = col_buf + (size_t)h * cap * kWave;
      int kept = 0;
      constexpr int CHUNK = 8;
#pragma unroll 1
      for (int e0 = 0; e0 < most[h]; e0 += CHUNK) {
        unsigned long long w[CHUNK];
#pragma unroll
        for (int i = 0; i < CHUNK; ++i) {
          w[i] = 0;
          if (e0 + i < n[h])
            w[i] = __hip_atomic_load(
                reinterpret_cast<const unsigned long long *>(
                    src + (size_t)(e0 + i) * kWave),
                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // (kept <= e0 + i: a store never reaches an entry not yet loaded)
#pragma unroll
        for (int i = 0; i < CHUNK; ++i) {
          if (e0 + i < n[h] &&
              __uint_as_float((uint32_t)w[i]) < cut_plain) {
            __hip_atomic_store(reinterpret_cast<unsigned long long *>(
                                   src + (size_t)kept * kWave),
                               w[i], __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            ++kept;
          }
        }
      }
      n[h] = kept;
      o.seen[h] = kept;
    }
    out.kept[h] = n[h];
  }
  o.bound = bound;
  o.posted = posted;
  o.tau_seen = tau_seen;
  o.flags = 1 | (over ? 2 : 0);
  out.part01 = 0;
  out.part2 = 0;
  out.recon = 0.0f;
  out.fill = 0;
  if (last) {
    count_out[0] = n[0];
    count_out[kWideQueries] = n[1];
    if (over && overflow_q != nullptr)
      *overflow_q = 1;
    return out;
  }

  // the cut for the query's operand
  uint32_t part[3] = {0, 0, 0};
  float my_recon = 0.0f;
  bool my_fill = own_active;
  if (own_active && cut_plain < __builtin_inff()) {
    const double c0 = (double)cut_plain;
    const double want = c0 + wide_fold_err(d, c0) * 1.002 + 1e-30;
    double rep = 0.0;
    if (wide_cut_parts(want, part, rep)) {
      const double err = wide_fold_err(d, rep);
      // (rep >= want covers D(rep) as long as rep is within 0.2 % of c0;
      // checked, not assumed)
      if (rep >= c0 + err) {
        // (the operand carries -c_rep)
#pragma unroll
        for (int i = 0; i < 3; ++i)
          part[i] = part[i] ? part[i] ^ 0x8000u : 0u;
        my_fill = false;
        my_recon = wide_float_below(rep - err);
        // (the list may hold values of every cut so far)
        fold_err = err > fold_err ? err : fold_err;
      } else {
        part[0] = part[1] = part[2] = 0;
      }
    } else {
      part[0] = part[1] = part[2] = 0;
    }
  }
  o.fold_err = fold_err;
  *o_mem = o;
  out.part01 = part[0] | (part[1] << 16);
  out.part2 = part[2];
  out.recon = my_recon;
  out.fill = my_fill ? 1 : 0;
  return out;
}

// K: width of the owners' lists (>= k; the first K - k slots hold -inf).
template <int NB, int K, bool COSINE>
__global__ __launch_bounds__(kWideThreads, 1) void knn_feat_wide_kernel(
    KnnFeatWideParams P) {
  typedef FeatShape<NB> S;
  constexpr int RSU = S::RSU;
  constexpr int TILE = kWideTileRows;
  constexpr int SUBS = TILE / kFeatStep; // 2
  static_assert(SUBS == 2, "a tile is two steps");
  constexpr int TILE_UNITS = TILE * RSU;
  constexpr int PIECES = (TILE_UNITS + kWave - 1) / kWave;
  constexpr int MAXP = (PIECES + kWideWaves - 1) / kWideWaves;
  constexpr int RING = kWideRing;
  constexpr int RB = 2;
  const KnnFeatParams &p = P.base;

  __shared__ __attribute__((aligned(16))) uint4 xs[RING][TILE_UNITS];
  __shared__ __attribute__((aligned(16))) uint4 dump[kWideThreads][4];
  // parked (value, row | block << 31) pairs of every lane: a ring of QCAP
  __shared__ uint2 queue[kWideQueue][kWideThreads];

  if (p.globals->odd_rows != 0)
    return; // everything is searched by the other kernel

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int half = lane >> 5;
  const int col = lane & 31;
  const int d = p.d;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);

  const long long total = P.unit_start[p.num_segments];
  if (total == 0)
    return;
  const long long stretch = wide_stretch(total, (int)gridDim.x);
  long long pos = (long long)blockIdx.x * stretch;
  const long long pos_end = min(total, pos + stretch);
  const float inv_sigma = COSINE ? 1.0f : feat_inv_sigma(p.globals->max_bits);
  float *my_list = P.lists + (size_t)blockIdx.x * K * kWideQueries + tid;

#ifdef PCA_FEAT_STATS
  unsigned long long st[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#define PCA_WSTAT(i, n) st[i] += (n)
#else
#define PCA_WSTAT(i, n)
#endif

#pragma unroll 1
  while (pos < pos_end) {
    // ---- the piece ---------------------------------------------------------
    const int seg = wide_segment_of(P.unit_start, p.num_segments, pos);
    const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
    const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
    const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
    const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
    const int units = (x_end - x_begin + TILE - 1) / TILE;
    const long long rel = pos - P.unit_start[seg];
    const int tile_in_seg = (int)(rel / units);
    const int u0 = (int)(rel - (long long)tile_in_seg * units);
    const int u1 = (int)min((long long)units, u0 + (pos_end - pos));
    const int tile = P.tile_start[seg] + tile_in_seg;
    const int piece = (int)blockIdx.x + tile;
    pos += u1 - u0;

    const int c_begin = x_begin + u0 * TILE;
    const int c_count = min(x_end, x_begin + u1 * TILE) - c_begin;
    const int num_tiles = u1 - u0;
    const int q_tile = y_begin + tile_in_seg * kWideQueries;
    // the query this lane owns, and the two whose values it sees
    const int q_own = q_tile + wave * kWave + lane;
    const bool own_valid = q_own < y_end;
    const float *yrow_own = p.y + (size_t)(own_valid ? q_own : y_begin) * d;
    const float ynorm_own = COSINE && own_valid ? p.y_norm[q_own] : 1.0f;
    const FeatQuery fq = feat_query<COSINE>(yrow_own, d, inv_sigma, ynorm_own);
    const bool own_active = own_valid && !fq.dead && !fq.odd;
    // (element 0 of a swap: in an upper lane, the lower lane's value; element
    // 1: in a lower lane, the upper lane's)
    auto partner = [&](uint32_t v) __attribute__((always_inline)) {
      const auto both = __builtin_amdgcn_permlane32_swap(v, v, false, false);
      return half ? both[0] : both[1];
    };
    const bool other_active = partner(own_active ? 1u : 0u) != 0;
    const float other_ynorm = __uint_as_float(partner(__float_as_uint(ynorm_own)));

    // B operands of the two blocks: this lane's 8 components of every block
    // (the piece's own copy of d keeps the offsets below from being computed
    // once for all pieces and held in registers across the loop)
    int d_here = d;
    asm volatile("" : "+s"(d_here));
    feat_f16x8_t yh[RB][NB];
    const bool vec4 = (d_here & 3) == 0;
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const int qb = q_tile + wave * kWave + b * 32 + col;
      const bool act = b == half ? own_active : other_active;
      const float yn = b == half ? ynorm_own : other_ynorm;
      const float *yrow = p.y + (size_t)(qb < y_end ? qb : y_begin) * d_here;
      const float y_scale =
          COSINE ? (act ? -1024.0f / yn : 0.0f) : -2.0f * inv_sigma;
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        uint32_t hb[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (i < NB - 1) {
          const int cb = 16 * i + 8 * half;
          float comp[8];
          if (vec4) {
            const float4 a =
                *reinterpret_cast<const float4 *>(yrow + min(cb, d_here - 4));
            const float4 c =
                *reinterpret_cast<const float4 *>(yrow + min(cb + 4, d_here - 4));
            comp[0] = a.x, comp[1] = a.y, comp[2] = a.z, comp[3] = a.w;
            comp[4] = c.x, comp[5] = c.y, comp[6] = c.z, comp[7] = c.w;
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              comp[e] = yrow[min(cb + e, d_here - 1)];
          }
#pragma unroll
          for (int e = 0; e < 8; ++e)
            hb[e] = (act && cb + e < d_here) ? feat_h(comp[e] * y_scale) : 0u;
        } else if (half == 0 && act) {
          hb[0] = 0x7800u; // 2^15
          hb[1] = 0x4c00u; // 2^4
          hb[2] = 0x2000u; // 2^-7
        }
        yh[b][i] = __builtin_bit_cast(
            feat_f16x8_t,
            make_uint4(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16),
                       hb[4] | (hb[5] << 16), hb[6] | (hb[7] << 16)));
        // (one operand at a time: all the rows' loads up front would not fit
        // the registers)
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- owner state -------------------------------------------------------
    WideOwner *const my_owner =
        P.owners + (size_t)blockIdx.x * kWideQueries + tid;
    {
      WideOwner o;
      o.bound = __builtin_inf();
      o.fold_err = 0.0;
      o.shift = fq.shift;
      o.widen = fq.widen;
      o.posted = __builtin_inff();
      o.tau_seen = own_valid
                       ? __hip_atomic_load(&p.tau[q_own], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT)
                       : __builtin_inff();
      o.seen[0] = o.seen[1] = 0;
      o.flags = 0;
      o.pad = 0;
      *my_owner = o;
    }
    // per block, for the values this lane sees: what is added to a flagged
    // value, whether the block's query has no cut yet (every row counts), and
    // the entries this lane has written to the query's buffer of its half
    float recon[RB] = {0.0f, 0.0f};
    bool fill[RB];
    int written[RB] = {0, 0};
#pragma unroll
    for (int b = 0; b < RB; ++b)
      fill[b] = b == half ? own_active : other_active;
    bool need_ckpt = false;
    bool fresh_stores = false; // stores issued since the last tile request
    int qh = 0, qt = 0;        // the lane's queue: entries qh .. qt - 1

    // (wave-uniform: a scalar base for the stores and loads below)
    uint2 *const my_buf =
        P.buf + ((size_t)piece * kWideWaves + wave_u) * 2 * P.cap * kWave;

    // ---- tile staging ------------------------------------------------------
    // (scalar base, one 32-bit lane offset: no per-lane pointers to keep)
    auto request_tile = [&](int t) __attribute__((always_inline)) {
      const uint4 *src = p.x_pack + ((size_t)c_begin + (size_t)t * TILE) * RSU;
      const uint32_t dst = (uint32_t)(uintptr_t)&xs[t % RING][0];
#pragma unroll
      for (int e = 0; e < MAXP; ++e) {
        const int pc = wave_u + kWideWaves * e;
        const int u = pc * kWave + lane;
        if (pc < PIECES && (TILE_UNITS % kWave == 0 || u < TILE_UNITS)) {
          const uint4 *g = src + pc * kWave; // (uniform)
          const uint32_t base = dst + (uint32_t)pc * (kWave * 16);
          asm volatile("s_mov_b32 m0, %2\n\t"
                       "s_nop 0\n\t"
                       "global_load_lds_dwordx4 %0, %1"
                       :
                       : "v"(lane * 16), "s"(g), "s"(base)
                       : "memory");
        }
      }
    };
    __syncthreads(); // everybody has left the previous piece
#pragma unroll
    for (int r = 0; r < RING - 1; ++r)
      if (r < num_tiles)
        request_tile(r);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---- parked values -------------------------------------------------------
    // The queues go to the buffers: entry (value, row) of block b to slot
    // written[b] of the buffer of (query, this lane's half).
    auto flush = [&]() __attribute__((always_inline)) {
#pragma unroll 1
      while (__any(qh != qt)) {
        if (qh != qt) {
          const uint2 e = queue[qh & (kWideQueue - 1)][tid];
          ++qh;
          const int b = (int)(e.y >> 31);
          const int at = b ? written[1] : written[0];
          written[0] += b ? 0 : 1;
          written[1] += b ? 1 : 0;
          int slot = lane;
          asm volatile("" : "+v"(slot));
          slot = (slot & 31) + b * 32 + (slot >> 5) * P.cap * kWave;
          if (at < P.cap)
            *reinterpret_cast<uint2 *>(reinterpret_cast<char *>(my_buf) +
                                       (unsigned)((at * kWave + slot) * 8)) =
                make_uint2(e.x, e.y & 0x7fffffffu);
          if (at >= P.cap - TILE)
            need_ckpt = true;
        }
      }
    };
    // parks a flagged value (the queue is flushed first when a lane's is full)
    auto park = [&](int b, float value, int row, bool on)
                    __attribute__((always_inline)) {
      if (__any(on && qt - qh >= kWideQueue)) {
        flush();
        fresh_stores = true;
      }
      if (on) {
        queue[qt & (kWideQueue - 1)][tid] = make_uint2(
            __float_as_uint(value), (uint32_t)row | ((uint32_t)b << 31));
        ++qt;
      }
    };

    // ---- what a step leaves: masks and minima of `old` ------------------------
    // bit 15 - v of mask[b]: value v of block b is negative
    auto signs = [&](const feat_acc_t (&old)[RB], uint32_t (&mask)[RB],
                     float (&lo)[RB]) __attribute__((always_inline)) {
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        const feat_acc_t &a = old[b];
        float m0 = min3f(a[0], a[1], a[2]);
        float m1 = min3f(a[3], a[4], a[5]);
        float m2 = min3f(a[6], a[7], a[8]);
        float m3 = min3f(a[9], a[10], a[11]);
        float m4 = min3f(a[12], a[13], a[14]);
        m0 = min3f(m0, m1, m2);
        m3 = min3f(m3, m4, a[15]);
        lo[b] = __builtin_fminf(m0, m3);
        uint32_t mk = __float_as_uint(a[0]) >> 31;
#pragma unroll
        for (int v = 1; v < 16; ++v)
          mk = __builtin_amdgcn_alignbit(mk, __float_as_uint(a[v]), 31);
        mask[b] = mk & 0xffffu;
      }
    };

    // The flagged values of a finished step go to the buffers.  row0: first
    // row of the step; rec / all: recon and fill as they were when the step's
    // matrix instructions were issued.
    auto events = [&](const feat_acc_t (&old)[RB], uint32_t (&mask)[RB],
                      float (&lo)[RB], int pos0, const float (&rec)[RB],
                      const bool (&all)[RB]) __attribute__((always_inline)) {
      const bool tail = pos0 + kFeatStep > c_count;
      bool any = false, several = false;
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        if (all[b])
          mask[b] = 0xffffu;
        if (tail) {
#pragma unroll
          for (int v = 0; v < 16; ++v)
            if (pos0 + 8 * (v / 4) + 4 * half + (v % 4) >= c_count)
              mask[b] &= ~(1u << (15 - v));
        }
        any |= mask[b] != 0;
        several |= (mask[b] & (mask[b] - 1u)) != 0;
      }
      PCA_WSTAT(0, 1);
      if (!__any(any))
        return;
      PCA_WSTAT(1, 1);
      const int row0 = c_begin + pos0 + 4 * half;
      if ((PCA_WIDE_EXP & 2) || (!tail && !__any(several))) {
        // at most one flagged value per lane and block: it is the minimum
#pragma unroll
        for (int b = 0; b < RB; ++b) {
          const int v = __builtin_clz(mask[b] | 1u) - 16;
          park(b, lo[b] + rec[b], row0 + 8 * (v >> 2) + (v & 3),
               mask[b] != 0);
        }
        return;
      }
      PCA_WSTAT(2, 1);
      // several: the lane's 16 values go to LDS and come back one by one,
      // addressed by the mask's bits
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        if (!__any(mask[b] != 0))
          continue;
        const feat_acc_t &a = old[b];
        if (mask[b] != 0) {
#pragma unroll
          for (int g = 0; g < 4; ++g)
            dump[tid][g] = make_uint4(
                __float_as_uint(a[4 * g]), __float_as_uint(a[4 * g + 1]),
                __float_as_uint(a[4 * g + 2]), __float_as_uint(a[4 * g + 3]));
        }
        uint32_t bits = mask[b];
        const float *mine = reinterpret_cast<const float *>(&dump[tid][0]);
#pragma unroll 1
        while (__any(bits != 0)) {
          const int v = __builtin_clz(bits | 1u) - 16;
          const bool on = bits != 0;
          bits &= ~(0x8000u >> v);
          const float s = on ? mine[v] : 0.0f;
          park(b, s + rec[b], row0 + 8 * (v >> 2) + (v & 3), on);
          PCA_WSTAT(3, 1);
        }
      }
    };

    // ---- checkpoint: the owners take their new candidates in ----------------
    // (a call, not inlined: the rare path's registers stay out of the loop's)
    auto checkpoint = [&](bool last) __attribute__((always_inline)) {
      PCA_WSTAT(4, 1);
      flush();
      // the entries of the owned query: this lane's, and the other half's
      const int mine = half ? written[1] : written[0];
      const int theirs = (int)partner((uint32_t)(half ? written[0] : written[1]));
      const WideCut cut = wide_checkpoint<K, COSINE>(
          my_owner, my_buf + lane, my_list, P.cap, half ? theirs : mine,
          half ? mine : theirs, d, p.k, own_valid ? &p.tau[q_own] : nullptr,
          own_active, last,
          &P.buf_count[(size_t)piece * 2 * kWideQueries + tid],
          own_valid ? &P.overflow[q_own] : nullptr);
      PCA_WSTAT(5, cut.rounds);
      fresh_stores = true;
      if (last)
        return;
      // what is left in the buffers: the own half's count, and the other
      // half's back to the lane that writes there
      {
        const int kept_mine = half ? cut.kept[1] : cut.kept[0];
        const int kept_theirs = half ? cut.kept[0] : cut.kept[1];
        const int back = (int)partner((uint32_t)kept_theirs);
        written[0] = half ? back : kept_mine;
        written[1] = half ? kept_mine : back;
      }
      // the cut goes into the query's operand: components 3..5 of the lower
      // lanes' registers (block 0's queries), 0..2 of the upper lanes'
      // (block 1's): k = 3..5 and 8..10
      {
        uint4 w0 = __builtin_bit_cast(uint4, yh[0][NB - 1]);
        uint4 w1 = __builtin_bit_cast(uint4, yh[1][NB - 1]);
        if (half == 0) {
          w0.y = (w0.y & 0xffffu) | (cut.part01 << 16);
          w0.z = (cut.part01 >> 16) | (cut.part2 << 16);
        } else {
          w1.x = cut.part01;
          w1.y = cut.part2;
        }
        yh[0][NB - 1] = __builtin_bit_cast(feat_f16x8_t, w0);
        yh[1][NB - 1] = __builtin_bit_cast(feat_f16x8_t, w1);
      }
      const float other_recon =
          __uint_as_float(partner(__float_as_uint(cut.recon)));
      const bool my_fill = cut.fill != 0;
      const bool other_fill = partner(my_fill ? 1u : 0u) != 0;
      recon[0] = half ? other_recon : cut.recon;
      recon[1] = half ? cut.recon : other_recon;
      fill[0] = half ? other_fill : my_fill;
      fill[1] = half ? my_fill : other_fill;
      need_ckpt = false;
    };

    // ---- the loop ------------------------------------------------------------
    // One step: the chains of matrix instructions of 32 rows x 64 queries into
    // `cur`, and in their shadow the masks and minima of the step before
    // (`old`); then that step's flagged values are appended.
    auto step = [&](feat_acc_t (&cur)[RB], feat_acc_t (&old)[RB], int t,
                    int sub, bool old_valid, int old_pos0,
                    const float (&rec_old)[RB], const bool (&all_old)[RB])
                    __attribute__((always_inline)) {
      const uint4 *arow =
          &xs[t % RING][(sub * kFeatStep + col) * RSU + half];
      constexpr int AHEAD = 3;
      uint4 window[AHEAD];
#pragma unroll
      for (int o = 0; o < AHEAD && o < NB; ++o)
        window[o] = arow[2 * o];
#pragma unroll
      for (int b = 0; b < RB; ++b)
        cur[b] = feat_acc_t{0};
      __builtin_amdgcn_sched_barrier(0);
      uint32_t mask[RB];
      float lo[RB];
      signs(old, mask, lo);
#pragma unroll
      for (int o = 0; o < NB; ++o) {
        const feat_f16x8_t a =
            __builtin_bit_cast(feat_f16x8_t, window[o % AHEAD]);
        if (o + AHEAD < NB)
          window[o % AHEAD] = arow[2 * (o + AHEAD)];
#pragma unroll
        for (int b = 0; b < RB; ++b) {
          cur[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, yh[b][o], cur[b],
                                                          0, 0, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (b == 0)
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
        }
      }
#pragma unroll
      for (int b = 0; b < RB; ++b)
        asm volatile("" : "+v"(mask[b]), "+v"(lo[b]));
      __builtin_amdgcn_sched_barrier(0);
      if (old_valid && !(PCA_WIDE_EXP & 1))
        events(old, mask, lo, old_pos0, rec_old, all_old);
    };

    {
      feat_acc_t acc_a[RB], acc_b[RB];
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        acc_a[b] = feat_acc_t{0};
        acc_b[b] = feat_acc_t{0};
      }
      float rec_a[RB] = {0.0f, 0.0f}, rec_b[RB] = {0.0f, 0.0f};
      bool all_a[RB] = {false, false}, all_b[RB] = {false, false};
      int next_ckpt = 1;
#pragma unroll 1
      for (int t = 0; t <= num_tiles; ++t) {
        // what the last tile's steps parked goes to the buffers now: by the
        // time this tile's end waits for the next one's loads, these stores
        // are a tile old
        flush();
        // this wave's pieces of tile t have arrived (awaited below); after
        // the barrier so have everybody's, and everybody is done with tile
        // t - 1
        __syncthreads();
        if (t + RING - 1 < num_tiles)
          request_tile(t + RING - 1); // into the buffer of tile t - 1
        // first half of tile t (t = num_tiles: no tile, nobody looks at the
        // result) and the values of the second half of tile t - 1
#pragma unroll
        for (int b = 0; b < RB; ++b) {
          rec_a[b] = recon[b];
          all_a[b] = fill[b];
        }
        step(acc_a, acc_b, t, 0, t > 0, (t - 1) * TILE + kFeatStep, rec_b,
             all_b);
        // (one call site: at the piece's end the same code writes the counts)
        const bool last = t == num_tiles;
        if (last || (!(PCA_WIDE_EXP & 16) &&
                     (t == next_ckpt || __any(need_ckpt)))) {
          checkpoint(last);
          if (t == next_ckpt)
            next_ckpt = max(t + 1, (int)((long long)t * P.ckpt_growth >> 4));
        }
        if (last)
          break;
#pragma unroll
        for (int b = 0; b < RB; ++b) {
          rec_b[b] = recon[b];
          all_b[b] = fill[b];
        }
        step(acc_b, acc_a, t, 1, true, t * TILE, rec_a, all_a);
        // the next tile's pieces of this wave
        if (t + 1 < num_tiles) {
          // requests in flight beyond tile t + 1: tiles t + 2 .. t + RING - 1
          const int newer = min(num_tiles - (t + 2), RING - 2);
          // (stores issued after the last request would be counted as the
          // newest requests: then everything is waited for)
          if (newer >= 2 && !fresh_stores)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (MAXP - 1))
                         : "memory");
          else if (newer == 1 && !fresh_stores)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(MAXP - 1) : "memory");
          else
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          fresh_stores = false;
        }
      }
    }
  }
#ifdef PCA_FEAT_STATS
  if (lane == 0)
    for (int i = 0; i < 8; ++i)
      atomicAdd(&p.globals->stats[i], st[i]);
#endif
}

// One lane per query: the k + 16 smallest (value, row) keys of the query's
// pieces, to cand[q][0 .. k + 16).
template <int KP>
__global__ __launch_bounds__(kBlock) void feat_wide_gather_kernel(
    KnnFeatWideParams P, int grid) {
  const KnnFeatParams &p = P.base;
  if (p.globals->odd_rows != 0)
    return;
  constexpr int PER_TILE = kWideQueries / kBlock; // workgroups per tile
  const int tid = threadIdx.x;
  const int tile = blockIdx.x / PER_TILE;
  const int total_tiles = P.tile_start[p.num_segments];
  if (tile >= total_tiles)
    return;
  const int local = (blockIdx.x - tile * PER_TILE) * kBlock + tid;
  const int seg = find_segment(P.tile_start, p.num_segments, tile);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int tile_in_seg = tile - P.tile_start[seg];
  const int q = y_begin + tile_in_seg * kWideQueries + local;
  const int kk = p.k + kFeatSlack;
  const int units = (x_end - x_begin + kWideTileRows - 1) / kWideTileRows;
  double best[KP];
#pragma unroll
  for (int j = 0; j < KP; ++j)
    best[j] = (j < KP - kk) ? lowest_key() : feat_empty_key();
  if (units > 0) {
    const long long total = P.unit_start[p.num_segments];
    const long long stretch = wide_stretch(total, grid);
    const long long first = P.unit_start[seg] + (long long)tile_in_seg * units;
    const int w_lo = (int)(first / stretch);
    const int w_hi = (int)((first + units - 1) / stretch);
    const int wave = local / kWave, lane = local % kWave;
    for (int w = w_lo; w <= w_hi; ++w) {
      const int piece = w + tile;
#pragma unroll 1
      for (int h = 0; h < 2; ++h) {
        const int n =
            P.buf_count[((size_t)piece * 2 + h) * kWideQueries + local];
        int most = n;
#pragma unroll
        for (int sh = 32; sh >= 1; sh >>= 1)
          most = max(most, __shfl_xor(most, sh));
        const uint2 *src = P.buf +
                           (((size_t)piece * kWideWaves + wave) * 2 + h) *
                               P.cap * kWave +
                           lane;
        constexpr int CHUNK = 8; // loads in flight at a time
        for (int e0 = 0; e0 < most; e0 += CHUNK) {
          uint2 w2[CHUNK];
#pragma unroll
          for (int i = 0; i < CHUNK; ++i) {
            w2[i] = make_uint2(0u, 0u);
            if (e0 + i < n)
              w2[i] = src[(size_t)(e0 + i) * kWave];
          }
#pragma unroll
          for (int i = 0; i < CHUNK; ++i) {
            const double key = e0 + i < n
                                   ? make_key(__uint_as_float(w2[i].x), w2[i].y)
                                   : feat_empty_key();
            if (!__any(key < best[KP - 1]))
              continue;
            sorted_insert<KP>(best, key);
          }
        }
      }
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

// Everything for one number of blocks (instantiated in its own translation
// unit so that the sizes build in parallel).
template <int NB>
hipError_t launch_knn_feat_wide_blocks(const KnnFeatWideParams &p, int kw,
                                       bool cosine, int grid,
                                       hipStream_t stream);

#define PCA_KNN_FEAT_WIDE_DEFINE(NB_)                                          \
  template <int K>                                                             \
  static void launch_feat_wide_one_##NB_(const KnnFeatWideParams &p,           \
                                         bool cosine, int grid,                \
                                         hipStream_t stream) {                 \
    if (cosine)                                                                \
      hipLaunchKernelGGL((knn_feat_wide_kernel<NB_, K, true>), dim3(grid),     \
                         dim3(kWideThreads), 0, stream, p);                    \
    else                                                                       \
      hipLaunchKernelGGL((knn_feat_wide_kernel<NB_, K, false>), dim3(grid),    \
                         dim3(kWideThreads), 0, stream, p);                    \
  }                                                                            \
  template <>                                                                  \
  hipError_t launch_knn_feat_wide_blocks<NB_>(const KnnFeatWideParams &p,      \
                                              int kw, bool cosine, int grid,   \
                                              hipStream_t stream) {            \
    switch (kw) {                                                              \
    case 16:                                                                   \
      launch_feat_wide_one_##NB_<16>(p, cosine, grid, stream);                 \
      break;                                                                   \
    case 32:                                                                   \
      launch_feat_wide_one_##NB_<32>(p, cosine, grid, stream);                 \
      break;                                                                   \
    case 64:                                                                   \
      launch_feat_wide_one_##NB_<64>(p, cosine, grid, stream);                 \
      break;                                                                   \
    case 100:                                                                  \
      launch_feat_wide_one_##NB_<100>(p, cosine, grid, stream);                \
      break;                                                                   \
    default:                                                                   \
      return hipErrorInvalidValue;                                             \
    }                                                                          \
    return hipGetLastError();                                                  \
  }

} // namespace pca
