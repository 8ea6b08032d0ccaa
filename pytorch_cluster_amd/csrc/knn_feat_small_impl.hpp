// Feature-space kNN for examples of up to some ten thousand rows (8 < d <= 128,
// k <= 48, Euclidean or cosine): ONE kernel, exact in itself.  It computes what
// knn_kernel of the reference computes (csrc/cuda/knn_cuda.cu:30-84), bit for
// bit, with the fp16 lower bound of knn_feat_impl.hpp as its filter.
//
// The long-scan kernels of that path keep lists of lower bounds, tighten a cut
// as they go, and hand k + 16 candidates per query to a second kernel; every
// piece of a scan starts cold, and a call is a dozen launches.  On examples of
// 1,024 - 4,096 rows (the dynamic graphs of point-cloud networks: 32 clouds of
// 1,024 points with 64 features, k = 20) that start-up is all there is: 0.5 ms
// per call for 4 GFLOP.  Here a workgroup of four waves owns 128 queries of one
// example (lanes l and l + 32 share a query and split every step's 32 rows, as
// in knn_lowd_mc_impl.hpp) and goes over the example's rows TWICE, 32 rows at a
// time.
//
//   1. Bound (the first 64 steps at most; the step's packed fp16 rows and its
//      fp32 rows both in LDS).  One chain of v_mfma_f32_32x32x16_f16 per step
//      gives a lane the values s of its 16 rows; it takes the row with the
//      smallest one (accumulator number in the four lowest mantissa bits
//      through a v_min3_f32 tree), evaluates THAT row exactly -- direct
//      differences, one fused multiply-add per component in ascending order,
//      the reference's chain -- and keeps the ceil(k / 2) smallest of these
//      distances.  The rows are all different, and different from the partner
//      lane's, so the larger of the two lanes' ceil(k / 2)-th samples is an
//      upper bound tau of the query's k-th distance.
//   2. Search (packed rows only).  The same chains again.  l = s + shift is a
//      lower bound of the scaled distance e / sigma^2 the reference computes
//      (knn_feat_impl.hpp), so every row with e below a bound has s <= bound /
//      sigma^2 - shift =: cut.  A lane parks the rows under its cut (one word
//      per step: step and 16-bit mask); when a queue is about to fill up,
//      and at the end, all waves turn to their parked rows: in rounds of one
//      row per lane the rows are fetched from global memory (four lanes per
//      64-byte line, handed to the owner through LDS), evaluated exactly, and
//      enter the lane's sorted list of (distance, row) keys; the list's k-th distance and the partner's
//      tighten the bound as in the low-dimensional kernel.  About 1.5 k rows
//      per query get that far.  Nothing is approximate in what is KEPT, and
//      every row that could be kept is looked at: no candidate list, no second
//      stage, no proof of completeness to fail.
//
// A workgroup has its compute unit to itself (one wave per SIMD: 200+
// registers for the lists, up to 157 KB of LDS), so nothing hides a wait but
// the wave's own instructions.  Hence: four tiles are on their way from
// global memory at any time, a round's rows are asked for one round ahead,
// all waves leave the scan for their parked rows at the same steps (a wave
// on its own would keep the other three at the tile's barrier), and no load
// sits under a condition (the compiler then counts loads in flight exactly
// instead of waiting for all of them).
//
// Rows the filter cannot represent: NaN / infinite components are nobody's
// neighbours (packed as padding); rows far larger than the rest (left out of
// the scale, FeatGlobals::out_rows) are evaluated exactly for every query at
// the end; if a row's squared norm overflows (FeatGlobals::odd_rows), or for a
// query the filter cannot take (FeatQuery::odd), the lanes concerned park
// every row instead of the rows under a cut: slow, and the same result.
//
// fp16 and bf16 rows (knn_kernel<c10::Half>, <c10::BFloat16>): the same
// kernel on the rows widened to fp32, with the reference's 16-bit arithmetic
// in the exact distances (SmallChain), and in the filter every component of
// rows and queries times what that arithmetic leaves of its term at worst
// (chain_keep: the first terms of the sum are rounded most often) -- the
// filter's distance is then a lower bound of the reference's value.  Such
// rows come here with any number of components up to 128, and in any number:
// 16-bit points of two or three dimensions have no other kernel but the
// exhaustive scan.
#pragma once

#include <type_traits>
#include <utility>

#include "knn_feat_impl.hpp"

namespace pca {

constexpr int kSmallStep = 32;        // rows per step and LDS tile
constexpr int kSmallSampleSteps = 64; // steps of an example the bound samples
constexpr int kSmallQueue = 16;       // parked steps per lane
// (a compiler vector: arrays of these are kept in registers where arrays of
// float4, a class, end up in scratch memory)
typedef float small_v4f __attribute__((ext_vector_type(4)));
typedef unsigned small_v4u __attribute__((ext_vector_type(4)));

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop
// whose counter is a constant in every turn (register arrays indexed by it
// stay in registers).
template <typename F, int... I>
__device__ __forceinline__ void static_for_each(
    F &&f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>()), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_each(f, std::make_integer_sequence<int, N>());
}

// The arithmetic of the exact distances.  R16 = 0: fp32 rows, one fused
// multiply-add per component (csrc/cuda/knn_cuda.cu:61-64 as a GPU compiler
// builds it); R16 = 3: the cosine distance of fp32 rows, 1 - x.y / (|x| |y|)
// with the dot product as such a chain (csrc/cuda/knn_cuda.cu:9-28).
// R16 = 1 / 2: the rows were fp16 / bf16 (widened to fp32 for
// this kernel, which is exact) and the reference computes in c10::Half /
// c10::BFloat16: every difference, square and sum is formed in fp32 and
// rounded to 16 bits (torch/headeronly/util/Half.h:501-560); the sentinel
// 1e10 is +inf in fp16.
template <int R16> struct SmallChain {
  static __device__ __forceinline__ float step(float x, float y, float acc) {
    // (the compiler turns "widen, operate, round" into 16-bit operations,
    // which is exact, and would then fuse the square into the sum, which is
    // one rounding fewer than the reference makes)
#pragma clang fp contract(off)
    if (R16 == 0) {
      const float dc = x - y;
      return __builtin_fmaf(dc, dc, acc);
    }
    if (R16 == 3) // (the cosine distance: the dot product, fp32 rows)
      return __builtin_fmaf(x, y, acc);
    const float dc = round_in_chain<R16 == 2>(x - y);
    const float sq = round_in_chain<R16 == 2>(dc * dc);
    return round_in_chain<R16 == 2>(acc + sq);
  }
  // Four components.  fp16 rows: two differences and two squares per
  // instruction (every half of a packed 16-bit operation rounds by itself,
  // like the single one); the sums stay one after the other.
  static __device__ __forceinline__ float step4(float x0, float x1, float x2,
                                                float x3, float y0, float y1,
                                                float y2, float y3,
                                                float acc) {
    if constexpr (R16 == 1) {
#pragma clang fp contract(off)
      typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
      // (exact: the numbers are fp16 numbers)
      const half2_t xa = {(_Float16)x0, (_Float16)x1};
      const half2_t xb = {(_Float16)x2, (_Float16)x3};
      const half2_t ya = {(_Float16)y0, (_Float16)y1};
      const half2_t yb = {(_Float16)y2, (_Float16)y3};
      const half2_t da = xa - ya, db = xb - yb;
      const half2_t sa = da * da, sb = db * db;
      _Float16 sum = (_Float16)acc;
      sum = sum + sa.x;
      sum = sum + sa.y;
      sum = sum + sb.x;
      sum = sum + sb.y;
      return (float)sum;
    } else {
      acc = step(x0, y0, acc);
      acc = step(x1, y1, acc);
      acc = step(x2, y2, acc);
      return step(x3, y3, acc);
    }
  }
  static __device__ __forceinline__ float sentinel() {
    return (R16 == 0 || R16 == 3) ? kKnnSentinel
                                  : round_to_16<R16 == 2>(1e10f);
  }
  // A 16-bit chain value H and the filter's distance D' -- the squared
  // distance, in real numbers, of row and query with every component times
  // chain_keep<R16> (device_utils.hpp: what the rounding of three operations
  // on a term and of the sums behind it leaves of that term, at worst):
  // H >= D' - d t, t what a square can lose below the normal range
  // (differences and sums there are exact: multiples of the smallest number
  // of the format).  Hence H < h only if D' < (h + slack()) * widen(d); the
  // factor carries (1 + (d + 2) 2^-24) for the fp32 chain the filter's bound
  // was proven against and 2 x 2^-24 more for the one case in which a scaled
  // component is not exact (a bf16 component below 2^-125, next to one that
  // is not).
  static __device__ __forceinline__ double widen(int d) {
    if (R16 == 0 || R16 == 3)
      return 1.0;
    return (1.0 + (double)(d + 4) * (1.0 / 16777216.0)) * (1.0 + 1e-9);
  }
  static __device__ __forceinline__ double slack(int d) {
    if (R16 == 0 || R16 == 3)
      return 0.0;
    // fp16: squares below 2^-14 round to multiples of 2^-24; bf16: squares
    // below 2^-126 may be flushed altogether
    return (double)d * (R16 == 2 ? 1.1754943508222875e-38 : 1.0 / 16777216.0);
  }
};

// The next float above v (any sign; v finite).
__device__ __forceinline__ float small_next_up(float v) {
  if (v == 0.0f)
    return 1.401298464324817e-45f;
  const uint32_t u = __float_as_uint(v);
  return __uint_as_float(v > 0.0f ? u + 1u : u - 1u);
}

template <int NB, int K, int R16 = 0, bool RADIUS = false>
__global__ __launch_bounds__(kBlock, 1) void knn_feat_small_kernel(
    KnnFeatParams p) {
  typedef SmallChain<R16> Chain;
  typedef FeatShape<NB> S;
  constexpr int RSU = S::RSU;
  constexpr int TILE = kSmallStep;
  constexpr int TILE_UNITS = TILE * RSU;
  constexpr int PU = (TILE_UNITS + kBlock - 1) / kBlock; // packed units/thread
  constexpr int MAX_D = S::MAX_D;
  constexpr int ROW_F = MAX_D + 4; // floats from row to row in LDS
  constexpr int XV = (TILE * MAX_D / 4 + kBlock - 1) / kBlock; // float4/thread
  constexpr int XS = (TILE * MAX_D + kBlock - 1) / kBlock;     // floats/thread
  constexpr int TQ = kFeatQueries;
  constexpr int SEEDS = K / 2;
  constexpr int DEPTH = 4; // tiles in flight
  static_assert(kSmallQueue % DEPTH == 0 && kSmallQueue >= 3 * DEPTH,
                "a queue outlasts two looks");
  static_assert(K % 8 == 0 && K <= 48, "list widths in steps of 8, up to 48");
  static_assert(kBlock == 256 && TQ == 128, "four waves of 32 queries");

  __shared__ __attribute__((aligned(16))) uint4 xs[2][TILE_UNITS];
  __shared__ __attribute__((aligned(16))) float x32[2][TILE * ROW_F];
  __shared__ __attribute__((aligned(16))) float ys[TQ * ROW_F];
  // parked steps of the search: (step << 16) | mask of the lane's 16 rows
  __shared__ uint32_t queue[kSmallQueue][kBlock];
  // per wave: 16 components of 64 gathered rows (five 16-byte units from row
  // to row: neighbouring rows fall on distinct banks)
  __shared__ __attribute__((aligned(16)))
  small_v4f gathered[kBlock / kWave][kWave][5];
  __shared__ int wave_full[kBlock / kWave];
  // what the waves said at the last two looks at their queues (see the search)
  __shared__ int wave_says[2][kBlock / kWave];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int half = lane >> 5;
  const int col = lane & 31;

  const int total_tiles = p.work_start[p.num_segments];
  const int tile = blockIdx.x;
  if (tile >= total_tiles)
    return;
  if (tid < 2 * (kBlock / kWave))
    (&wave_says[0][0])[tid] = 0; // (a barrier follows before the first look)
  const int seg = find_segment(p.work_start, p.num_segments, tile);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int q = y_begin + (tile - p.work_start[seg]) * TQ + wave * 32 + col;
  const bool valid = q < y_end;

  const int d = p.d;
  const int k = p.k;
  const bool vec4 = (d & 3) == 0;
  // the workgroup's query rows (one block of y) into LDS: everything below
  // reads them from there (lanes without a query hold zeros)
  {
    const int q0 = y_begin + (tile - p.work_start[seg]) * TQ;
    const int rows_here = min(TQ, y_end - q0);
    const float *src = p.y + (size_t)q0 * d;
    if (vec4) {
      const int per_row = d >> 2;
      const float4 *src4 = reinterpret_cast<const float4 *>(src);
      for (int f = tid; f < TQ * per_row; f += kBlock) {
        const int r = f / per_row;
        const int c4 = f - r * per_row;
        *reinterpret_cast<float4 *>(&ys[r * ROW_F + 4 * c4]) =
            r < rows_here ? src4[f] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    } else {
      for (int f = tid; f < TQ * d; f += kBlock) {
        const int r = f / d;
        ys[r * ROW_F + (f - r * d)] = r < rows_here ? src[f] : 0.0f;
      }
    }
  }
  __syncthreads();
  const float *const my_y = &ys[(wave * 32 + col) * ROW_F];

  constexpr bool COSINE = R16 == 3;
  static_assert(!(COSINE && RADIUS), "no radius search by cosine distance");
  const float ynorm = COSINE && valid ? p.y_norm[q] : 1.0f;
  const float inv_sigma =
      COSINE ? 1.0f : feat_inv_sigma(p.globals->max_bits);
  const FeatQuery fq = feat_query<COSINE, R16>(my_y, d, inv_sigma, ynorm);
  // active: the query searches (a NaN component: no neighbours).  filtered:
  // it does so with the fp16 lower bound; if the filter cannot take the query
  // (a component beyond the range the scale was made for) or some row of x
  // (a squared norm that overflows), every row is evaluated instead.
  const bool active = valid && !fq.dead;
  const bool filtered = active && !fq.odd && p.globals->odd_rows == 0;
  const float sentinel = Chain::sentinel();
  const double scale2 =
      COSINE ? kFeatCosScale : (double)inv_sigma * (double)inv_sigma;
  const float y_scale = COSINE ? -1024.0f / ynorm : -2.0f * inv_sigma;
  // what the reference makes of a chain's value and row g (the cosine
  // distance divides the dot product by the norms)
  auto finish = [&](float acc, int g) {
    if (COSINE) {
      acc = acc / (p.x_norm[g] * ynorm);
      acc = 1.0f - acc;
    }
    return acc;
  };
  const int seg_len = x_end - x_begin;
  const int num_tiles = (seg_len + TILE - 1) / TILE;

  // B operands: this lane's 8 components of every block; the last block
  // holds the powers of two that W's parts are multiplied by (lower lanes)
  feat_f16x8_t yh[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    uint32_t hb[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (i < NB - 1) {
      const int cb = 16 * i + 8 * half;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        hb[e] = (filtered && cb + e < d)
                    ? feat_h(my_y[min(cb + e, d - 1)] *
                             chain_keep<R16>(d, min(cb + e, d - 1)) * y_scale)
                    : 0u;
    } else if (half == 0 && filtered) {
      hb[0] = 0x7800u; // 2^15
      hb[1] = 0x4c00u; // 2^4
      hb[2] = 0x2000u; // 2^-7
    }
    yh[i] = __builtin_bit_cast(
        feat_f16x8_t,
        make_uint4(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16),
                   hb[4] | (hb[5] << 16), hb[6] | (hb[7] << 16)));
  }

  // ---- tile staging: packed rows and fp32 rows of 32 rows -------------------
  // Two buffers in LDS; DEPTH tiles on their way from global memory in
  // registers (a thread holds a few 16-byte units of a tile: with one tile in
  // flight a step would last as long as a load does).
  small_v4u stage_p[DEPTH][PU];
  small_v4f stage_v[DEPTH][XV];
  float stage_s[DEPTH][XS];
  // (No load sits under a condition -- indices are clamped instead, and what
  // a clamped index fetches is never stored or never looked at: the compiler
  // counts the loads in flight only along straight code, and waits for all
  // of them, the tiles just asked for included, where it cannot.)
  auto load_tile = [&](auto slot_c, int t, auto rows_c, auto vec4_c) {
    constexpr int slot = decltype(slot_c)::value;
    const size_t row0 = (size_t)x_begin + (size_t)t * TILE;
#pragma unroll
    for (int i = 0; i < PU; ++i) {
      const int u = min(i * kBlock + tid, TILE_UNITS - 1);
      // (the packed copy ends with a tile of spare rows)
      stage_p[slot][i] =
          reinterpret_cast<const small_v4u *>(p.x_pack)[row0 * RSU + u];
    }
    if constexpr (!decltype(rows_c)::value)
      return;
    // rows behind the last one of x are not read (rows of the next example
    // are masked out later)
    if constexpr (decltype(vec4_c)::value) {
      const small_v4f *src = reinterpret_cast<const small_v4f *>(p.x);
      const size_t first = row0 * (size_t)(d >> 2);
      const size_t last = (size_t)p.n * (size_t)(d >> 2) - 1;
#pragma unroll
      for (int i = 0; i < XV; ++i)
        stage_v[slot][i] = src[min(first + (size_t)(i * kBlock + tid), last)];
    } else {
      const size_t first = row0 * (size_t)d;
      const size_t last = (size_t)p.n * (size_t)d - 1;
#pragma unroll
      for (int i = 0; i < XS; ++i)
        stage_s[slot][i] = p.x[min(first + (size_t)(i * kBlock + tid), last)];
    }
  };
  auto store_tile = [&](auto slot_c, int buf, auto rows_c, auto vec4_c) {
    constexpr int slot = decltype(slot_c)::value;
#pragma unroll
    for (int i = 0; i < PU; ++i) {
      const int u = i * kBlock + tid;
      if (u < TILE_UNITS)
        *reinterpret_cast<small_v4u *>(&xs[buf][u]) = stage_p[slot][i];
    }
    if constexpr (!decltype(rows_c)::value)
      return;
    if constexpr (decltype(vec4_c)::value) {
      const int per_row = d >> 2;
#pragma unroll
      for (int i = 0; i < XV; ++i) {
        const int f = i * kBlock + tid;
        if (f < TILE * per_row) {
          const int r = f / per_row;
          const int c4 = f - r * per_row;
          *reinterpret_cast<small_v4f *>(&x32[buf][r * ROW_F + 4 * c4]) =
              stage_v[slot][i];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < XS; ++i) {
        const int f = i * kBlock + tid;
        if (f < TILE * d) {
          const int r = f / d;
          x32[buf][r * ROW_F + (f - r * d)] = stage_s[slot][i];
        }
      }
    }
  };

  // the step's 32 x 32 values: s of row 8 (v / 4) + 4 half + v % 4 and the
  // lane's query in accumulator v
  auto products = [&](int buf) {
    const uint4 *arow = &xs[buf][col * RSU + half];
    feat_acc_t acc = {0};
#pragma unroll
    for (int o = 0; o < NB; ++o)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
          __builtin_bit_cast(feat_f16x8_t, arow[2 * o]), yh[o], acc, 0, 0, 0);
    return acc;
  };
  // exact squared distance of row j of the tile to the lane's query, as the
  // reference accumulates it (csrc/cuda/knn_cuda.cu:61-64)
  auto exact = [&](int buf, int j) {
    const float *xr = &x32[buf][j * ROW_F];
    float acc = 0.0f;
    if (vec4) {
      const float4 *x4 = reinterpret_cast<const float4 *>(xr);
      const float4 *y4 = reinterpret_cast<const float4 *>(my_y);
#pragma unroll 4
      for (int c = 0; c < (d >> 2); ++c) {
        const float4 a = x4[c];
        const float4 b = y4[c];
        acc = Chain::step4(a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w, acc);
      }
    } else {
      for (int c = 0; c < d; ++c) {
        acc = Chain::step(xr[c], my_y[c], acc);
      }
    }
    return acc;
  };
  // row of the tile that accumulator v of this lane stands for
  auto row_of = [&](int v) { return 8 * (v >> 2) + 4 * half + (v & 3); };

  // One pass over the example's tiles; body(t, buf, rows) with the tile in
  // LDS, every(group, last) after each DEPTH tiles (true: the pass ends
  // there).  (One
  // barrier per tile: a buffer is overwritten a whole tile after its last
  // reader passed the barrier before.)  Slot t % DEPTH of the registers
  // holds tile t + 1 until it is stored, then tile t + 1 + DEPTH.
  // (with_rows: the fp32 rows are staged beside the packed ones)
  auto for_tiles = [&](int count, auto rows_c, auto vec4_c, auto &&body,
                       auto &&every) {
    if (count <= 0)
      return;
    __syncthreads(); // (nobody still reads the buffers of the pass before)
    load_tile(std::integral_constant<int, 0>(), 0, rows_c, vec4_c);
    store_tile(std::integral_constant<int, 0>(), 0, rows_c, vec4_c);
    static_for<DEPTH>([&](auto j) {
      load_tile(j, min(1 + j.value, count - 1), rows_c, vec4_c);
    });
    __syncthreads();
    for (int t0 = 0; t0 < count; t0 += DEPTH) {
      static_for<DEPTH>([&](auto j) {
        const int t = t0 + j.value;
        if (t < count) { // (uniform)
          body(t, t & 1, min(TILE, seg_len - t * TILE));
          // (behind the last tile: stored where nobody reads any more, and
          // the last tile fetched again)
          store_tile(j, (t + 1) & 1, rows_c, vec4_c);
          load_tile(j, min(t + 1 + DEPTH, count - 1), rows_c, vec4_c);
          __syncthreads();
        }
      });
      if (every(t0 / DEPTH, t0 + DEPTH >= count))
        break; // (uniform)
    }
  };

  // ---- 1. the bound ---------------------------------------------------------
  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - k) ? lowest_key() : empty_key();
  // exact distances must be strictly below thresh; `shared`: what the sampled
  // rows and the partner lane say about the query's final k-th distance
  // (equality admitted: the rows at the bound are found again by the search)
  float thresh = active ? (RADIUS ? p.r2 : sentinel) : -__builtin_inff();
  float shared = sentinel;
  // (the radius search: hits so far, and "no later row of this lane can be
  // among the query's first k hits")
  int hits = 0;
  bool full = !active;
  if constexpr (!RADIUS) {
    float seed[SEEDS];
#pragma unroll
    for (int j = 0; j < SEEDS; ++j)
      seed[j] = __builtin_inff();
    auto sample_step = [&](int t, int buf, int rows) {
      const feat_acc_t acc = products(buf);
      // the smallest of the lane's 16 values, its accumulator number in the
      // four lowest bits (which of two nearly equal rows is taken does not
      // matter); rows behind the example's end do not count
      float tagged[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        tagged[v] = __uint_as_float((__float_as_uint(acc[v]) & ~15u) |
                                    (uint32_t)v);
        if (rows < TILE && row_of(v) >= rows)
          tagged[v] = __builtin_inff();
      }
      float m0 = min3f(tagged[0], tagged[1], tagged[2]);
      float m1 = min3f(tagged[3], tagged[4], tagged[5]);
      float m2 = min3f(tagged[6], tagged[7], tagged[8]);
      float m3 = min3f(tagged[9], tagged[10], tagged[11]);
      float m4 = min3f(tagged[12], tagged[13], tagged[14]);
      m0 = min3f(m0, m1, m2);
      m3 = min3f(m3, m4, tagged[15]);
      const float least = __builtin_fminf(m0, m3);
      const int v = (int)(__float_as_uint(least) & 15u);
      const int j = row_of(v);
      const float e =
          finish(exact(buf, j), min(x_begin + t * TILE + j, p.n - 1));
      // (a padding row, a NaN or a distance beyond the limit is no sample)
      const float sample =
          (active && j < rows && least < __builtin_inff() && e < sentinel)
              ? e
              : __builtin_inff();
#pragma unroll
      for (int i = SEEDS - 1; i >= 1; --i)
        seed[i] = __builtin_amdgcn_fmed3f(seed[i - 1], seed[i], sample);
      seed[0] = __builtin_fminf(seed[0], sample);
    };
    const int sampled = min(num_tiles, kSmallSampleSteps);
    if (vec4)
      for_tiles(sampled, std::true_type(), std::true_type(), sample_step,
                [](int, bool) { return false; });
    else
      for_tiles(sampled, std::true_type(), std::false_type(), sample_step,
                [](int, bool) { return false; });
    // the ceil(k / 2)-th smallest sample of this lane and of its partner
    const int mine = (k + 1) / 2 - 1;
    float own = __builtin_inff();
#pragma unroll
    for (int i = 0; i < SEEDS; ++i)
      if (i == mine) {
        asm volatile(""); // (keeps this a branch)
        own = seed[i];
      }
    const auto both = __builtin_amdgcn_permlane32_swap(
        __float_as_uint(own), __float_as_uint(own), false, false);
    const float partner = __uint_as_float(half ? both[0] : both[1]);
    const float bound = __builtin_fmaxf(own, partner);
    if (active && bound < sentinel) {
      shared = small_next_up(bound);
      thresh = __builtin_fminf(thresh, shared);
    }
  }

  // ---- 2. the search -------------------------------------------------------
  // s below cut: the row's distance may lie below thresh (a strict test
  // against feat_float_above(c) admits everything up to c = thresh / sigma^2
  // - shift)
  float cut = -__builtin_inff();
  const double widen = Chain::widen(d) * scale2;
  const double slack = Chain::slack(d);
  auto set_cut = [&]() {
    if (filtered)
      cut = feat_float_above(((double)thresh + slack) * widen - fq.shift);
  };
  set_cut();
  // What the two lanes of a query tell each other (knn_lowd_mc_impl.hpp).
  auto partner_bounds = [&]() {
    const float own = key_dist(best[K - 1]);
    const auto both = __builtin_amdgcn_permlane32_swap(
        __float_as_uint(own), __float_as_uint(own), false, false);
    float partner = __uint_as_float(half ? both[0] : both[1]);
    const int c = k >> 1;
    float mid = sentinel;
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
    if (active && partner < sentinel) {
      shared = __builtin_fminf(shared, small_next_up(partner));
      thresh = __builtin_fminf(thresh, shared);
    }
  };
  // Exact squared distances of 64 rows of x, one per lane (row g of lane l to
  // the query of lane l), the rows read from global memory.  A lane reading
  // its own row would touch a 64-byte line per 16-byte load; here four lanes
  // read one line of one row together (sixteen rows per load instruction,
  // every line used in full), 64 components of all rows at a time (a
  // "chunk": gather_chunk), and the pieces reach the lane that owns the row
  // through LDS, sixteen components at a time, in ascending order
  // (chain_chunk): the chain is the reference's.
  auto gather_chunk = [&](small_v4f (&a)[4][4], int g, int f0) {
    const int quads = d >> 2;
    const small_v4f *x4 = reinterpret_cast<const small_v4f *>(p.x);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      // the row of lane 16 r + lane / 4: one of the four this lane helps with
      const size_t base = (size_t)__shfl(g, 16 * r + (lane >> 2)) * quads;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        a[c][r] = x4[base + min(f0 + 4 * c + (lane & 3), quads - 1)];
    }
  };
  auto chain_chunk = [&](const small_v4f (&a)[4][4], int f0, float acc) {
    const int quads = d >> 2;
    const small_v4f *y4 = reinterpret_cast<const small_v4f *>(my_y);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (f0 + 4 * c < quads) { // (uniform)
        // (the wave is done reading the piece before)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < 4; ++r)
          gathered[wave][16 * r + (lane >> 2)][lane & 3] = a[c][r];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (f0 + 4 * c + e < quads) {
            const small_v4f xv = gathered[wave][lane][e];
            const small_v4f b = y4[f0 + 4 * c + e];
            acc = Chain::step4(xv.x, xv.y, xv.z, xv.w, b.x, b.y, b.z, b.w,
                               acc);
          }
        }
      }
    }
    return acc;
  };
  // (d not a multiple of four: every lane reads its own row)
  auto exact_unaligned = [&](int g) {
    const float *xr = p.x + (size_t)g * d;
    float acc = 0.0f;
    for (int c = 0; c < d; ++c) {
      acc = Chain::step(xr[c], my_y[c], acc);
    }
    return acc;
  };
  // Parked steps: a lane with rows under its cut parks (step, mask); the
  // rows are evaluated exactly -- from global memory: by then their tile has
  // left LDS -- by all lanes together, in rounds, when a queue is about to
  // fill up and at the end (the bound from the sampled rows is tight from the
  // start, so nothing is lost by looking late).
  int qn = 0;
  // (with -DPCA_FEAT_STATS: rounds of the waves, lanes that had a row in a
  // round, lanes whose row was kept -> FeatGlobals::stats[0..2])
#ifdef PCA_FEAT_STATS
  unsigned counted[3] = {0, 0, 0};
#define PCA_SSTAT(i, v) (counted[i] += (v) ? 1u : 0u)
#else
#define PCA_SSTAT(i, v) ((void)0)
#endif
  auto drain = [&]() {
    bool changed = false;
    int taken = 0;
    uint32_t pending = 0;
    int step_row = 0; // first of the lane's rows of that step, in the example
    // the lane's next parked row (on: it has one)
    auto pop = [&](int &g, bool &on) {
      if (pending == 0 && taken < qn) {
        const uint32_t word = queue[taken][tid];
        ++taken;
        pending = word & 0xffffu;
        step_row = (int)(word >> 16) * TILE;
      }
      // (radius search: a lane that holds its k hits looks no further)
      on = pending != 0 && !(RADIUS && full);
      const int v = __builtin_clz(pending | 1u) - 16;
      pending &= ~(0x8000u >> v);
      g = min(x_begin + (on ? step_row + row_of(v) : 0), p.n - 1);
    };
    auto take = [&](float e, int g, bool on) {
      bool ok = on && e < thresh;
      if (RADIUS)
        ok = ok && !full && !(p.ignore_same != 0 && g == q);
      PCA_SSTAT(0, lane == 0);
      PCA_SSTAT(1, on);
      if (!__any(ok))
        return;
      PCA_SSTAT(2, ok);
      // (radius search: the key is the row number alone, the list keeps the
      // k smallest rows among the hits; a lane's rows arrive in ascending
      // order, so once it holds k nothing more of it can count)
      const double key = RADIUS ? make_key(0.0f, (uint32_t)g)
                                : make_key(e, (uint32_t)g);
      sorted_insert<K>(best, ok ? key : empty_key());
      if (RADIUS) {
        hits += ok ? 1 : 0;
        full = full || hits >= k;
      } else if (active) {
        thresh = __builtin_fminf(key_dist(best[K - 1]), shared);
      }
      changed = true;
    };
    int g;
    bool on;
    pop(g, on);
    if (vec4) {
      // One chunk ahead: while a chunk goes through LDS and the chain, the
      // next one (of the same rows, or the first of the next rows; after the
      // last rows, one nobody looks at) is on its way from global memory.
      // Two sets of registers take turns, and the fetch is unconditional
      // (see load_tile).
      const int quads = d >> 2;
      small_v4f set_a[4][4], set_b[4][4];
      bool more = __any(on);
      int f0 = 0;
      float acc = 0.0f;
      auto chunk = [&](small_v4f (&now)[4][4], small_v4f (&next)[4][4]) {
        const bool last = f0 + 16 >= quads; // (uniform)
        int g_next = g;
        bool on_next = on;
        if (last)
          pop(g_next, on_next);
        const int f0_next = last ? 0 : f0 + 16;
        gather_chunk(next, g_next, f0_next);
        acc = chain_chunk(now, f0, acc);
        if (last) {
          take(finish(acc, g), g, on);
          acc = 0.0f;
          more = __any(on_next);
        }
        g = g_next;
        on = on_next;
        f0 = f0_next;
      };
      if (more)
        gather_chunk(set_a, g, 0);
      while (more) {
        chunk(set_a, set_b);
        if (!more)
          break;
        chunk(set_b, set_a);
      }
    } else {
      while (__any(on)) {
        take(finish(exact_unaligned(g), g), g, on);
        pop(g, on);
      }
    }
    qn = 0;
    if (RADIUS) {
      // both lanes of the query have looked at every row so far: k hits
      // between them settle the query
      const auto both = __builtin_amdgcn_permlane32_swap(
          (unsigned)hits, (unsigned)hits, false, false);
      full = full || hits + (int)(half ? both[0] : both[1]) >= k;
    } else if (changed) {
      partner_bounds();
      set_cut();
    }
  };
  for_tiles(num_tiles, std::false_type(), std::false_type(),
            [&](int t, int buf, int rows) {
    const feat_acc_t a = products(buf);
    float m0 = min3f(a[0], a[1], a[2]);
    float m1 = min3f(a[3], a[4], a[5]);
    float m2 = min3f(a[6], a[7], a[8]);
    float m3 = min3f(a[9], a[10], a[11]);
    float m4 = min3f(a[12], a[13], a[14]);
    m0 = min3f(m0, m1, m2);
    m3 = min3f(m3, m4, a[15]);
    const float least = __builtin_fminf(m0, m3);
    const bool all_rows = active && !filtered;
    const bool looking = !RADIUS || !full;
    if (__any((least < cut || all_rows) && looking)) {
      // the lane's rows under the cut: bit 15 - v for accumulator v
      uint32_t mask = 0;
#pragma unroll
      for (int v = 0; v < 16; ++v)
        if ((a[v] < cut || all_rows) && looking && row_of(v) < rows)
          mask |= 0x8000u >> v;
      if (mask != 0) {
        queue[qn][tid] = ((uint32_t)t << 16) | mask;
        ++qn;
      }
    }
  }, [&](int group, bool last) {
    // All waves turn to their parked rows together (a wave on its own would
    // keep the others waiting at the tiles' barriers), and only when it is
    // time: at the end, and when some lane's queue could fill up before the
    // next but one look -- a lane parks at most one word per tile, and what
    // the waves say here is read at the next look, DEPTH tiles and as many
    // barriers later.  Long scans with a tight cut park little: their drains
    // are few and their rounds well filled.
    bool go = last;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w)
      go = go || wave_says[(group & 1) ^ 1][w] != 0;
    if (go)
      drain();
    const int want = __any(qn > kSmallQueue - 2 * DEPTH) ? 1 : 0;
    if (lane == 0)
      wave_says[group & 1][wave] = want;
    if constexpr (RADIUS) {
      if (go) { // (uniform; hits only come in with a drain)
        // a workgroup whose queries all have their k hits leaves the scan
        const int all_full = __any(!full) ? 0 : 1;
        if (lane == 0)
          wave_full[wave] = all_full;
        __syncthreads();
        const bool stop = (wave_full[0] & wave_full[1] & wave_full[2] &
                           wave_full[3]) != 0;
        __syncthreads();
        return stop;
      }
    }
    return false;
  });

  // rows that were left out of the scale: every query looks at them exactly
  // (the lower lane of a pair; a handful of rows at most)
  if (p.globals->n_out > 0) {
    const int n_out = min(p.globals->n_out, kFeatMaxOutliers);
    for (int o = 0; o < n_out; ++o) {
      const int g = p.globals->out_rows[o];
      if (g < x_begin || g >= x_end)
        continue; // (uniform: the workgroup has one example)
      float e = 0.0f;
      const float *xr = p.x + (size_t)g * d;
      for (int c = 0; c < d; ++c) {
        e = Chain::step(xr[c], my_y[c], e);
      }
      e = finish(e, g);
      // (a query without a bound -- fewer sampled rows than it takes -- cuts
      // nowhere and has met the row among its parked ones already: the same
      // key in its list or in the partner's)
      const double key = RADIUS ? make_key(0.0f, (uint32_t)g)
                                : make_key(e, (uint32_t)g);
      bool listed = false;
#pragma unroll
      for (int j = 0; j < K; ++j)
        listed = listed || best[j] == key;
      const auto both = __builtin_amdgcn_permlane32_swap(
          (unsigned)listed, (unsigned)listed, false, false);
      listed = listed || (half ? both[0] : both[1]) != 0u;
      const bool ok = active && half == 0 && !listed &&
                      (RADIUS ? e < p.r2 && !(p.ignore_same != 0 && g == q)
                              : e < sentinel);
      sorted_insert<K>(best, ok ? key : empty_key());
    }
  }

  unite_halves<K>(best, k, half);
  if (half == 0 && valid) {
    int found = 0;
    if (active)
      found = write_dense<K>(best, k, q, p.out_idx, p.out_dist, p.out_count);
    else
      p.out_count[q] = 0;
    p.redo_q[q] = 0;
    // (edges counted here: the compaction starts from the block sums)
    note_edges<K>(best, k, q, found, p.edge_sums, p.self_pos, p.kept);
  }
#ifdef PCA_FEAT_STATS
  // (one addition per wave and counter: additions to one word take turns)
  for (int i = 0; i < 3; ++i) {
    unsigned v = (i == 0 && lane != 0) ? 0u : counted[i];
    for (int o = 32; o >= 1; o >>= 1)
      v += __shfl_xor(v, o);
    if (lane == 0)
      atomicAdd(&p.globals->stats[i], (unsigned long long)v);
  }
#endif
#undef PCA_SSTAT
}

// Everything for one number of blocks (instantiated in its own translation
// unit so that the sizes build in parallel).
template <int NB, int R16>
hipError_t launch_knn_feat_small_blocks(const KnnFeatParams &p, int kbucket,
                                        int grid, hipStream_t stream);

#define PCA_KNN_FEAT_SMALL_DEFINE(NB_, R16_)                                   \
  template <>                                                                  \
  hipError_t launch_knn_feat_small_blocks<NB_, R16_>(                          \
      const KnnFeatParams &p, int kbucket, int grid, hipStream_t stream) {     \
    switch (kbucket) {                                                         \
    case 8:                                                                    \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 8, R16_>), dim3(grid),    \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 16:                                                                   \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 16, R16_>), dim3(grid),   \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 24:                                                                   \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 24, R16_>), dim3(grid),   \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 32:                                                                   \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 32, R16_>), dim3(grid),   \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 40:                                                                   \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 40, R16_>), dim3(grid),   \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    case 48:                                                                   \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 48, R16_>), dim3(grid),   \
                         dim3(kBlock), 0, stream, p);                          \
      break;                                                                   \
    default:                                                                   \
      return hipErrorInvalidValue;                                             \
    }                                                                          \
    return hipGetLastError();                                                  \
  }

// The radius search with the same kernel (RADIUS): no bound pass, a fixed cut
// from r^2, lists of the k smallest ROW NUMBERS among the rows within the
// radius -- what radius_kernel of the reference returns
// (csrc/cuda/radius_cuda.cu:9-42: the first max_num_neighbors rows in
// ascending order).
template <int NB, int R16>
hipError_t launch_radius_feat_blocks(const KnnFeatParams &p, int kbucket,
                                     int grid, hipStream_t stream);

#define PCA_RADIUS_FEAT_DEFINE(NB_, R16_)                                      \
  template <>                                                                  \
  hipError_t launch_radius_feat_blocks<NB_, R16_>(                             \
      const KnnFeatParams &p, int kbucket, int grid, hipStream_t stream) {     \
    switch (kbucket) {                                                         \
    case 8:                                                                    \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 8, R16_, true>),          \
                         dim3(grid), dim3(kBlock), 0, stream, p);              \
      break;                                                                   \
    case 16:                                                                   \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 16, R16_, true>),         \
                         dim3(grid), dim3(kBlock), 0, stream, p);              \
      break;                                                                   \
    case 24:                                                                   \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 24, R16_, true>),         \
                         dim3(grid), dim3(kBlock), 0, stream, p);              \
      break;                                                                   \
    case 32:                                                                   \
      hipLaunchKernelGGL((knn_feat_small_kernel<NB_, 32, R16_, true>),         \
                         dim3(grid), dim3(kBlock), 0, stream, p);              \
      break;                                                                   \
    default:                                                                   \
      return hipErrorInvalidValue;                                             \
    }                                                                          \
    return hipGetLastError();                                                  \
  }

} // namespace pca
