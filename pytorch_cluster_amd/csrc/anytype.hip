// kNN and radius search for the element types other than fp32: fp64, fp16,
// bf16.  Completeness path -- same results as the reference's kernels
// instantiated for these `scalar_t` (csrc/cuda/knn_cuda.cu:125,
// csrc/cuda/radius_cuda.cu:84-85), no tuning beyond LDS tiling.  Also the
// `nearest` search (csrc/cuda/nearest_cuda.cu:10-66) for fp64, fp16 and for
// fp32 points of more than 8 dimensions.
//
// Arithmetic per element type (`Traits`):
//   fp64        everything in double, `acc += a * b` as one fused multiply-add
//               (what a GPU compiler makes of the reference source), sentinel
//               1e10;
//   fp16, bf16  c10::Half / c10::BFloat16 semantics: every operator converts
//               to float, operates, and rounds the result back to 16 bits
//               (torch/headeronly/util/Half.h:501-560), so each difference,
//               product and sum rounds once and nothing is fused; the kNN
//               sentinel 1e10 becomes +inf in fp16.  Values travel as floats
//               that are representable in the 16-bit type, which lets the
//               16-bit types reuse the 64-bit (float distance, row) keys.
#include "device_utils.hpp"

#include <algorithm>
#include <cstdlib>
#include "launchers.hpp"

#include <hip/hip_fp16.h>

namespace pca {

namespace {

// float -> nearest IEEE half (ties to even) -> float, on the host
float host_round_to_half(float f) {
  uint32_t x;
  __builtin_memcpy(&x, &f, 4);
  const uint32_t sign = x & 0x80000000u;
  uint32_t ax = x & 0x7fffffffu;
  uint32_t out;
  if (ax > 0x7f800000u) {
    out = 0x7fc00000u; // NaN
  } else if (ax >= 0x477ff000u) {
    out = 0x7f800000u; // overflows to infinity
  } else if (ax < 0x38800000u) {
    // subnormal half: multiples of 2^-24; adding and subtracting 0.5 makes
    // the float adder do the round-to-nearest-even at that position
    float a;
    __builtin_memcpy(&a, &ax, 4);
    a = (a + 0.5f) - 0.5f;
    __builtin_memcpy(&out, &a, 4);
  } else {
    // normal half: keep 10 fraction bits
    const uint32_t rem = ax & 0x1fffu;
    ax &= ~0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (ax & 0x2000u)))
      ax += 0x2000u;
    out = ax;
  }
  out |= sign;
  float r;
  __builtin_memcpy(&r, &out, 4);
  return r;
}

// ---- element-type traits ---------------------------------------------------

struct F64Traits {
  typedef double store_t;
  typedef double calc_t;
  static __device__ __forceinline__ calc_t load(store_t v) { return v; }
  static __device__ __forceinline__ calc_t sq_step(calc_t x, calc_t y,
                                                   calc_t acc) {
    const calc_t d = x - y;
    return __builtin_fma(d, d, acc);
  }
  static __device__ __forceinline__ calc_t dot_step(calc_t x, calc_t y,
                                                    calc_t acc) {
    return __builtin_fma(x, y, acc);
  }
  static __device__ __forceinline__ calc_t norm(calc_t sq) {
    return __builtin_sqrt(sq);
  }
  static __device__ __forceinline__ calc_t cosine(calc_t dot, calc_t xn,
                                                  calc_t yn) {
    return 1.0 - dot / (xn * yn);
  }
  static __device__ __forceinline__ calc_t sentinel() { return 1e10; }
  static __device__ __forceinline__ calc_t nearest_limit() { return 1e38; }
  static calc_t narrow_r2(double r2) { return r2; }
};

// fp32 with fused multiply-adds (the `nearest` search only; kNN and radius
// have their own fp32 kernels)
struct F32Traits {
  typedef float store_t;
  typedef float calc_t;
  static __device__ __forceinline__ calc_t load(store_t v) { return v; }
  static __device__ __forceinline__ calc_t sq_step(calc_t x, calc_t y,
                                                   calc_t acc) {
    const calc_t d = x - y;
    return __builtin_fmaf(d, d, acc);
  }
  static __device__ __forceinline__ calc_t nearest_limit() {
    return kNearestLimit;
  }
};

template <bool BF16> struct R16Traits {
  typedef uint16_t store_t;
  typedef float calc_t;
  static __device__ __forceinline__ float round16(float v) {
    return round_to_16<BF16>(v);
  }
  static __device__ __forceinline__ calc_t load(store_t v) {
    if (BF16)
      return __uint_as_float((uint32_t)v << 16);
    return __half2float(__ushort_as_half(v));
  }
  // (the sums below end in comparisons only: round_in_chain)
  static __device__ __forceinline__ calc_t sq_step(calc_t x, calc_t y,
                                                   calc_t acc) {
    const float d = round_in_chain<BF16>(x - y);
    const float p = round_in_chain<BF16>(d * d);
    return round_in_chain<BF16>(acc + p);
  }
  static __device__ __forceinline__ calc_t dot_step(calc_t x, calc_t y,
                                                    calc_t acc) {
    const float p = round_in_chain<BF16>(x * y);
    return round_in_chain<BF16>(acc + p);
  }
  static __device__ __forceinline__ calc_t norm(calc_t sq) {
    return round16(__builtin_sqrtf(sq));
  }
  static __device__ __forceinline__ calc_t cosine(calc_t dot, calc_t xn,
                                                  calc_t yn) {
    const float den = round16(xn * yn);
    const float t = round16(dot / den);
    return round16((float)(1.0 - (double)t));
  }
  static __device__ __forceinline__ calc_t sentinel() {
    return round16(1e10f);
  }
  // `scalar_t best = 1e38`: +inf in fp16
  static __device__ __forceinline__ calc_t nearest_limit() {
    return round16(1e38f);
  }
  // (scalar_t)(r * r): double -> float -> 16 bits
  static calc_t narrow_r2(double r2) {
    float f = (float)r2;
    uint32_t x;
    __builtin_memcpy(&x, &f, 4);
    if (BF16) {
      if ((x & 0x7fffffffu) > 0x7f800000u)
        x = 0x7fc00000u;
      else {
        x += 0x7fffu + ((x >> 16) & 1u);
        x &= 0xffff0000u;
      }
      __builtin_memcpy(&f, &x, 4);
      return f;
    }
    return host_round_to_half(f);
  }
};

// ---- top-k lists -----------------------------------------------------------

// float distances: 64-bit (distance, row) keys, see device_utils.hpp.  The
// empty slot carries the type's sentinel distance.
template <int K> struct KeyList {
  double b[K];
  float sentinel;
  __device__ __forceinline__ void init(int k, float sent) {
    sentinel = sent;
#pragma unroll
    for (int j = 0; j < K; ++j)
      b[j] = (j < K - k) ? lowest_key() : make_key(sent, 0xffffffffu);
  }
  __device__ __forceinline__ float worst() const { return key_dist(b[K - 1]); }
  // d < worst() for the lanes with `take`
  __device__ __forceinline__ void insert(bool take, float d, int row) {
    const double key =
        take ? make_key(d, (uint32_t)row) : make_key(sentinel, 0xffffffffu);
    sorted_insert<K>(b, key);
  }
  __device__ __forceinline__ int row_at(int j) const { return key_row(b[j]); }
  __device__ __forceinline__ double dist_at(int j) const {
    return (double)key_dist(b[j]);
  }
};

// double distances: separate distance / row arrays, branch-free insertion
// that keeps an earlier entry ahead of a later one of equal distance.
template <int K> struct PairList {
  double dist[K];
  int row[K];
  __device__ __forceinline__ void init(int k, double sent) {
#pragma unroll
    for (int j = 0; j < K; ++j) {
      dist[j] = (j < K - k) ? -__builtin_inf() : sent;
      row[j] = -1;
    }
  }
  __device__ __forceinline__ double worst() const { return dist[K - 1]; }
  __device__ __forceinline__ void insert(bool take, double d, int r) {
    const double dd = take ? d : __builtin_inf();
#pragma unroll
    for (int j = K - 1; j >= 1; --j) {
      const bool here = dd < dist[j];
      const bool before = dd < dist[j - 1];
      row[j] = before ? row[j - 1] : (here ? r : row[j]);
      dist[j] = before ? dist[j - 1] : (here ? dd : dist[j]);
    }
    const bool here = dd < dist[0];
    row[0] = here ? r : row[0];
    dist[0] = here ? dd : dist[0];
  }
  __device__ __forceinline__ int row_at(int j) const { return row[j]; }
  __device__ __forceinline__ double dist_at(int j) const { return dist[j]; }
};

template <typename Tr, int K> struct ListFor {
  typedef KeyList<K> type;
};
template <int K> struct ListFor<F64Traits, K> {
  typedef PairList<K> type;
};

// ---- kernels ---------------------------------------------------------------

template <typename Tr>
__global__ __launch_bounds__(kBlock) void row_norm_any_kernel(
    const typename Tr::store_t *__restrict__ x, int n, int d,
    typename Tr::calc_t *__restrict__ norm) {
  const int row = blockIdx.x * kBlock + threadIdx.x;
  if (row >= n)
    return;
  typename Tr::calc_t s = 0;
  for (int c = 0; c < d; ++c) {
    const typename Tr::calc_t v = Tr::load(x[(size_t)row * d + c]);
    s = Tr::dot_step(v, v, s);
  }
  norm[row] = Tr::norm(s);
}

constexpr int kAnyTile = 16;  // candidates per LDS tile
constexpr int kAnySlab = 128; // components of a tile resident in LDS
constexpr int kAnyChunk = 8;  // query components held in registers

// One query per lane, 256 queries of one segment per workgroup; every
// candidate's distance is accumulated in the reference's operation order and
// offered to the lane's list as soon as its tile is complete.
template <typename Tr, int K, bool COSINE>
__global__ __launch_bounds__(kBlock) void knn_any_kernel(
    const typename Tr::store_t *__restrict__ x,
    const typename Tr::store_t *__restrict__ y,
    const int64_t *__restrict__ ptr_x, const int64_t *__restrict__ ptr_y,
    const typename Tr::calc_t *__restrict__ x_norm, int n, int m, int d,
    int num_segments, int k, const int *__restrict__ work_start,
    int *__restrict__ out_idx, int *__restrict__ out_count, int num_chunks,
    double *__restrict__ part_dist, int *__restrict__ part_row) {
  typedef typename Tr::calc_t calc_t;
  constexpr int TG = kAnyTile;
  __shared__ calc_t xs[TG][kAnySlab];
  __shared__ calc_t xn[TG];

  const int tid = threadIdx.x;
  // work item = (slice of the segment's x rows, tile of queries)
  const int total_tiles = work_start[num_segments];
  if (total_tiles == 0)
    return;
  const int chunk = blockIdx.x / total_tiles;
  const int tile = blockIdx.x - chunk * total_tiles;
  if (chunk >= num_chunks)
    return;
  const int seg = find_segment(work_start, num_segments, tile);
  const int x_begin = ptr_x ? (int)ptr_x[seg] : 0;
  const int x_end = ptr_x ? (int)ptr_x[seg + 1] : n;
  const int y_begin = ptr_y ? (int)ptr_y[seg] : 0;
  const int y_end = ptr_y ? (int)ptr_y[seg + 1] : m;
  const int q = y_begin + (tile - work_start[seg]) * kBlock + tid;
  const bool valid = q < y_end;
  const typename Tr::store_t *yrow = y + (size_t)(valid ? q : y_begin) * d;
  const int seg_len = x_end - x_begin;
  const int chunk_len =
      ((seg_len + num_chunks - 1) / num_chunks + TG - 1) / TG * TG;
  const int c_begin = min(x_end, x_begin + chunk * chunk_len);
  const int c_end = min(x_end, c_begin + chunk_len);

  typename ListFor<Tr, K>::type list;
  list.init(k, Tr::sentinel());

  calc_t y_norm = 0;
  if (COSINE) {
    calc_t s = 0;
    for (int c = 0; c < d; ++c) {
      const calc_t v = Tr::load(yrow[c]);
      s = Tr::dot_step(v, v, s);
    }
    y_norm = Tr::norm(s);
  }

  for (int base = c_begin; base < c_end; base += TG) {
    const int rows = min(TG, c_end - base);
    calc_t acc[TG];
#pragma unroll
    for (int j = 0; j < TG; ++j)
      acc[j] = 0;

    for (int slab = 0; slab < d; slab += kAnySlab) {
      const int width = min(kAnySlab, d - slab);
      __syncthreads();
      for (int i = tid; i < TG * width; i += kBlock) {
        const int r = i / width;
        const int c = i - r * width;
        xs[r][c] = r < rows ? Tr::load(x[(size_t)(base + r) * d + slab + c])
                            : (calc_t)0;
      }
      if (COSINE && slab == 0 && tid < TG)
        xn[tid] = tid < rows ? x_norm[base + tid] : (calc_t)1;
      __syncthreads();

      for (int c0 = 0; c0 < width; c0 += kAnyChunk) {
        calc_t yv[kAnyChunk];
#pragma unroll
        for (int c = 0; c < kAnyChunk; ++c)
          yv[c] = (c0 + c < width) ? Tr::load(yrow[slab + c0 + c]) : (calc_t)0;
        const int count = min(kAnyChunk, width - c0);
#pragma unroll
        for (int j = 0; j < TG; ++j) {
#pragma unroll
          for (int c = 0; c < kAnyChunk; ++c) {
            if (c < count) {
              if (COSINE)
                acc[j] = Tr::dot_step(xs[j][c0 + c], yv[c], acc[j]);
              else
                acc[j] = Tr::sq_step(xs[j][c0 + c], yv[c], acc[j]);
            }
          }
        }
      }
    }

#pragma unroll
    for (int j = 0; j < TG; ++j) {
      if (j < rows) { // uniform
        calc_t dist = acc[j];
        if (COSINE)
          dist = Tr::cosine(dist, xn[j], y_norm);
        // strict: an equal distance never displaces an earlier, lower row
        const bool take = dist < list.worst();
        if (__any(take))
          list.insert(take, dist, base + j);
      }
    }
  }

  if (num_chunks > 1) {
    // this slice's list, [item][slot][query of the tile]: knn_any_merge_kernel
    // unites the slices
    const size_t at = (size_t)(chunk * total_tiles + tile) * k * kBlock + tid;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int e = j - (K - k);
      if (e >= 0) {
        part_dist[at + (size_t)e * kBlock] = list.dist_at(j);
        part_row[at + (size_t)e * kBlock] = list.row_at(j);
      }
    }
    return;
  }
  if (valid) {
    int found = 0;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int e = j - (K - k);
      const int r = list.row_at(j);
      if (e >= 0 && r >= 0) {
        out_idx[(size_t)q * k + e] = r;
        ++found;
      }
    }
    out_count[q] = found;
  }
}

// Unites the lists of a query's slices (ascending slices = ascending rows, so
// an entry of equal distance from a later slice stays behind the earlier
// ones, as in one scan over all rows).
template <typename Tr, int K>
__global__ __launch_bounds__(kBlock) void knn_any_merge_kernel(
    const int64_t *__restrict__ ptr_y, int m, int num_segments, int k,
    const int *__restrict__ work_start, int num_chunks,
    const double *__restrict__ part_dist, const int *__restrict__ part_row,
    int *__restrict__ out_idx, int *__restrict__ out_count) {
  typedef typename Tr::calc_t calc_t;
  const int tid = threadIdx.x;
  const int total_tiles = work_start[num_segments];
  const int tile = blockIdx.x;
  if (tile >= total_tiles)
    return;
  const int seg = find_segment(work_start, num_segments, tile);
  const int y_begin = ptr_y ? (int)ptr_y[seg] : 0;
  const int y_end = ptr_y ? (int)ptr_y[seg + 1] : m;
  const int q = y_begin + (tile - work_start[seg]) * kBlock + tid;
  typename ListFor<Tr, K>::type list;
  list.init(k, Tr::sentinel());
  for (int c = 0; c < num_chunks; ++c) {
    const size_t at = (size_t)(c * total_tiles + tile) * k * kBlock + tid;
    for (int e = 0; e < k; ++e) {
      const int row = part_row[at + (size_t)e * kBlock];
      const calc_t dist = (calc_t)part_dist[at + (size_t)e * kBlock];
      // (lists are ascending: behind an entry that does not get in, or an
      // empty slot, nothing of this slice does)
      const bool take = row >= 0 && dist < list.worst();
      if (!__any(take))
        break;
      list.insert(take, dist, row);
    }
  }
  if (q < y_end) {
    int found = 0;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int e = j - (K - k);
      const int r = list.row_at(j);
      if (e >= 0 && r >= 0) {
        out_idx[(size_t)q * k + e] = r;
        ++found;
      }
    }
    out_count[q] = found;
  }
}

// The `nearest` search with the mapping of knn_any_kernel: one searching row
// (a row of y here) per lane, candidates (rows of x) through LDS.  A lane
// keeps the candidate that is smallest by (distance, (row - start) % 1024,
// row) -- the one the reference's block reduction returns -- and the result
// is 0 when no distance is below the limit (csrc/cuda/nearest_cuda.cu:31-64).
template <typename Tr>
__global__ __launch_bounds__(kBlock) void nearest_any_kernel(
    const typename Tr::store_t *__restrict__ x,
    const typename Tr::store_t *__restrict__ y,
    const int64_t *__restrict__ ptr_x, const int64_t *__restrict__ ptr_y,
    int n, int m, int d, int num_segments, const int *__restrict__ work_start,
    int64_t *__restrict__ out) {
  typedef typename Tr::calc_t calc_t;
  constexpr int TG = kAnyTile;
  __shared__ calc_t xs[TG][kAnySlab];

  const int tid = threadIdx.x;
  const int tile = blockIdx.x;
  if (tile >= work_start[num_segments])
    return;
  const int seg = find_segment(work_start, num_segments, tile);
  const int x_begin = ptr_x ? (int)ptr_x[seg] : 0;
  const int x_end = ptr_x ? (int)ptr_x[seg + 1] : n;
  const int y_begin = ptr_y ? (int)ptr_y[seg] : 0;
  const int y_end = ptr_y ? (int)ptr_y[seg + 1] : m;
  const int q = y_begin + (tile - work_start[seg]) * kBlock + tid;
  const bool valid = q < y_end;
  const typename Tr::store_t *yrow = y + (size_t)(valid ? q : y_begin) * d;

  constexpr uint32_t kNone = 0xffffffffu;
  const calc_t limit = Tr::nearest_limit();
  calc_t best = limit;
  uint32_t best_tie = kNone;

  for (int base = x_begin; base < x_end; base += TG) {
    const int rows = min(TG, x_end - base);
    calc_t acc[TG];
#pragma unroll
    for (int j = 0; j < TG; ++j)
      acc[j] = 0;

    for (int slab = 0; slab < d; slab += kAnySlab) {
      const int width = min(kAnySlab, d - slab);
      __syncthreads();
      for (int i = tid; i < TG * width; i += kBlock) {
        const int r = i / width;
        const int c = i - r * width;
        xs[r][c] = r < rows ? Tr::load(x[(size_t)(base + r) * d + slab + c])
                            : (calc_t)0;
      }
      __syncthreads();

      for (int c0 = 0; c0 < width; c0 += kAnyChunk) {
        calc_t yv[kAnyChunk];
#pragma unroll
        for (int c = 0; c < kAnyChunk; ++c)
          yv[c] = (c0 + c < width) ? Tr::load(yrow[slab + c0 + c]) : (calc_t)0;
        const int count = min(kAnyChunk, width - c0);
#pragma unroll
        for (int j = 0; j < TG; ++j) {
#pragma unroll
          for (int c = 0; c < kAnyChunk; ++c) {
            if (c < count)
              acc[j] = Tr::sq_step(xs[j][c0 + c], yv[c], acc[j]);
          }
        }
      }
    }

#pragma unroll
    for (int j = 0; j < TG; ++j) {
      if (j < rows) { // uniform
        const calc_t dist = acc[j];
        const uint32_t tie = nearest_tie((uint32_t)(base + j - x_begin));
        // (best < limit exactly when a candidate has been kept)
        const bool take =
            dist < limit && (dist < best || (dist == best && tie < best_tie));
        best = take ? dist : best;
        best_tie = take ? tie : best_tie;
      }
    }
  }

  if (valid)
    out[q] = best_tie != kNone
                 ? (int64_t)x_begin + (int64_t)nearest_rel(best_tie)
                 : 0;
}

constexpr int QW = kRadiusQueriesPerWave;
constexpr int kWavesPerBlock = kBlock / kWave;

// Same mapping as radius_kernel in radius.hip (a wave owns QW queries, its
// lanes take 64 consecutive x rows, hits are compacted with ballot + mbcnt).
template <typename Tr>
__global__ __launch_bounds__(kBlock) void radius_any_kernel(
    const typename Tr::store_t *__restrict__ x,
    const typename Tr::store_t *__restrict__ y,
    const int64_t *__restrict__ ptr_x, const int64_t *__restrict__ ptr_y,
    int n, int m, int d, int num_segments, typename Tr::calc_t r2, int slots,
    int ignore_same_index, const int *__restrict__ work_start,
    int *__restrict__ out_idx, int *__restrict__ out_count) {
  typedef typename Tr::calc_t calc_t;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int task = blockIdx.x * kWavesPerBlock + wave;
  if (task >= work_start[num_segments])
    return;
  const int seg = find_segment(work_start, num_segments, task);
  const int x_begin = ptr_x ? (int)ptr_x[seg] : 0;
  const int x_end = ptr_x ? (int)ptr_x[seg + 1] : n;
  const int y_begin = ptr_y ? (int)ptr_y[seg] : 0;
  const int y_end = ptr_y ? (int)ptr_y[seg + 1] : m;
  const int q0 = y_begin + (task - work_start[seg]) * QW;
  const int nq = min(QW, y_end - q0);

  int count[QW];
  bool open[QW];
#pragma unroll
  for (int qi = 0; qi < QW; ++qi) {
    count[qi] = 0;
    open[qi] = qi < nq;
  }
  int num_open = nq;

  for (int base = x_begin; base < x_end && num_open > 0; base += kWave) {
    const int row = base + lane;
    const bool in_range = row < x_end;
    calc_t acc[QW];
#pragma unroll
    for (int qi = 0; qi < QW; ++qi)
      acc[qi] = 0;
    for (int c = 0; c < d; ++c) {
      const calc_t xv = in_range ? Tr::load(x[(size_t)row * d + c]) : (calc_t)0;
#pragma unroll
      for (int qi = 0; qi < QW; ++qi) {
        if (!open[qi])
          continue;
        acc[qi] =
            Tr::sq_step(xv, Tr::load(y[(size_t)(q0 + qi) * d + c]), acc[qi]);
      }
    }
#pragma unroll
    for (int qi = 0; qi < QW; ++qi) {
      if (!open[qi])
        continue;
      const int q = q0 + qi;
      bool hit = in_range && acc[qi] < r2;
      if (ignore_same_index)
        hit = hit && row != q;
      const uint64_t mask = __ballot(hit);
      if (mask != 0) {
        const int pos =
            count[qi] + __builtin_amdgcn_mbcnt_hi(
                            (uint32_t)(mask >> 32),
                            __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
        if (hit && pos < slots)
          out_idx[(size_t)q * slots + pos] = row;
        count[qi] += __builtin_popcountll(mask);
        if (count[qi] >= slots) {
          open[qi] = false;
          --num_open;
        }
      }
    }
  }

  if (lane < nq) {
    int c = 0;
#pragma unroll
    for (int qi = 0; qi < QW; ++qi)
      if (lane == qi)
        c = min(count[qi], slots);
    out_count[q0 + lane] = c;
  }
}

// ---- launch helpers --------------------------------------------------------

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// bytes of the slices' distances (then their rows follow)
size_t part_dist_bytes(int m, int num_segments, int k, int chunks) {
  const size_t tiles = plan_upper_bound(m, num_segments, kBlock);
  return align256(sizeof(double) * tiles * chunks * (size_t)k * kBlock);
}

template <typename Tr, int K>
void launch_knn_any_k(const SearchInput &in, int k, bool cosine, void *x_norm,
                      const int *work_start, int grid, const DenseResult &out,
                      hipStream_t stream, int chunks, void *scratch) {
  typedef typename Tr::store_t store_t;
  typedef typename Tr::calc_t calc_t;
  const store_t *x = static_cast<const store_t *>(in.x);
  const store_t *y = static_cast<const store_t *>(in.y);
  calc_t *norms = static_cast<calc_t *>(x_norm);
  double *part_dist = static_cast<double *>(scratch);
  int *part_row =
      chunks > 1 ? reinterpret_cast<int *>(
                       static_cast<char *>(scratch) +
                       part_dist_bytes(in.m, in.num_segments, k, chunks))
                 : nullptr;
  if (cosine) {
    hipLaunchKernelGGL((row_norm_any_kernel<Tr>),
                       dim3((in.n + kBlock - 1) / kBlock), dim3(kBlock), 0,
                       stream, x, in.n, in.d, norms);
    hipLaunchKernelGGL((knn_any_kernel<Tr, K, true>), dim3(grid * chunks),
                       dim3(kBlock), 0, stream, x, y, in.ptr_x, in.ptr_y,
                       norms, in.n, in.m, in.d, in.num_segments, k, work_start,
                       out.idx, out.count, chunks, part_dist, part_row);
  } else {
    hipLaunchKernelGGL((knn_any_kernel<Tr, K, false>), dim3(grid * chunks),
                       dim3(kBlock), 0, stream, x, y, in.ptr_x, in.ptr_y,
                       norms, in.n, in.m, in.d, in.num_segments, k, work_start,
                       out.idx, out.count, chunks, part_dist, part_row);
  }
  if (chunks > 1)
    hipLaunchKernelGGL((knn_any_merge_kernel<Tr, K>), dim3(grid), dim3(kBlock),
                       0, stream, in.ptr_y, in.m, in.num_segments, k,
                       work_start, chunks, part_dist, part_row, out.idx,
                       out.count);
}

template <typename Tr>
hipError_t launch_knn_any_t(const SearchInput &in, int k, bool cosine,
                            void *x_norm, const int *work_start, int grid,
                            const DenseResult &out, hipStream_t stream,
                            void *scratch) {
  const int chunks =
      scratch ? knn_anytype_slices(in.n, in.m, in.num_segments) : 1;
  if (k <= 16)
    launch_knn_any_k<Tr, 16>(in, k, cosine, x_norm, work_start, grid, out,
                             stream, chunks, scratch);
  else if (k <= 48)
    launch_knn_any_k<Tr, 48>(in, k, cosine, x_norm, work_start, grid, out,
                             stream, chunks, scratch);
  else
    launch_knn_any_k<Tr, 100>(in, k, cosine, x_norm, work_start, grid, out,
                              stream, chunks, scratch);
  return hipGetLastError();
}

template <typename Tr>
hipError_t launch_radius_any_t(const SearchInput &in, double r,
                               bool ignore_same_index, const int *work_start,
                               int task_bound, const DenseResult &out,
                               hipStream_t stream) {
  typedef typename Tr::store_t store_t;
  const int grid = (task_bound + kWavesPerBlock - 1) / kWavesPerBlock;
  if (grid <= 0)
    return hipSuccess;
  hipLaunchKernelGGL((radius_any_kernel<Tr>), dim3(grid), dim3(kBlock), 0,
                     stream, static_cast<const store_t *>(in.x),
                     static_cast<const store_t *>(in.y), in.ptr_x, in.ptr_y,
                     in.n, in.m, in.d, in.num_segments, Tr::narrow_r2(r * r),
                     out.slots, ignore_same_index ? 1 : 0, work_start, out.idx,
                     out.count);
  return hipGetLastError();
}

template <typename Tr>
hipError_t launch_nearest_any_t(const SearchInput &in, const int *work_start,
                                int grid, int64_t *out, hipStream_t stream) {
  typedef typename Tr::store_t store_t;
  if (grid <= 0)
    return hipSuccess;
  hipLaunchKernelGGL((nearest_any_kernel<Tr>), dim3(grid), dim3(kBlock), 0,
                     stream, static_cast<const store_t *>(in.x),
                     static_cast<const store_t *>(in.y), in.ptr_x, in.ptr_y,
                     in.n, in.m, in.d, in.num_segments, work_start, out);
  return hipGetLastError();
}

} // namespace

hipError_t launch_nearest_any(int dtype, const SearchInput &in,
                              const int *work_start, int grid_bound,
                              int64_t *out, hipStream_t stream) {
  switch (dtype) {
  case 0:
    return launch_nearest_any_t<F32Traits>(in, work_start, grid_bound, out,
                                           stream);
  case 1:
    return launch_nearest_any_t<F64Traits>(in, work_start, grid_bound, out,
                                           stream);
  case 2:
    return launch_nearest_any_t<R16Traits<false>>(in, work_start, grid_bound,
                                                  out, stream);
  default:
    return hipErrorInvalidValue;
  }
}

size_t anytype_norm_bytes(int n) { return sizeof(double) * (size_t)n; }

int knn_anytype_slices(int n, int m, int num_segments) {
  // enough work items for four workgroups per CU, slices of at least 32 LDS
  // tiles on average
  const int tiles = plan_upper_bound(m, num_segments, kBlock);
  const int want = (1024 + tiles - 1) / tiles;
  const int by_length = (n / num_segments) / (32 * kAnyTile);
  int chunks = std::max(1, std::min(std::min(want, 64), by_length));
  if (const char *env = std::getenv("PCA_KNN_SLICES")) {
    const int v = std::atoi(env);
    if (v >= 1 && v <= 64)
      chunks = v;
  }
  return chunks;
}

size_t knn_anytype_scratch_bytes(int n, int m, int num_segments, int k) {
  const int chunks = knn_anytype_slices(n, m, num_segments);
  if (chunks <= 1)
    return 0;
  const size_t tiles = plan_upper_bound(m, num_segments, kBlock);
  return part_dist_bytes(m, num_segments, k, chunks) +
         align256(sizeof(int) * tiles * chunks * (size_t)k * kBlock);
}

hipError_t launch_knn_anytype(int dtype, const SearchInput &in, int k,
                              bool cosine, void *x_norm,
                              const int *work_start, int grid_bound,
                              const DenseResult &out, hipStream_t stream,
                              void *scratch) {
  switch (dtype) {
  case 1:
    return launch_knn_any_t<F64Traits>(in, k, cosine, x_norm, work_start,
                                       grid_bound, out, stream, scratch);
  case 2:
    return launch_knn_any_t<R16Traits<false>>(in, k, cosine, x_norm,
                                              work_start, grid_bound, out,
                                              stream, scratch);
  case 3:
    return launch_knn_any_t<R16Traits<true>>(in, k, cosine, x_norm,
                                             work_start, grid_bound, out,
                                             stream, scratch);
  default:
    return hipErrorInvalidValue;
  }
}

float narrow_r2_16bit(double r2, bool bf16) {
  return bf16 ? R16Traits<true>::narrow_r2(r2) : R16Traits<false>::narrow_r2(r2);
}

hipError_t launch_radius_anytype(int dtype, const SearchInput &in, double r,
                                 bool ignore_same_index,
                                 const int *work_start, int task_bound,
                                 const DenseResult &out, hipStream_t stream) {
  switch (dtype) {
  case 1:
    return launch_radius_any_t<F64Traits>(in, r, ignore_same_index, work_start,
                                          task_bound, out, stream);
  case 2:
    return launch_radius_any_t<R16Traits<false>>(
        in, r, ignore_same_index, work_start, task_bound, out, stream);
  case 3:
    return launch_radius_any_t<R16Traits<true>>(
        in, r, ignore_same_index, work_start, task_bound, out, stream);
  default:
    return hipErrorInvalidValue;
  }
}

} // namespace pca
