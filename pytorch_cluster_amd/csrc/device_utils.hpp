// Device-side helpers shared by the neighbour-search kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pca {

constexpr int kWave = 64;
constexpr int kBlock = 256; // 4 waves: one per SIMD of a CU

// v rounded to the nearest fp16 (BF16: bfloat16) number, ties to even, as a
// float: what c10::Half / c10::BFloat16 arithmetic does after every operation
// (torch/headeronly/util/Half.h:501-560, BFloat16.h).
template <bool BF16> __device__ __forceinline__ float round_to_16(float v) {
  if (BF16) {
    // the device's own conversion (v_cvt_pk_bf16_f32) and a shift: for every
    // float that is not a NaN it returns the bits of c10's integer formula
    // (x + 0x7fff + ((x >> 16) & 1), upper half), denormal numbers and the
    // overflow to infinity included -- all 2^32 inputs are compared by
    // pca_probe_bf16_rounding (csrc/probes/rounding_probe.hip); it keeps a
    // NaN's sign and payload where c10 returns 0x7fc0, hence the first line
    if (v != v)
      return __uint_as_float(0x7fc00000u);
    return (float)(__bf16)v;
  }
  return (float)(_Float16)v;
}

// The same inside a chain of operations whose end is only ever compared
// (a NaN stays a NaN, whatever its sign and payload): two instructions fewer
// per rounding for bfloat16.
template <bool BF16> __device__ __forceinline__ float round_in_chain(float v) {
  if (BF16)
    return (float)(__bf16)v;
  return (float)(_Float16)v;
}

// What is left of a term of a sum in 16-bit arithmetic, at worst.  The
// reference adds d squares (x_j - y_j)^2 one after the other and rounds the
// difference, the square and every sum to 16 bits: a term has been rounded
// 3 + e times when e sums lie behind it, so the value H the chain ends on is
// at least  sum_j (1 - u)^(3 + d - j) (x_j - y_j)^2  minus what underflow takes
// (u = 2^-11 for fp16, 2^-8 for bf16, plus 2^-23: the fp32 operation under
// every rounding).  kChainKeep.s[bf16][e] is the square root of
// (1 - u)^(3 + e), rounded DOWN to 13 (bf16: 16) significant bits: a number
// of 11 (8) significant bits times such a factor is exact in fp32, so rows
// and queries scaled by it component
// by component have exactly  sum_j s_j^2 (x_j - y_j)^2 <= H + underflow  as
// their squared distance -- the lower bound of the 16-bit searches' filter.
constexpr int kChainKeepSums = 128; // sums behind a term: up to this many
struct ChainKeep {
  float s[2][kChainKeepSums + 1];
};
constexpr double chain_keep_root(double v) { // sqrt of v in (1/4, 1]
  double r = v;
  for (int i = 0; i < 64; ++i)
    r = 0.5 * (r + v / r);
  return r;
}
constexpr ChainKeep make_chain_keep() {
  ChainKeep t{};
  for (int b = 0; b < 2; ++b) {
    const double u = (b ? 1.0 / 256.0 : 1.0 / 2048.0) + 1.0 / 8388608.0;
    double keep = (1.0 - u) * (1.0 - u) * (1.0 - u);
    for (int e = 0; e <= kChainKeepSums; ++e) {
      // (1 - 2^-30: the root above is a double's, not the real number's)
      const double root = chain_keep_root(keep) * (1.0 - 1.0 / 1073741824.0);
      // root in [1/2, 1): 13 (16) bits behind the binary point, the first of
      // them 1
      const double unit = b ? 65536.0 : 8192.0;
      const long long cut = (long long)(root * unit);
      t.s[b][e] = (float)((double)cut / unit);
      keep *= 1.0 - u;
    }
  }
  return t;
}
__device__ constexpr ChainKeep kChainKeep = make_chain_keep();
static_assert(make_chain_keep().s[1][kChainKeepSums] >= 0.5f &&
                  make_chain_keep().s[0][0] < 1.0f,
              "bits behind the point are significant bits");
// the factor of component j of d (fp32 rows: 1)
template <int R16>
__device__ __forceinline__ float chain_keep(int d, int j) {
  if (R16 == 1 || R16 == 2)
    return kChainKeep.s[R16 - 1][d - j];
  return 1.0f;
}

// c10::BFloat16's rounding as the integer formula it is written as
// (torch/headeronly/util/BFloat16.h round_to_nearest_even): the yardstick of
// the comparison named above.
__device__ __forceinline__ float round_to_bf16_by_integers(float v) {
  uint32_t x = __float_as_uint(v);
  if ((x & 0x7fffffffu) > 0x7f800000u)
    return __uint_as_float(0x7fc00000u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return __uint_as_float(x & 0xffff0000u);
}

// Smallest norm of a row or query the cosine filters take: below it the
// squares and products of the reference's own chains reach the denormal range
// (a few bits each), the distance it computes strays from the cosine by
// whole per cents, and no margin of a filter holds; such vectors are always
// evaluated exactly.
constexpr float kCosTinyNorm = 1e-18f;

// Distance every kNN slot starts from; a candidate must be strictly below it
// to be returned (csrc/cuda/knn_cuda.cu:48,68 in the reference).
constexpr float kKnnSentinel = 1e10f;

// ---------------------------------------------------------------------------
// 64-bit selection keys.
//
// A candidate is the pair (distance, x row).  The reference orders neighbours
// by ascending distance and, among equal distances, by ascending row.  Packing
// the float's bit pattern into the high word and the row into the low word of
// one 64-bit value and reading that value as an IEEE double gives a single
// number whose floating-point order is exactly that lexicographic order:
//   * for d >= 0 the bit patterns of floats order like the floats, and
//     positive doubles order like their bit patterns;
//   * for d < 0 (only the cosine distance can be slightly negative) a larger
//     magnitude is more negative in both formats; the low word then holds the
//     complemented row so that ties still come out in ascending row order.
// The high word is biased by one double-exponent step so that no key is a
// denormal double, whatever the kernel's denormal mode is.  Keys are never
// NaN: the high word stays below 0x7ff00000 because only distances below
// kKnnSentinel are ever packed.
//
// With keys as doubles, one step of a sorted-insertion network is
//   b[j] = min(b[j], max(b[j-1], key))
// i.e. two full-rate f64 VALU instructions per slot and no index bookkeeping.
// ---------------------------------------------------------------------------
constexpr uint32_t kKeyBias = 0x00100000u;

__device__ __forceinline__ double make_key(float d, uint32_t row) {
  uint32_t hi = __float_as_uint(d);
  uint32_t lo = (hi & 0x80000000u) ? ~row : row;
  hi += kKeyBias;
  return __hiloint2double((int)hi, (int)lo);
}

__device__ __forceinline__ float key_dist(double key) {
  return __uint_as_float((uint32_t)__double2hiint(key) - kKeyBias);
}

__device__ __forceinline__ int key_row(double key) {
  uint32_t hi = (uint32_t)__double2hiint(key) - kKeyBias;
  uint32_t lo = (uint32_t)__double2loint(key);
  return (int)((hi & 0x80000000u) ? ~lo : lo);
}

// Key of an empty slot: distance = sentinel, row = -1.  Larger than every key
// a real candidate can have.
__device__ __forceinline__ double empty_key() {
  return __hiloint2double((int)(0x501502F9u /* 1e10f */ + kKeyBias), -1);
}

// The `nearest` operator (csrc/cuda/nearest_cuda.cu:10-66 in the reference)
// is a search for one neighbour with two differences: a candidate must be
// strictly below 1e38 instead of 1e10 (:31,41), and among candidates of equal
// distance the reference's block of 1,024 threads -- thread t scans the rows
// start + t, start + t + 1024, ... and keeps its first minimum (:33-44), the
// pairwise reduction keeps the lower thread on ties (:46-59) -- returns the
// one with the smallest (row - start) % 1024, then the smallest row.  With
// that pair in the low word of the key (10 bits of slot, 22 bits of
// (row - start) / 1024; rows stay below 2^31) the key order is that rule.
constexpr float kNearestLimit = 1e38f;

__device__ __forceinline__ uint32_t nearest_tie(uint32_t rel) {
  return ((rel & 1023u) << 22) | (rel >> 10);
}

__device__ __forceinline__ uint32_t nearest_rel(uint32_t tie) {
  return ((tie & 0x3fffffu) << 10) | (tie >> 22);
}

// Limit and empty-slot key of a search: the kNN ones, or those of `nearest`.
template <bool NEAREST> struct SearchLimit {
  static constexpr float value = NEAREST ? kNearestLimit : kKnnSentinel;
  static __device__ __forceinline__ double empty() {
    return __hiloint2double((int)(__float_as_uint(value) + kKeyBias), -1);
  }
};

// Key below every real key: fills the slots of a K-wide list that the caller
// did not ask for (k < K), so that they never take part in the selection.
__device__ __forceinline__ double lowest_key() {
  return __hiloint2double((int)0xfff00000u, 0); // -inf
}

// v_min_f64 / v_max_f64 issued directly: the operands are never NaN, so the
// canonicalisation a compiler adds around fmin()/fmax() is not needed.
__device__ __forceinline__ double key_min(double a, double b) {
  double r;
  asm("v_min_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

__device__ __forceinline__ double key_max(double a, double b) {
  double r;
  asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// Inserts `key` into the ascending list b[0..K) and drops the largest entry.
template <int K>
__device__ __forceinline__ void sorted_insert(double (&b)[K], double key) {
#pragma unroll
  for (int j = K - 1; j >= 1; --j)
    b[j] = key_min(b[j], key_max(b[j - 1], key));
  b[0] = key_min(b[0], key);
}

// Unites the sorted lists of the two lanes of a query (l and l + 32) in the
// lower lane: afterwards its slots K - k .. K - 1 hold the k smallest keys of
// both lists, ascending (slots below K - k: the padding they held before).
// Entry i of the lower lane meets the upper lane's entry K - 1 - (i - s),
// s = K - k: the minimum of an ascending and a descending sequence holds the
// k smallest of both and is bitonic, and a bitonic merge network (over the
// next power of two, the padding in front staying where it is) sorts it:
// K + K log2(K) minimum / maximum operations instead of the K (2 K - 1) of K
// insertions.  s takes one of eight values for a list width (k is uniform),
// picked by a branch so that every register index is a constant.
template <int K>
__device__ __forceinline__ void unite_halves(double (&best)[K], int k,
                                                 int half) {
  constexpr int P = K <= 8 ? 8 : K <= 16 ? 16 : K <= 32 ? 32 : 64;
  static_assert(K <= 64 && K % 8 == 0 || K < 8, "list widths in steps of 8");
  const int s_now = K - k;
#pragma unroll
  for (int s = 0; s < (K < 8 ? K : 8); ++s) {
    if (s != s_now)
      continue;
    asm volatile(""); // (keeps this a branch)
#pragma unroll
    for (int i = s; i < K; ++i) {
      const int j = K - 1 - (i - s); // the partner's entry for slot i
      const auto hi = __builtin_amdgcn_permlane32_swap(
          (unsigned)__double2hiint(best[j]), (unsigned)__double2hiint(best[j]),
          false, false);
      const auto lo = __builtin_amdgcn_permlane32_swap(
          (unsigned)__double2loint(best[j]), (unsigned)__double2loint(best[j]),
          false, false);
      // (element 1 of a swap: in a lower lane, the upper lane's value)
      const double upper = __hiloint2double((int)hi[1], (int)lo[1]);
      // (the upper lanes' lists stay as they are: later slots still read
      // them)
      const double united = key_min(best[i], upper);
      best[i] = half ? best[i] : united;
    }
  }
  // entry e of the network is slot e - (P - K); entries in front of it are
  // padding below every key and never move
#pragma unroll
  for (int stride = P / 2; stride >= 1; stride >>= 1) {
#pragma unroll
    for (int e = 0; e < P; ++e) {
      if ((e & stride) != 0 || e < P - K)
        continue;
      const int a = e - (P - K), b = a + stride;
      const double lo = key_min(best[a], best[b]);
      const double hi = key_max(best[a], best[b]);
      best[a] = lo;
      best[b] = hi;
    }
  }
}

// ---- fp32 values as sums of two bf16 numbers (matrix-core pre-filters) -----
typedef __bf16 mc_bf16x8_t __attribute__((ext_vector_type(8)));

// bf16 nearest-even of a finite float of moderate size, as the upper half of
// a float
__device__ __forceinline__ uint32_t mc_bf16_bits(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// v = hi + lo + r, |r| <= 2^-16 |v|
__device__ __forceinline__ void mc_split(float v, uint32_t &hi, uint32_t &lo) {
  hi = mc_bf16_bits(v);
  lo = mc_bf16_bits(v - __uint_as_float(hi << 16)); // the difference is exact
}

__device__ __forceinline__ float min3f(float a, float b, float c) {
  return __builtin_fminf(__builtin_fminf(a, b), c);
}

// Largest b in [0, num_segments) with start[b] <= v; `start` has
// num_segments + 1 non-decreasing entries and start[num_segments] > v.
__device__ __forceinline__ int find_segment(const int *__restrict__ start,
                                            int num_segments, int v) {
  int lo = 0, hi = num_segments;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (start[mid] <= v)
      lo = mid;
    else
      hi = mid;
  }
  return lo;
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  This
// maps the hardware block id to a logical one such that blocks with
// neighbouring logical ids (which scan the same segment of x) land on the same
// XCD.  `grid` must be a multiple of 8.
__device__ __forceinline__ int xcd_swizzle(int block, int grid) {
  return (block & 7) * (grid >> 3) + (block >> 3);
}

// Work items of ragged segments, by a single workgroup of kPlanThreads
// threads: work_start[b] = exclusive scan of ceil(rows of segment b /
// per_item), work_start[num_segments] = their total.  ptr == nullptr: one
// segment of m rows.  `partial`: kPlanThreads ints of LDS.
constexpr int kPlanThreads = 1024;
__device__ __forceinline__ void
plan_segments(const int64_t *__restrict__ ptr, int m, int num_segments,
              int per_item, int *__restrict__ work_start, int *partial) {
  const int tid = threadIdx.x;
  // contiguous chunk of segments per thread
  const int per_thread = (num_segments + kPlanThreads - 1) / kPlanThreads;
  const int b0 = min(tid * per_thread, num_segments);
  const int b1 = min(b0 + per_thread, num_segments);

  int sum = 0;
  for (int b = b0; b < b1; ++b) {
    const int64_t lo = ptr ? ptr[b] : 0;
    const int64_t hi = ptr ? ptr[b + 1] : m;
    const int len = (int)max((int64_t)0, hi - lo);
    sum += (len + per_item - 1) / per_item;
  }
  partial[tid] = sum;
  __syncthreads();
  // Hillis-Steele inclusive scan over the partial sums
  for (int off = 1; off < kPlanThreads; off <<= 1) {
    const int v = tid >= off ? partial[tid - off] : 0;
    __syncthreads();
    partial[tid] += v;
    __syncthreads();
  }
  int run = partial[tid] - sum; // exclusive prefix of this thread's chunk
  for (int b = b0; b < b1; ++b) {
    work_start[b] = run;
    const int64_t lo = ptr ? ptr[b] : 0;
    const int64_t hi = ptr ? ptr[b + 1] : m;
    const int len = (int)max((int64_t)0, hi - lo);
    run += (len + per_item - 1) / per_item;
  }
  if (tid == kPlanThreads - 1)
    work_start[num_segments] = partial[tid];
}

// Pointers of both sides from sorted example ids, by all waves of one
// workgroup: ptr[b] = number of rows whose id is below b.  A wave takes one
// (side, b) at a time and narrows the range 65-fold per step -- its 64 lanes
// probe evenly spaced rows at once, so a million rows take four dependent
// reads instead of twenty.  Src is launchers.hpp's SegmentSource.
template <typename Src>
__device__ __forceinline__ void pointers_from_ids(const Src &src,
                                                  int num_segments) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves = blockDim.x >> 6;
  const int searches = 2 * (num_segments + 1);
  // for a caller that guessed num_segments: the examples the ids speak of
  // (sorted ids: the last ones are the largest)
  if (src.examples_out != nullptr && threadIdx.x == 0) {
    int64_t last = -1;
    if (src.n > 0)
      last = src.ids_x[src.n - 1];
    if (src.m > 0 && src.ids_y[src.m - 1] > last)
      last = src.ids_y[src.m - 1];
    *src.examples_out = last + 1;
  }
  for (int s = wave; s < searches; s += waves) {
    const int side = s & 1;
    const int b = s >> 1;
    const int64_t *ids = side ? src.ids_y : src.ids_x;
    const int count = side ? src.m : src.n;
    // invariant: ids[i] < b for i < lo, ids[i] >= b for i >= hi
    int lo = 0, hi = count;
    while (hi - lo > 64) {
      const int64_t span = (int64_t)hi - lo;
      // probes lo + (l + 1) span / 65 - 1, l = 0 .. 63: inside [lo, hi),
      // ascending, distinct (span > 64)
      const int at = lo + (int)(span * (lane + 1) / 65) - 1;
      const uint64_t below = __ballot(ids[at] < (int64_t)b);
      // (sorted ids: the lanes that see an id below b are the first ones)
      const int first_not = __builtin_popcountll(below);
      const int new_lo =
          first_not == 0 ? lo : lo + (int)(span * first_not / 65);
      const int new_hi =
          first_not == 64 ? hi : lo + (int)(span * (first_not + 1) / 65) - 1;
      lo = new_lo;
      hi = new_hi;
    }
    const bool is_below = lo + lane < hi && ids[lo + lane] < (int64_t)b;
    int result = lo + __builtin_popcountll(__ballot(is_below));
    // Rows whose id is num_segments or more (a caller's batch_size below the
    // largest id + 1): the reference's lookup hands such a query to the LAST
    // example (csrc/cuda/utils.cuh:11-19 returns num_examples - 1 when no
    // pointer lies above the row), and never searches such a row of x.
    if (side == 1 && b == num_segments)
      result = count;
    if (lane == 0)
      (side ? src.ptr_y : src.ptr_x)[b] = result;
  }
}

} // namespace pca

// experiment switch: -DPCA_NO_SWIZZLE maps workgroup ids to tiles directly
#ifdef PCA_NO_SWIZZLE
#define PCA_TILE_OF_BLOCK(b, g) (b)
#else
#define PCA_TILE_OF_BLOCK(b, g) pca::xcd_swizzle(b, g)
#endif
