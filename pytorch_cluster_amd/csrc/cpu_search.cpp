// Host (CPU) implementation of the kNN and radius searches: what stands behind
// the operators for tensors that are not on a GPU, where the reference runs
// knn_cpu / radius_cpu (csrc/cpu/knn_cpu.cpp:7-105,
// csrc/cpu/radius_cpu.cpp:7-117, nanoflann k-d trees).
//
// Written from scratch, and with the result contract of the GPU kernels rather
// than nanoflann's: neighbours by ascending (distance, row) for kNN, the first
// max_num_neighbors rows in ascending row order for radius, distances
// accumulated with one fused multiply-add per component in ascending order
// (csrc/cuda/knn_cuda.cu:61-64 as a GPU compiler contracts it), candidates at
// distance >= 1e10 or NaN never returned.  A tensor therefore gets the same
// edges on either device.
//
// Points of up to 8 dimensions (fp32 / fp64) are searched through a k-d tree
// per segment (median splits along the widest axis, leaves of up to 16 rows,
// a bounding box per node).  A node is skipped only when the distance of the
// query to its box -- evaluated with the same operations in the same order as
// a row's distance, each of them monotone under rounding -- is not below the
// current bound, so pruning never changes a result.  Higher dimensions and the
// 16-bit types scan every row of the segment; fp32 / fp64 rows go through
// transposed tiles of 16 rows so that the per-component loop vectorises.
// Queries are dealt to `num_threads` host threads in blocks.
#include "../../include/pca_neighbors.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <limits>
#include <thread>
#include <utility>
#include <vector>

namespace {

thread_local char g_host_error[256] = "";

int host_fail(int status, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_host_error, sizeof(g_host_error), fmt, ap);
  va_end(ap);
  return status;
}

// ---- element types -----------------------------------------------------------

// fp16 / bf16 values are kept as floats that are exactly representable in the
// 16-bit type; every operator rounds its result back to that type, as
// c10::Half / c10::BFloat16 arithmetic does.
inline float round_bf16(float v) {
  uint32_t u;
  std::memcpy(&u, &v, 4);
  if ((u & 0x7f800000u) == 0x7f800000u)
    return v; // inf / NaN
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  std::memcpy(&v, &u, 4);
  return v;
}

inline float round_f16(float v) {
  if (!(std::fabs(v) < std::numeric_limits<float>::infinity()))
    return v;
  const float a = std::fabs(v);
  if (a >= 65520.0f) // rounds to infinity
    return std::copysign(std::numeric_limits<float>::infinity(), v);
  // spacing of fp16 at this magnitude: 2^(e - 10), not below 2^-24
  int e;
  std::frexp(a, &e); // a = f * 2^e, f in [0.5, 1)
  const int ulp_exp = std::max(e - 1, -14) - 10;
  const float ulp = std::ldexp(1.0f, ulp_exp);
  // nearest even multiple of ulp (the division and product are exact)
  const float r = std::nearbyint(a / ulp) * ulp;
  return std::copysign(r, v);
}

inline float from_f16_bits(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const int exp = (h >> 10) & 31;
  const uint32_t man = h & 0x3ffu;
  float v;
  if (exp == 0)
    v = std::ldexp((float)man, -24);
  else if (exp == 31)
    v = man ? std::numeric_limits<float>::quiet_NaN()
            : std::numeric_limits<float>::infinity();
  else
    v = std::ldexp((float)(man | 0x400u), exp - 25);
  uint32_t u;
  std::memcpy(&u, &v, 4);
  u |= sign;
  std::memcpy(&v, &u, 4);
  return v;
}

inline float from_bf16_bits(uint16_t h) {
  const uint32_t u = (uint32_t)h << 16;
  float v;
  std::memcpy(&v, &u, 4);
  return v;
}

// Arithmetic of a distance in element type T: `Acc` holds values, step() adds
// one component.
template <typename T> struct Exact {
  typedef T value;
  static inline T step(T a, T b, T acc) {
    const T diff = a - b;
    return std::fma(diff, diff, acc);
  }
  static constexpr bool tree = true;
  static inline T limit() { return (T)1e10; }
};
struct Half16 {
  typedef float value;
  static inline float step(float a, float b, float acc) {
    const float diff = round_f16(a - b);
    return round_f16(acc + round_f16(diff * diff));
  }
  static constexpr bool tree = false;
  // (1e10 narrows to +inf in fp16)
  static inline float limit() { return std::numeric_limits<float>::infinity(); }
  static inline float narrow(double v) { return round_f16((float)v); }
};
struct Bf16 {
  typedef float value;
  static inline float step(float a, float b, float acc) {
    const float diff = round_bf16(a - b);
    return round_bf16(acc + round_bf16(diff * diff));
  }
  static constexpr bool tree = false;
  static inline float limit() { return round_bf16(1e10f); }
  static inline float narrow(double v) { return round_bf16((float)v); }
};

template <typename A>
inline typename A::value distance(const typename A::value *a,
                                  const typename A::value *b, int d) {
  typename A::value acc = 0;
  for (int c = 0; c < d; ++c)
    acc = A::step(a[c], b[c], acc);
  return acc;
}

// ---- the two selections -------------------------------------------------------

// k smallest (distance, row) pairs, as a max-heap while the search runs.
template <typename V> struct KnnList {
  typedef std::pair<V, int64_t> entry;
  std::vector<entry> heap;
  size_t k;
  V limit; // distances must stay below it (the sentinel, narrowed to V)
  explicit KnnList(size_t k_, V limit_) : k(k_), limit(limit_) {
    heap.reserve(k_);
  }
  void clear() { heap.clear(); }
  // rows whose box distance is above this cannot enter any more
  V bound() const { return heap.size() < k ? limit : heap.front().first; }
  bool full() const { return heap.size() >= k; }
  void offer(V dist, int64_t row) {
    if (!(dist < limit)) // also NaN
      return;
    const entry e(dist, row);
    if (heap.size() < k) {
      heap.push_back(e);
      std::push_heap(heap.begin(), heap.end());
    } else if (e < heap.front()) {
      std::pop_heap(heap.begin(), heap.end());
      heap.back() = e;
      std::push_heap(heap.begin(), heap.end());
    }
  }
  // ascending (distance, row)
  void finish() { std::sort_heap(heap.begin(), heap.end()); }
};

// The `cap` smallest row numbers among the rows in range, as a max-heap.
struct RadiusList {
  std::vector<int64_t> heap;
  size_t cap;
  explicit RadiusList(size_t cap_) : cap(cap_) { heap.reserve(cap_); }
  void clear() { heap.clear(); }
  bool full() const { return heap.size() >= cap; }
  // rows numbered at or above this cannot enter any more
  int64_t row_bound() const {
    return full() ? heap.front() : std::numeric_limits<int64_t>::max();
  }
  void offer(int64_t row) {
    if (heap.size() < cap) {
      heap.push_back(row);
      std::push_heap(heap.begin(), heap.end());
    } else if (row < heap.front()) {
      std::pop_heap(heap.begin(), heap.end());
      heap.back() = row;
      std::push_heap(heap.begin(), heap.end());
    }
  }
  void finish() { std::sort_heap(heap.begin(), heap.end()); }
};

// ---- k-d tree over the finite rows of one segment ------------------------------

constexpr int kMaxTreeDim = 8;
constexpr int kLeafRows = 16;

template <typename T> struct KdTree {
  struct Node {
    int begin, end;   // rows order[begin .. end)
    int left, right;  // children, -1 for a leaf
    int64_t min_row;  // smallest row number below this node
    T lo[kMaxTreeDim], hi[kMaxTreeDim];
  };
  const T *x = nullptr;
  int d = 0;
  std::vector<int64_t> order; // global row numbers
  std::vector<Node> nodes;

  void build(const T *x_, int d_, int64_t row_begin, int64_t row_end) {
    x = x_;
    d = d_;
    order.clear();
    nodes.clear();
    for (int64_t r = row_begin; r < row_end; ++r) {
      bool finite = true;
      for (int c = 0; c < d; ++c)
        finite = finite && std::isfinite(x[r * d + c]);
      // (a row with an infinite or NaN coordinate has no distance below any
      // limit: leaving it out changes nothing)
      if (finite)
        order.push_back(r);
    }
    if (!order.empty()) {
      nodes.reserve(2 * order.size() / kLeafRows + 2);
      split(0, (int)order.size());
    }
  }

  int split(int begin, int end) {
    const int id = (int)nodes.size();
    nodes.emplace_back();
    {
      Node &n = nodes[id];
      n.begin = begin;
      n.end = end;
      n.left = n.right = -1;
      n.min_row = std::numeric_limits<int64_t>::max();
      for (int c = 0; c < d; ++c) {
        n.lo[c] = std::numeric_limits<T>::infinity();
        n.hi[c] = -std::numeric_limits<T>::infinity();
      }
      for (int i = begin; i < end; ++i) {
        const int64_t r = order[i];
        n.min_row = std::min(n.min_row, r);
        for (int c = 0; c < d; ++c) {
          n.lo[c] = std::min(n.lo[c], x[r * d + c]);
          n.hi[c] = std::max(n.hi[c], x[r * d + c]);
        }
      }
    }
    if (end - begin > kLeafRows) {
      int axis = 0;
      T widest = -1;
      for (int c = 0; c < d; ++c) {
        const T w = nodes[id].hi[c] - nodes[id].lo[c];
        if (w > widest) {
          widest = w;
          axis = c;
        }
      }
      if (widest > 0) {
        const int mid = begin + (end - begin) / 2;
        const T *xs = x;
        const int dd = d;
        std::nth_element(order.begin() + begin, order.begin() + mid,
                         order.begin() + end,
                         [xs, dd, axis](int64_t a, int64_t b) {
                           return xs[a * dd + axis] < xs[b * dd + axis];
                         });
        const int l = split(begin, mid);
        const int r = split(mid, end);
        nodes[id].left = l;
        nodes[id].right = r;
      }
    }
    return id;
  }

  // Distance of q to the node's box with a row distance's own operations:
  // never above the computed distance of any row inside.
  T box_distance(const Node &n, const T *q) const {
    T acc = 0;
    for (int c = 0; c < d; ++c) {
      const T gap = std::max(std::max(n.lo[c] - q[c], q[c] - n.hi[c]), (T)0);
      acc = std::fma(gap, gap, acc);
    }
    return acc;
  }

  void knn(const T *q, KnnList<T> &list) const {
    if (nodes.empty())
      return;
    // (node, box distance) still to visit, nearer child on top
    std::pair<int, T> stack[128];
    int top = 0;
    stack[top++] = std::make_pair(0, box_distance(nodes[0], q));
    while (top > 0) {
      const std::pair<int, T> item = stack[--top];
      // equal distances still compete through their row numbers
      if (item.second > list.bound() || !(item.second < list.limit))
        continue;
      const Node &n = nodes[item.first];
      if (n.left < 0) {
        for (int i = n.begin; i < n.end; ++i) {
          const int64_t r = order[i];
          list.offer(distance<Exact<T>>(x + r * d, q, d), r);
        }
        continue;
      }
      const T dl = box_distance(nodes[n.left], q);
      const T dr = box_distance(nodes[n.right], q);
      if (dl <= dr) {
        stack[top++] = std::make_pair(n.right, dr);
        stack[top++] = std::make_pair(n.left, dl);
      } else {
        stack[top++] = std::make_pair(n.left, dl);
        stack[top++] = std::make_pair(n.right, dr);
      }
    }
  }

  void radius(const T *q, T r2, int64_t skip_row, RadiusList &list) const {
    if (nodes.empty())
      return;
    int stack[128];
    int top = 0;
    stack[top++] = 0;
    while (top > 0) {
      const Node &n = nodes[stack[--top]];
      if (n.min_row >= list.row_bound() || !(box_distance(n, q) < r2))
        continue;
      if (n.left < 0) {
        for (int i = n.begin; i < n.end; ++i) {
          const int64_t r = order[i];
          if (r != skip_row && distance<Exact<T>>(x + r * d, q, d) < r2)
            list.offer(r);
        }
        continue;
      }
      stack[top++] = n.right;
      stack[top++] = n.left;
    }
  }
};

// ---- scans of every row of a segment --------------------------------------------

constexpr int kTileRows = 16;

// Distances of one query to kTileRows rows held component-major.
template <typename T>
inline void tile_distances(const T *tile, const T *q, int d, T *out) {
  T acc[kTileRows];
  for (int j = 0; j < kTileRows; ++j)
    acc[j] = 0;
  for (int c = 0; c < d; ++c) {
    const T qc = q[c];
    const T *col = tile + (size_t)c * kTileRows;
    for (int j = 0; j < kTileRows; ++j) {
      const T diff = col[j] - qc;
      acc[j] = std::fma(diff, diff, acc[j]);
    }
  }
  for (int j = 0; j < kTileRows; ++j)
    out[j] = acc[j];
}

// ---- the search of one block of queries ------------------------------------------

struct Problem {
  const void *x, *y;
  const int64_t *ptr_x, *ptr_y;
  int64_t n, m, d, num_segments;
  int dtype;
  // kNN
  int64_t k;
  // radius
  bool is_radius;
  double r;
  int64_t cap;
  bool ignore_same_index;
  // results: rows per query, then their count
  int64_t slots;
  int64_t *rows; // [m, slots]
  void *dist;    // [m, slots] element type (kNN only, may be NULL)
  int64_t *count;
};

// Rows of segment [xb, xe) for the queries [qb, qe) of the same segment.
template <typename A, typename Load>
void scan_block(const Problem &p, Load load, int64_t xb, int64_t xe,
                int64_t qb, int64_t qe) {
  typedef typename A::value V;
  const int d = (int)p.d;
  std::vector<V> qrow(d), xrow(d);
  KnnList<V> knn((size_t)std::max<int64_t>(p.k, 1), A::limit());
  RadiusList rad((size_t)std::max<int64_t>(p.cap, 1));
  const V r2 = A::narrow(p.r * p.r);
  for (int64_t q = qb; q < qe; ++q) {
    for (int c = 0; c < d; ++c)
      qrow[c] = load(p.y, q * d + c);
    int64_t found = 0;
    if (p.is_radius) {
      rad.clear();
      for (int64_t r = xb; r < xe && !rad.full(); ++r) {
        if (p.ignore_same_index && r == q)
          continue;
        for (int c = 0; c < d; ++c)
          xrow[c] = load(p.x, r * d + c);
        if (distance<A>(xrow.data(), qrow.data(), d) < r2)
          rad.offer(r);
      }
      rad.finish();
      for (int64_t row : rad.heap)
        p.rows[q * p.slots + found++] = row;
    } else {
      knn.clear();
      for (int64_t r = xb; r < xe; ++r) {
        for (int c = 0; c < d; ++c)
          xrow[c] = load(p.x, r * d + c);
        knn.offer(distance<A>(xrow.data(), qrow.data(), d), r);
      }
      knn.finish();
      for (const auto &e : knn.heap) {
        p.rows[q * p.slots + found] = e.second;
        if (p.dist)
          static_cast<V *>(p.dist)[q * p.slots + found] = e.first;
        ++found;
      }
    }
    p.count[q] = found;
  }
}

// fp32 / fp64 rows of any dimension through transposed tiles.
template <typename T>
void tiled_block(const Problem &p, int64_t xb, int64_t xe, int64_t qb,
                 int64_t qe) {
  const int d = (int)p.d;
  const T *x = static_cast<const T *>(p.x);
  const T *y = static_cast<const T *>(p.y);
  const int64_t nq = qe - qb;
  std::vector<KnnList<T>> knn;
  std::vector<RadiusList> rad;
  for (int64_t i = 0; i < nq; ++i) {
    if (p.is_radius)
      rad.emplace_back((size_t)p.cap);
    else
      knn.emplace_back((size_t)p.k, (T)1e10);
  }
  const T r2 = (T)(p.r * p.r);
  std::vector<T> tile((size_t)d * kTileRows);
  T dist[kTileRows];
  for (int64_t base = xb; base < xe; base += kTileRows) {
    const int rows = (int)std::min<int64_t>(kTileRows, xe - base);
    for (int j = 0; j < kTileRows; ++j) {
      const int64_t r = base + std::min(j, rows - 1);
      for (int c = 0; c < d; ++c)
        tile[(size_t)c * kTileRows + j] = x[r * d + c];
    }
    for (int64_t i = 0; i < nq; ++i) {
      const int64_t q = qb + i;
      if (p.is_radius && rad[i].full())
        continue; // rows arrive in ascending order: nothing can enter
      tile_distances<T>(tile.data(), y + q * d, d, dist);
      for (int j = 0; j < rows; ++j) {
        const int64_t r = base + j;
        if (p.is_radius) {
          if (dist[j] < r2 && !(p.ignore_same_index && r == q) &&
              !rad[i].full())
            rad[i].offer(r);
        } else {
          knn[i].offer(dist[j], r);
        }
      }
    }
  }
  for (int64_t i = 0; i < nq; ++i) {
    const int64_t q = qb + i;
    int64_t found = 0;
    if (p.is_radius) {
      rad[i].finish();
      for (int64_t row : rad[i].heap)
        p.rows[q * p.slots + found++] = row;
    } else {
      knn[i].finish();
      for (const auto &e : knn[i].heap) {
        p.rows[q * p.slots + found] = e.second;
        if (p.dist)
          static_cast<T *>(p.dist)[q * p.slots + found] = e.first;
        ++found;
      }
    }
    p.count[q] = found;
  }
}

template <typename T>
void tree_block(const Problem &p, const KdTree<T> &tree, int64_t qb,
                int64_t qe) {
  const int d = (int)p.d;
  const T *y = static_cast<const T *>(p.y);
  KnnList<T> knn((size_t)std::max<int64_t>(p.k, 1), (T)1e10);
  RadiusList rad((size_t)std::max<int64_t>(p.cap, 1));
  const T r2 = (T)(p.r * p.r);
  for (int64_t q = qb; q < qe; ++q) {
    int64_t found = 0;
    if (p.is_radius) {
      rad.clear();
      tree.radius(y + q * d, r2, p.ignore_same_index ? q : -1, rad);
      rad.finish();
      for (int64_t row : rad.heap)
        p.rows[q * p.slots + found++] = row;
    } else {
      knn.clear();
      tree.knn(y + q * d, knn);
      knn.finish();
      for (const auto &e : knn.heap) {
        p.rows[q * p.slots + found] = e.second;
        if (p.dist)
          static_cast<T *>(p.dist)[q * p.slots + found] = e.first;
        ++found;
      }
    }
    p.count[q] = found;
  }
}

// ---- threads ------------------------------------------------------------------

template <typename F> void parallel_blocks(int64_t blocks, int threads, F fn) {
  threads = (int)std::max<int64_t>(1, std::min<int64_t>(threads, blocks));
  if (threads == 1) {
    for (int64_t b = 0; b < blocks; ++b)
      fn(b);
    return;
  }
  std::atomic<int64_t> next(0);
  std::vector<std::thread> pool;
  for (int t = 0; t < threads; ++t)
    pool.emplace_back([&]() {
      for (;;) {
        const int64_t b = next.fetch_add(1);
        if (b >= blocks)
          return;
        fn(b);
      }
    });
  for (auto &t : pool)
    t.join();
}

struct Block {
  int64_t seg, qb, qe;
};

template <typename T> void search_real(const Problem &p, int threads) {
  const bool use_tree = p.d <= kMaxTreeDim;
  std::vector<KdTree<T>> trees;
  auto seg_begin = [&](const int64_t *ptr, int64_t b, int64_t total) {
    return ptr ? ptr[b] : (b == 0 ? 0 : total);
  };
  const int64_t nseg = p.num_segments;
  if (use_tree) {
    trees.resize(nseg);
    parallel_blocks(nseg, threads, [&](int64_t b) {
      const int64_t xb = seg_begin(p.ptr_x, b, p.n);
      const int64_t xe = seg_begin(p.ptr_x, b + 1, p.n);
      const int64_t qb = seg_begin(p.ptr_y, b, p.m);
      const int64_t qe = seg_begin(p.ptr_y, b + 1, p.m);
      if (xe > xb && qe > qb)
        trees[b].build(static_cast<const T *>(p.x), (int)p.d, xb, xe);
    });
  }
  const int64_t per_block = use_tree ? 256 : 32;
  std::vector<Block> blocks;
  for (int64_t b = 0; b < nseg; ++b) {
    const int64_t qb = seg_begin(p.ptr_y, b, p.m);
    const int64_t qe = seg_begin(p.ptr_y, b + 1, p.m);
    for (int64_t q = qb; q < qe; q += per_block)
      blocks.push_back({b, q, std::min(q + per_block, qe)});
  }
  parallel_blocks((int64_t)blocks.size(), threads, [&](int64_t i) {
    const Block &blk = blocks[i];
    if (use_tree) {
      tree_block<T>(p, trees[blk.seg], blk.qb, blk.qe);
    } else {
      tiled_block<T>(p, seg_begin(p.ptr_x, blk.seg, p.n),
                     seg_begin(p.ptr_x, blk.seg + 1, p.n), blk.qb, blk.qe);
    }
  });
}

template <typename A, typename Load>
void search_16bit(const Problem &p, int threads, Load load) {
  auto seg_begin = [&](const int64_t *ptr, int64_t b, int64_t total) {
    return ptr ? ptr[b] : (b == 0 ? 0 : total);
  };
  std::vector<Block> blocks;
  for (int64_t b = 0; b < p.num_segments; ++b) {
    const int64_t qb = seg_begin(p.ptr_y, b, p.m);
    const int64_t qe = seg_begin(p.ptr_y, b + 1, p.m);
    for (int64_t q = qb; q < qe; q += 64)
      blocks.push_back({b, q, std::min<int64_t>(q + 64, qe)});
  }
  parallel_blocks((int64_t)blocks.size(), threads, [&](int64_t i) {
    const Block &blk = blocks[i];
    scan_block<A>(p, load, seg_begin(p.ptr_x, blk.seg, p.n),
                  seg_begin(p.ptr_x, blk.seg + 1, p.n), blk.qb, blk.qe);
  });
}

// fp16 distances above the fp16 range are +inf, and the sentinel 1e10 narrows
// to +inf as well: `dist < limit` then keeps every finite distance, as the
// reference's comparison in c10::Half does.
int run(Problem &p, int edge_flags, int threads, int64_t *edges,
        int64_t *num_edges, void *dist_out) {
  // distances per slot first, in edge order at the end
  const size_t elem = p.dtype == PCA_F64 ? 8 : 4;
  std::vector<char> dense_dist;
  if (dist_out) {
    dense_dist.resize((size_t)p.m * (size_t)p.slots * elem);
    p.dist = dense_dist.data();
  }
  std::vector<int64_t> rows((size_t)p.m * (size_t)p.slots);
  std::vector<int64_t> count((size_t)p.m, 0);
  p.rows = rows.data();
  p.count = count.data();
  switch (p.dtype) {
  case PCA_F32:
    search_real<float>(p, threads);
    break;
  case PCA_F64:
    search_real<double>(p, threads);
    break;
  case PCA_F16:
    search_16bit<Half16>(p, threads, [](const void *base, int64_t i) {
      return from_f16_bits(static_cast<const uint16_t *>(base)[i]);
    });
    break;
  case PCA_BF16:
    search_16bit<Bf16>(p, threads, [](const void *base, int64_t i) {
      return from_bf16_bits(static_cast<const uint16_t *>(base)[i]);
    });
    break;
  default:
    return host_fail(PCA_ERR_UNSUPPORTED, "element type %d is not built",
                     p.dtype);
  }
  // [2, E]: query rows, then x rows (or the other way round), without the
  // pairs of a row with itself when asked to
  const bool drop_self = (edge_flags & PCA_EDGES_DROP_SELF) != 0;
  const bool x_first = (edge_flags & PCA_EDGES_X_FIRST) != 0;
  std::vector<int64_t> start((size_t)p.m + 1, 0);
  for (int64_t q = 0; q < p.m; ++q) {
    int64_t kept = count[q];
    if (drop_self)
      for (int64_t e = 0; e < count[q]; ++e)
        if (rows[q * p.slots + e] == q)
          --kept;
    start[q + 1] = start[q] + kept;
  }
  const int64_t total = start[p.m];
  *num_edges = total;
  int64_t *first = edges, *second = edges + total;
  const int64_t chunk = 4096;
  parallel_blocks((p.m + chunk - 1) / chunk, threads, [&](int64_t b) {
    for (int64_t q = b * chunk; q < std::min(p.m, (b + 1) * chunk); ++q) {
      int64_t at = start[q];
      for (int64_t e = 0; e < count[q]; ++e) {
        const int64_t r = rows[q * p.slots + e];
        if (drop_self && r == q)
          continue;
        (x_first ? second : first)[at] = q;
        (x_first ? first : second)[at] = r;
        if (dist_out)
          std::memcpy(static_cast<char *>(dist_out) + (size_t)at * elem,
                      dense_dist.data() + ((size_t)q * p.slots + e) * elem,
                      elem);
        ++at;
      }
    }
  });
  return PCA_OK;
}

bool host_sizes_ok(int64_t n, int64_t m, int64_t d, int64_t num_segments) {
  return n >= 0 && m >= 0 && d >= 1 && num_segments >= 1;
}

// ---- fps and nearest on the host ---------------------------------------------
// Both follow the result contract of the GPU operators (which is the one of
// the reference's CUDA kernels), so that CPU and GPU tensors give the same
// rows.

// Farthest point sampling of one example (csrc/cuda/fps_cuda.cu:10-66 is the
// contract: running minima that start at 5e4, the next sample is the row with
// the largest one, among equal ones the smallest (row - start) % 256, then the
// smallest row; global row 0 when no row has a value).
template <typename T>
void fps_example(const T *src, int64_t d, int64_t begin, int64_t end,
                 int64_t first, int64_t out_begin, int64_t out_end,
                 int64_t *out) {
  if (out_begin >= out_end)
    return;
  const int64_t rows = end - begin;
  std::vector<T> nearest_sample((size_t)std::max<int64_t>(rows, 1), (T)5e4);
  int64_t current = begin + first;
  out[out_begin] = current;
  for (int64_t s = out_begin + 1; s < out_end; ++s) {
    const T *centre = src + current * d;
    T best = (T)-1;
    int64_t best_row = 0, best_slot = 0;
    bool found = false;
    for (int64_t i = 0; i < rows; ++i) {
      const T *row = src + (begin + i) * d;
      T acc = 0;
      for (int64_t c = 0; c < d; ++c) {
        const T diff = row[c] - centre[c];
        acc = std::fma(diff, diff, acc);
      }
      // (a NaN distance leaves the minimum as it is)
      T v = nearest_sample[(size_t)i];
      v = acc < v ? acc : v;
      nearest_sample[(size_t)i] = v;
      const int64_t slot = i & 255;
      // larger value; equal value: the smaller slot, then the smaller row
      // (rows are visited in ascending order)
      if (v > best || (found && v == best && slot < best_slot)) {
        best = v;
        best_row = begin + i;
        best_slot = slot;
        found = true;
      }
    }
    current = found ? best_row : 0;
    out[s] = current;
  }
}

// The nearest row of y for one row of x (csrc/cuda/nearest_cuda.cu:10-66 is
// the contract: strictly below 1e38, among equal distances the smallest
// (row - start) % 1024, then the smallest row; 0 when nothing qualifies).
template <typename T>
int64_t nearest_row(const T *xrow, const T *y, int64_t d, int64_t begin,
                    int64_t end) {
  const T limit = (T)1e38f;
  T best = limit;
  int64_t best_row = 0, best_slot = 0;
  bool found = false;
  for (int64_t j = begin; j < end; ++j) {
    const T *row = y + j * d;
    T acc = 0;
    for (int64_t c = 0; c < d; ++c) {
      const T diff = xrow[c] - row[c];
      acc = std::fma(diff, diff, acc);
    }
    const int64_t slot = (j - begin) & 1023;
    if (acc < best || (found && acc == best && slot < best_slot)) {
      if (!(acc < limit))
        continue;
      best = acc;
      best_row = j;
      best_slot = slot;
      found = true;
    }
  }
  return found ? best_row : 0;
}

bool host_cpu_ok() {
  return __builtin_cpu_supports("fma") && __builtin_cpu_supports("avx2");
}

} // namespace

extern "C" {

const char *pca_host_last_error(void) { return g_host_error; }

int pca_knn_host(const void *x, const void *y, const int64_t *ptr_x,
                 const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                 int64_t num_segments, int64_t k, int dtype, int edge_flags,
                 int num_threads, int64_t *edges, int64_t *num_edges,
                 void *dist) {
  g_host_error[0] = 0;
  if (!host_cpu_ok())
    return host_fail(PCA_ERR_NO_DEVICE,
                     "this build needs a CPU with AVX2 and FMA");
  if ((ptr_x == nullptr) != (ptr_y == nullptr))
    return host_fail(PCA_ERR_INVALID_ARGUMENT,
                     "ptr_x and ptr_y must both be given or both be NULL");
  if (ptr_x == nullptr)
    num_segments = 1;
  if (!host_sizes_ok(n, m, d, num_segments) || k < 1 || num_edges == nullptr)
    return host_fail(PCA_ERR_INVALID_ARGUMENT, "bad sizes or NULL num_edges");
  if (n == 0 || m == 0) {
    *num_edges = 0;
    return PCA_OK;
  }
  if (x == nullptr || y == nullptr || edges == nullptr)
    return host_fail(PCA_ERR_INVALID_ARGUMENT, "x, y or edges is NULL");
  if (dist != nullptr && dtype != PCA_F32 && dtype != PCA_F64)
    return host_fail(PCA_ERR_UNSUPPORTED,
                     "per-edge distances are returned for fp32 / fp64 only");
  Problem p{};
  p.x = x, p.y = y, p.ptr_x = ptr_x, p.ptr_y = ptr_y;
  p.n = n, p.m = m, p.d = d, p.num_segments = num_segments;
  p.dtype = dtype;
  p.k = k;
  p.is_radius = false;
  p.slots = std::min(k, n);
  p.k = p.slots;
  return run(p, edge_flags, num_threads, edges, num_edges, dist);
}

int pca_radius_host(const void *x, const void *y, const int64_t *ptr_x,
                    const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                    int64_t num_segments, double r, int64_t max_num_neighbors,
                    int ignore_same_index, int dtype, int edge_flags,
                    int num_threads, int64_t *edges, int64_t *num_edges) {
  g_host_error[0] = 0;
  if (!host_cpu_ok())
    return host_fail(PCA_ERR_NO_DEVICE,
                     "this build needs a CPU with AVX2 and FMA");
  if ((ptr_x == nullptr) != (ptr_y == nullptr))
    return host_fail(PCA_ERR_INVALID_ARGUMENT,
                     "ptr_x and ptr_y must both be given or both be NULL");
  if (ptr_x == nullptr)
    num_segments = 1;
  if (!host_sizes_ok(n, m, d, num_segments) || max_num_neighbors < 1 ||
      num_edges == nullptr)
    return host_fail(PCA_ERR_INVALID_ARGUMENT, "bad sizes or NULL num_edges");
  if (n == 0 || m == 0) {
    *num_edges = 0;
    return PCA_OK;
  }
  if (x == nullptr || y == nullptr || edges == nullptr)
    return host_fail(PCA_ERR_INVALID_ARGUMENT, "x, y or edges is NULL");
  Problem p{};
  p.x = x, p.y = y, p.ptr_x = ptr_x, p.ptr_y = ptr_y;
  p.n = n, p.m = m, p.d = d, p.num_segments = num_segments;
  p.dtype = dtype;
  p.is_radius = true;
  p.r = r;
  p.cap = std::min(max_num_neighbors, n);
  p.slots = p.cap;
  p.ignore_same_index = ignore_same_index != 0;
  p.dist = nullptr;
  return run(p, edge_flags, num_threads, edges, num_edges, nullptr);
}

int pca_fps_host(const void *src, const int64_t *ptr, const int64_t *out_ptr,
                 const int64_t *start, int64_t n, int64_t d,
                 int64_t num_segments, int dtype, int num_threads,
                 int64_t *out) {
  g_host_error[0] = 0;
  if (n < 0 || d < 1 || num_segments < 1 || ptr == nullptr ||
      out_ptr == nullptr)
    return host_fail(PCA_ERR_INVALID_ARGUMENT, "bad sizes or NULL pointers");
  if (dtype != PCA_F32 && dtype != PCA_F64)
    return host_fail(PCA_ERR_UNSUPPORTED,
                     "fps on the host takes fp32 and fp64 points");
  if (n == 0)
    return PCA_OK;
  if (src == nullptr || out == nullptr)
    return host_fail(PCA_ERR_INVALID_ARGUMENT, "src or out is NULL");
  parallel_blocks(num_segments, std::max(num_threads, 1), [&](int64_t b) {
    const int64_t first = start ? start[b] : 0;
    if (dtype == PCA_F32)
      fps_example(static_cast<const float *>(src), d, ptr[b], ptr[b + 1],
                  first, out_ptr[b], out_ptr[b + 1], out);
    else
      fps_example(static_cast<const double *>(src), d, ptr[b], ptr[b + 1],
                  first, out_ptr[b], out_ptr[b + 1], out);
  });
  return PCA_OK;
}

int pca_nearest_host(const void *x, const void *y, const int64_t *ptr_x,
                     const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                     int64_t num_segments, int dtype, int num_threads,
                     int64_t *out) {
  g_host_error[0] = 0;
  if (n < 0 || m < 0 || d < 1 || num_segments < 1 || ptr_x == nullptr ||
      ptr_y == nullptr)
    return host_fail(PCA_ERR_INVALID_ARGUMENT, "bad sizes or NULL pointers");
  if (dtype != PCA_F32 && dtype != PCA_F64)
    return host_fail(PCA_ERR_UNSUPPORTED,
                     "nearest on the host takes fp32 and fp64 points");
  if (n == 0)
    return PCA_OK;
  if (x == nullptr || out == nullptr || (m > 0 && y == nullptr))
    return host_fail(PCA_ERR_INVALID_ARGUMENT, "x, y or out is NULL");
  // blocks of 256 searching rows, each inside one segment
  struct Piece {
    int64_t seg, begin, end;
  };
  std::vector<Piece> pieces;
  for (int64_t b = 0; b < num_segments; ++b)
    for (int64_t r = ptr_x[b]; r < ptr_x[b + 1]; r += 256)
      pieces.push_back({b, r, std::min(r + 256, ptr_x[b + 1])});
  // (rows behind the last pointer: the reference's lookup gives them the
  // last example, csrc/cuda/utils.cuh:11-19)
  for (int64_t r = ptr_x[num_segments]; r < n; r += 256)
    pieces.push_back({num_segments - 1, r, std::min(r + 256, n)});
  parallel_blocks((int64_t)pieces.size(), std::max(num_threads, 1),
                  [&](int64_t i) {
                    const Piece &pc = pieces[(size_t)i];
                    for (int64_t r = pc.begin; r < pc.end; ++r) {
                      if (dtype == PCA_F32)
                        out[r] = nearest_row(
                            static_cast<const float *>(x) + r * d,
                            static_cast<const float *>(y), d, ptr_y[pc.seg],
                            ptr_y[pc.seg + 1]);
                      else
                        out[r] = nearest_row(
                            static_cast<const double *>(x) + r * d,
                            static_cast<const double *>(y), d, ptr_y[pc.seg],
                            ptr_y[pc.seg + 1]);
                    }
                  });
  return PCA_OK;
}

} // extern "C"
