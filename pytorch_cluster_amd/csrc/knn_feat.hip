// Dispatch of the feature-space kNN with the fp16 matrix-core filter (see
// knn_feat_impl.hpp): preparation, the filter kernel, the exact second kernel
// and the second pass for the queries that one flags.
#include "knn_feat_small_impl.hpp"
#include "knn_feat_wide_impl.hpp"

#include <algorithm>
#include <cstdlib>

namespace pca {

#define PCA_DECLARE_FEAT_BLOCKS(NB)                                            \
  template <>                                                                  \
  hipError_t launch_knn_feat_blocks<NB>(const KnnFeatParams &, int, bool,      \
                                        int, hipStream_t);                     \
  template <>                                                                  \
  hipError_t launch_feat_pack<NB>(const float *, const float *,                \
                                  const float *, const unsigned *, int, int,   \
                                  bool, FeatGlobals *, uint4 *, hipStream_t);
PCA_DECLARE_FEAT_BLOCKS(3)
PCA_DECLARE_FEAT_BLOCKS(5)
PCA_DECLARE_FEAT_BLOCKS(9)
PCA_DECLARE_FEAT_BLOCKS(17)
PCA_DECLARE_FEAT_BLOCKS(33)
#undef PCA_DECLARE_FEAT_BLOCKS

#define PCA_DECLARE_FEAT_WIDE_BLOCKS(NB)                                       \
  template <>                                                                  \
  hipError_t launch_knn_feat_wide_blocks<NB>(const KnnFeatWideParams &, int,   \
                                             bool, int, hipStream_t);
PCA_DECLARE_FEAT_WIDE_BLOCKS(3)
PCA_DECLARE_FEAT_WIDE_BLOCKS(5)
PCA_DECLARE_FEAT_WIDE_BLOCKS(9)
#undef PCA_DECLARE_FEAT_WIDE_BLOCKS

#define PCA_DECLARE_FEAT_SMALL_BLOCKS(NB, R16)                                 \
  template <>                                                                  \
  hipError_t launch_knn_feat_small_blocks<NB, R16>(const KnnFeatParams &, int, \
                                                   int, hipStream_t);
PCA_DECLARE_FEAT_SMALL_BLOCKS(3, 0)
PCA_DECLARE_FEAT_SMALL_BLOCKS(5, 0)
PCA_DECLARE_FEAT_SMALL_BLOCKS(9, 0)
PCA_DECLARE_FEAT_SMALL_BLOCKS(3, 1)
PCA_DECLARE_FEAT_SMALL_BLOCKS(5, 1)
PCA_DECLARE_FEAT_SMALL_BLOCKS(9, 1)
PCA_DECLARE_FEAT_SMALL_BLOCKS(3, 2)
PCA_DECLARE_FEAT_SMALL_BLOCKS(5, 2)
PCA_DECLARE_FEAT_SMALL_BLOCKS(9, 2)
PCA_DECLARE_FEAT_SMALL_BLOCKS(3, 3)
PCA_DECLARE_FEAT_SMALL_BLOCKS(5, 3)
PCA_DECLARE_FEAT_SMALL_BLOCKS(9, 3)
#undef PCA_DECLARE_FEAT_SMALL_BLOCKS

#define PCA_DECLARE_RADIUS_FEAT_BLOCKS(NB, R16)                                \
  template <>                                                                  \
  hipError_t launch_radius_feat_blocks<NB, R16>(const KnnFeatParams &, int,    \
                                                int, hipStream_t);
PCA_DECLARE_RADIUS_FEAT_BLOCKS(3, 0)
PCA_DECLARE_RADIUS_FEAT_BLOCKS(5, 0)
PCA_DECLARE_RADIUS_FEAT_BLOCKS(9, 0)
PCA_DECLARE_RADIUS_FEAT_BLOCKS(3, 1)
PCA_DECLARE_RADIUS_FEAT_BLOCKS(5, 1)
PCA_DECLARE_RADIUS_FEAT_BLOCKS(9, 1)
PCA_DECLARE_RADIUS_FEAT_BLOCKS(3, 2)
PCA_DECLARE_RADIUS_FEAT_BLOCKS(5, 2)
PCA_DECLARE_RADIUS_FEAT_BLOCKS(9, 2)
#undef PCA_DECLARE_RADIUS_FEAT_BLOCKS

namespace {

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// The one-kernel search (knn_feat_small_impl.hpp): up to 128 components,
// k <= 48, examples of moderate length.  A workgroup of that
// kernel (128 queries) goes over its whole example, twice, with a compute unit
// to itself and one wave per SIMD; the staged searches share an example among
// workgroups and keep the matrix cores busier, but a call of theirs is a
// dozen launches and every piece of a scan starts its lists cold.  Measured on
// clouds searched in themselves, k = 20, one kernel / the better staged
// search, whole calls in ms:
//   32 x 1,024 x 64   0.22 / 0.51     256 x 1,024 x 64   1.29 / 2.00
//   64 x 2,048 x 64   0.93 / 1.20     128 x 2,048 x 64   1.79 / 2.23
//   8 x 4,096 x 64    0.39 / 0.62     64 x 4,096 x 64    2.57 / 2.51
//   32 x 4,096 x 128  2.07 / 1.83     4 x 8,192 x 64     0.52 / 0.77
//   8 x 8,192 x 128   1.73 / 1.62     16 x 8,192 x 32    1.33 / 1.01
//   2 x 16,384 x 64   0.77 / 0.91     4 x 16,384 x 128   2.17 / 1.62
//   1 x 32,768 x 64   1.19 / 1.12     1 x 65,536 x 64    3.81 / 2.25
// Hence: examples of up to 2,048 rows on average always; up to 4,096 rows
// while the workgroups fit the device at once (256) or the rows have at most
// 64 components; up to 8,192 rows while the workgroups fit at once.
// PCA_KNN_FEAT_SMALL: 0 never, 1 whenever the shape fits.
constexpr int kFeatSmallMaxK = 48; // widest list of the one-kernel search

bool feat_small_applies(int n, int m, int d, int num_segments, int k,
                        bool cosine) {
  const bool fits = d <= 128 && k <= kFeatSmallMaxK;
  if (const char *env = std::getenv("PCA_KNN_FEAT_SMALL")) {
    if (env[0] == '0')
      return false;
    if (env[0] == '1')
      return fits;
  }
  const long long rows = n, segments = num_segments > 0 ? num_segments : 1;
  const bool at_once = (m + kFeatQueries - 1) / kFeatQueries <= 256;
  return fits && (rows <= 2048 * segments ||
                  (rows <= 4096 * segments && (at_once || d <= 64)) ||
                  (rows <= 8192 * segments && at_once));
}

// list width for k neighbours: k + 16 real entries
int feat_width(int k) {
  static const int widths[] = {24, 32, 48, 64, 80, 116};
  for (int w : widths)
    if (k + kFeatSlack <= w)
      return w;
  return 0;
}

// blocks of 16 components: the coordinates and the block that carries W
int feat_blocks(int d) {
  if (d <= 32)
    return 3;
  if (d <= 64)
    return 5;
  if (d <= 128)
    return 9;
  if (d <= 256)
    return 17;
  return 33;
}

int feat_tile_rows(int d) { return feat_blocks(d) <= 9 ? 64 : 32; }

// flagged queries the threshold scan can take
int feat_redo_cap(int m) { return std::min(m, std::max(8192, m / 4)); }

// rows the threshold scan holds per query: the k it looks for and the ones a
// loose bound let through beside them
int feat_hit_cap(int k) {
  return std::min(kFeatMaxHits, (k + 60 + kWave - 1) / kWave * kWave);
}

size_t feat_pack_bytes(int n, int d) {
  const size_t units = 2 * (size_t)feat_blocks(d) + 1; // FeatShape::RSU
  return align256(sizeof(uint4) * units * ((size_t)n + feat_tile_rows(d)));
}

__global__ __launch_bounds__(kBlock) void feat_init_kernel(
    FeatGlobals *g, float *tau, int m, int *hit_count, int redo_cap,
    int *overflow, unsigned long long *edge_sums, int edge_blocks) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  // (the compaction's block sums, when the search counts the edges)
  if (edge_sums != nullptr && i < edge_blocks)
    edge_sums[i] = 0ull;
  if (i < m) {
    tau[i] = __builtin_inff();
    if (overflow != nullptr)
      overflow[i] = 0;
  }
  if (i < redo_cap)
    hit_count[i] = 0;
  for (int j = i; j < kFeatHistCopies * 256; j += gridDim.x * kBlock) {
    g->hist_x[j] = 0;
    g->hist_y[j] = 0;
  }
  if (i == 0) {
    g->max_bits = 0;
    g->odd_rows = 0;
    g->any_redo = 0;
    g->unresolved = 0;
    g->queued = 0;
    g->out_limit = 0xffffffffu;
    g->n_out = 0;
  }
}

// slices of every segment's x rows of the second pass of the exact kernel
constexpr int kSecondPassChunks = 16;

// Squared norms of rows (16 lanes per row, coalesced reads; any summation
// order serves the filter; NaN for a row with a non-finite component) and the
// largest finite |component| of the matrix.
// big_out (or null): per row, the float bits of that largest |component|;
// hist (or null): rows per binary exponent of it.
__global__ __launch_bounds__(kBlock) void feat_rows_kernel(
    const float *__restrict__ x, int n, int d, float *__restrict__ sq_out,
    FeatGlobals *g, unsigned *__restrict__ big_out,
    unsigned *__restrict__ hist) {
  __shared__ unsigned part[kBlock / kWave];
  __shared__ unsigned local_hist[256];
  static_assert(kBlock == 256, "one thread per exponent");
  local_hist[threadIdx.x] = 0;
  __syncthreads();
  const int sub = threadIdx.x & 15;
  const int row = blockIdx.x * (kBlock / 16) + (threadIdx.x >> 4);
  float s = 0.0f;
  unsigned big = 0;
  if (row < n) {
    const float *p = x + (size_t)row * d;
    bool finite = true;
    auto take = [&](float v) {
      s = __builtin_fmaf(v, v, s);
      const unsigned u = __float_as_uint(v) & 0x7fffffffu;
      if (u >= 0x7f800000u)
        finite = false;
      else if (u > big)
        big = u;
    };
    if ((d & 3) == 0) {
      const float4 *p4 = reinterpret_cast<const float4 *>(p);
      for (int c = sub; c < d / 4; c += 16) {
        const float4 v = p4[c];
        take(v.x), take(v.y), take(v.z), take(v.w);
      }
    } else {
      for (int c = sub; c < d; c += 16)
        take(p[c]);
    }
    // a row with an infinite or NaN component is nobody's neighbour
    // (csrc/cuda/knn_cuda.cu:48,68: its distances are infinite or NaN); it is
    // told apart from a finite row whose squared norm overflows
    if (!finite)
      s = __builtin_nanf("");
  }
#pragma unroll
  for (int sh = 8; sh >= 1; sh >>= 1)
    s += __shfl_xor(s, sh);
  if (row < n && sub == 0 && sq_out != nullptr)
    sq_out[row] = s;
  // rows the filter leaves out do not set the scale
  if (!(s < __builtin_inff()))
    big = 0;
  // the row's own largest component (its 16 lanes)
#pragma unroll
  for (int sh = 8; sh >= 1; sh >>= 1) {
    const unsigned o = (unsigned)__shfl_xor((int)big, sh);
    big = o > big ? o : big;
  }
  if (row < n && sub == 0) {
    if (big_out != nullptr)
      big_out[row] = big;
    if (hist != nullptr && big != 0)
      atomicAdd(&local_hist[big >> 23], 1u);
  }
#pragma unroll
  for (int sh = 32; sh >= 16; sh >>= 1) {
    const unsigned o = (unsigned)__shfl_xor((int)big, sh);
    big = o > big ? o : big;
  }
  if ((threadIdx.x & (kWave - 1)) == 0)
    part[threadIdx.x / kWave] = big;
  __syncthreads();
  // (with a histogram the scale is made from it, feat_scale_kernel: the
  // first couple of thousand workgroups of a launch all find this word at
  // zero, and their maxima on one word took 20 us)
  if (threadIdx.x == 0 && hist == nullptr && g != nullptr) {
    for (int w = 1; w < kBlock / kWave; ++w)
      big = part[w] > big ? part[w] : big;
    // (one word for the whole call: only workgroups that raise it go there)
    if (big != 0 && big > __hip_atomic_load(&g->max_bits, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT))
      atomicMax(&g->max_bits, big);
  }
  if (hist != nullptr && local_hist[threadIdx.x] != 0)
    atomicAdd(&hist[(blockIdx.x % kFeatHistCopies) * 256 + threadIdx.x],
              local_hist[threadIdx.x]);
}

// The scale of the Euclidean filter: made for the largest component of all
// rows, unless a few rows (up to kFeatMaxOutliers of x and as many of y, and
// never more than one in 64) are at least four times larger than all others --
// then for the others, which keep their bits in fp16; the few are handled
// exactly (see FeatGlobals).  One workgroup of 256 threads.
// (y_is_x: the queries are the rows of x, whose histogram stands for both)
__global__ __launch_bounds__(256) void feat_scale_kernel(FeatGlobals *g, int n,
                                                         int m, bool y_is_x) {
  __shared__ unsigned hx[256], hy[256];
  __shared__ int need_x, need_y, top;
  const int t = threadIdx.x;
  unsigned sum_x = 0, sum_y = 0;
  for (int c = 0; c < kFeatHistCopies; ++c) {
    sum_x += g->hist_x[c * 256 + t];
    sum_y += g->hist_y[c * 256 + t];
  }
  if (y_is_x)
    sum_y = sum_x;
  hx[t] = sum_x;
  hy[t] = sum_y;
  if (t == 0) {
    need_x = 255;
    need_y = 255;
    top = -1;
  }
  __syncthreads();
  // rows with a larger exponent than t: one wave, four bins per lane, a
  // suffix sum over the lanes
  __shared__ unsigned ax[256], ay[256];
  if (t < kWave) {
    unsigned vx[4], vy[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      vx[i] = hx[4 * t + i];
      vy[i] = hy[4 * t + i];
    }
    const unsigned own_x = vx[0] + vx[1] + vx[2] + vx[3];
    const unsigned own_y = vy[0] + vy[1] + vy[2] + vy[3];
    unsigned sx = own_x, sy = own_y; // this lane's bins and all behind them
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1) {
      const unsigned ox = __shfl_down(sx, sh);
      const unsigned oy = __shfl_down(sy, sh);
      if (t + sh < kWave) {
        sx += ox;
        sy += oy;
      }
    }
    unsigned behind_x = sx - own_x, behind_y = sy - own_y;
#pragma unroll
    for (int i = 3; i >= 0; --i) {
      ax[4 * t + i] = behind_x;
      ay[4 * t + i] = behind_y;
      behind_x += vx[i];
      behind_y += vy[i];
    }
  }
  __syncthreads();
  const unsigned above_x = ax[t], above_y = ay[t];
  const unsigned allow_x = (unsigned)min(kFeatMaxOutliers, n / 64);
  const unsigned allow_y = (unsigned)min(kFeatMaxOutliers, m / 64);
  // the smallest exponent that leaves at most that many rows above it (not
  // below the smallest one in use: rows, not bins, are what is left out)
  if (above_x <= allow_x && (hx[t] != 0 || above_x == 0))
    atomicMin(&need_x, t);
  if (above_y <= allow_y && (hy[t] != 0 || above_y == 0))
    atomicMin(&need_y, t);
  if (hx[t] != 0 || hy[t] != 0)
    atomicMax(&top, t);
  __syncthreads();
  if (t == 0) {
    // (only the exponent of max_bits is used: the largest number of the
    // binade stands for the largest component)
    const int need = max(need_x, need_y);
    if (top - need >= 2) {
      g->max_bits = ((unsigned)(need + 1) << 23) - 1u;
      g->out_limit = g->max_bits;
    } else {
      g->max_bits = top < 0 ? 0u : ((unsigned)(top + 1) << 23) - 1u;
    }
  }
}

// The k smallest keys of a queued query's hit list (one wave per query); a
// list that overflowed sends its query to the full second pass.
__global__ __launch_bounds__(kBlock) void feat_redo_select_kernel(
    KnnFeatParams p) {
  constexpr int WAVES = kBlock / kWave;
  constexpr int PER = kFeatMaxHits / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int j = blockIdx.x * WAVES + threadIdx.x / kWave;
  const int queued = min(p.globals->queued, p.redo_cap);
  if (j >= queued)
    return;
  const int q = p.redo_list[j];
  const int found = p.hit_count[j];
  if (found > p.hit_cap) {
    if (lane == 0) {
      p.redo_q[q] = 1;
      atomicAdd(&p.globals->unresolved, 1);
    }
    return;
  }
  double keys[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = i * kWave + lane;
    keys[i] = e < found ? p.hits[(size_t)j * p.hit_cap + e] : empty_key();
  }
  const int k = p.k;
  const size_t slot0 = (size_t)q * k;
  int taken = 0;
  for (; taken < k; ++taken) {
    double mine = keys[0];
#pragma unroll
    for (int i = 1; i < PER; ++i)
      mine = keys[i] < mine ? keys[i] : mine;
    double least = mine;
#pragma unroll
    for (int sh = 32; sh >= 1; sh >>= 1) {
      const double o = __shfl_xor(least, sh);
      least = o < least ? o : least;
    }
    if (!(least < empty_key()))
      break;
    // (keys differ: rows differ)
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (keys[i] == least)
        keys[i] = empty_key();
    if (lane == 0) {
      p.out_idx[slot0 + taken] = key_row(least);
      if (p.out_dist)
        p.out_dist[slot0 + taken] = key_dist(least);
    }
  }
  if (lane == 0)
    p.out_count[q] = taken;
}

template <int KP>
void launch_feat_merge(const KnnFeatParams &p, int tiles_bound,
                       hipStream_t stream) {
  hipLaunchKernelGGL((feat_merge_kernel<KP>), dim3(tiles_bound), dim3(kBlock),
                     0, stream, p);
}

// Single workgroup: per segment the first 512-query tile and the first
// (tile, unit) pair -- exclusive sums of tiles_s and of tiles_s * units_s.
__global__ __launch_bounds__(kPlanThreads) void feat_wide_plan_kernel(
    const int64_t *__restrict__ ptr_x, const int64_t *__restrict__ ptr_y,
    int n, int m, int num_segments, int *__restrict__ tile_start,
    long long *__restrict__ unit_start) {
  __shared__ long long part_u[kPlanThreads];
  __shared__ int part_t[kPlanThreads];
  const int tid = threadIdx.x;
  const int per_thread = (num_segments + kPlanThreads - 1) / kPlanThreads;
  const int b0 = min(tid * per_thread, num_segments);
  const int b1 = min(b0 + per_thread, num_segments);
  auto counts = [&](int b, int &tiles, long long &pairs) {
    const int64_t xl = ptr_x ? ptr_x[b] : 0, xh = ptr_x ? ptr_x[b + 1] : n;
    const int64_t yl = ptr_y ? ptr_y[b] : 0, yh = ptr_y ? ptr_y[b + 1] : m;
    const int rows = (int)max((int64_t)0, xh - xl);
    const int queries = (int)max((int64_t)0, yh - yl);
    tiles = (queries + kWideQueries - 1) / kWideQueries;
    pairs = (long long)tiles * ((rows + kWideTileRows - 1) / kWideTileRows);
  };
  int st = 0;
  long long su = 0;
  for (int b = b0; b < b1; ++b) {
    int t;
    long long u;
    counts(b, t, u);
    st += t;
    su += u;
  }
  part_t[tid] = st;
  part_u[tid] = su;
  __syncthreads();
  for (int off = 1; off < kPlanThreads; off <<= 1) {
    const int vt = tid >= off ? part_t[tid - off] : 0;
    const long long vu = tid >= off ? part_u[tid - off] : 0;
    __syncthreads();
    part_t[tid] += vt;
    part_u[tid] += vu;
    __syncthreads();
  }
  int rt = part_t[tid] - st;
  long long ru = part_u[tid] - su;
  for (int b = b0; b < b1; ++b) {
    tile_start[b] = rt;
    unit_start[b] = ru;
    int t;
    long long u;
    counts(b, t, u);
    rt += t;
    ru += u;
  }
  if (tid == kPlanThreads - 1) {
    tile_start[num_segments] = part_t[tid];
    unit_start[num_segments] = part_u[tid];
  }
}

// list width of the eight-wave first stage: the k smallest values
int feat_wide_width(int k) {
  static const int widths[] = {16, 32, 64, 100};
  for (int w : widths)
    if (k <= w)
      return w;
  return 0;
}

int device_cu_count() {
  static int cached = 0;
  if (cached == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount,
                              dev) != hipSuccess ||
        cus <= 0)
      cus = 256;
    cached = cus;
  }
  return cached;
}

// The eight-wave first stage (knn_feat_wide_impl.hpp) takes calls with enough
// queries per segment to fill its tiles of 512.
bool feat_wide_applies(int m, int d, int num_segments, int k) {
  const bool fits = d <= kWideMaxDim && feat_wide_width(k) != 0;
  // PCA_KNN_FEAT_WIDE: 0 never, 1 whenever the shape fits (the tests)
  if (const char *env = std::getenv("PCA_KNN_FEAT_WIDE")) {
    if (env[0] == '0')
      return false;
    if (env[0] == '1')
      return fits;
  }
  return fits && m >= 4096 && (long long)num_segments * 1024 <= (long long)m;
}

struct FeatWidePlan {
  int grid;      // workgroups of the first stage
  int tiles;     // upper bound of the 512-query tiles
  int cap;       // buffer entries per (piece, query)
  size_t pieces; // upper bound of the pieces
};

FeatWidePlan feat_wide_plan(int n, int m, int num_segments, int k) {
  FeatWidePlan w;
  w.tiles = plan_upper_bound(m, num_segments, kWideQueries);
  // (tile, unit) pairs, roughly: every tile of a segment meets the segment's
  // units
  const long long units_per_segment =
      ((long long)n / num_segments + kWideTileRows - 1) / kWideTileRows + 1;
  const long long pairs = (long long)w.tiles * units_per_segment;
  w.grid = (int)std::max(1LL, std::min((long long)device_cu_count(),
                                       pairs / 4));
  if (const char *env = std::getenv("PCA_FEAT_WIDE_GRID")) {
    const int v = std::atoi(env);
    if (v >= 1 && v <= 4096)
      w.grid = v;
  }
  // (per query, piece and half of the wave; a checkpoint tidies a buffer
  // that is half full, and one that comes within two tiles of its end)
  w.cap = (96 + 2 * (k + kFeatSlack) + 63) / 64 * 64;
  if (const char *env = std::getenv("PCA_FEAT_WIDE_CAP")) {
    const int v = std::atoi(env);
    if (v >= 192 && v <= 8192)
      w.cap = v / 64 * 64;
  }
  w.pieces = (size_t)w.grid + (size_t)w.tiles;
  return w;
}

struct FeatLayout {
  size_t globals, x_norm, x_class, y_norm, tau, redo, over, plan256;
  size_t redo_list, redo_tau, hit_count, hits; // threshold scan
  size_t pack, partial, cand; // first pass
  // eight-wave first stage: `partial` is then these four
  size_t wide_plan = 0, wide_buf = 0, wide_count = 0, wide_lists = 0,
         wide_owners = 0;
  size_t second;              // second pass (reuses the first pass's bytes)
  size_t shared() const {
    return globals + x_norm + x_class + y_norm + tau + redo + over + plan256 +
           redo_list + redo_tau + hit_count + hits;
  }
  size_t total() const {
    return shared() + std::max(pack + partial + cand, second);
  }
};

} // namespace

bool knn_feat_supported(int d, int k, bool cosine) {
  if (const char *env = std::getenv("PCA_KNN_NO_MFMA"))
    if (env[0] == '1')
      return false;
  if (const char *env = std::getenv("PCA_KNN_FEAT"))
    if (env[0] == '0')
      return false;
  (void)cosine;
  return d > 8 && d <= kFeatMaxDim && k >= 1 && feat_width(k) != 0;
}

int knn_feat_slices(int n, int m, int d, int num_segments) {
  const int tiles = plan_upper_bound(m, num_segments, kFeatQueries);
  const int want = (3072 + tiles - 1) / tiles;
  const int by_length = (n / num_segments) / (8 * feat_tile_rows(d));
  int chunks = std::max(1, std::min(std::min(want, 32), by_length));
  if (const char *env = std::getenv("PCA_KNN_SLICES")) {
    const int v = std::atoi(env);
    if (v >= 1 && v <= 64)
      chunks = v;
  }
  return chunks;
}

// the full second pass: the exact matrix-core kernel where it applies, else
// the any-dimension kernel
static bool second_pass_on_matrix_cores(int d, int k) {
  return d <= 128 && k <= 64;
}

static FeatLayout feat_layout(int n, int m, int d, int num_segments, int k) {
  FeatLayout w;
  const size_t tiles = plan_upper_bound(m, num_segments, kFeatQueries);
  const int chunks = knn_feat_slices(n, m, d, num_segments);
  const size_t kk = (size_t)k + kFeatSlack;
  w.globals = align256(sizeof(FeatGlobals));
  w.x_norm = align256(sizeof(float) * (size_t)n);
  w.x_class = align256(sizeof(float) * (size_t)n);
  w.y_norm = align256(sizeof(float) * (size_t)m);
  w.tau = align256(sizeof(float) * (size_t)m);
  w.redo = align256(sizeof(int) * (size_t)m);
  w.over = align256(sizeof(int) * (size_t)m);
  w.plan256 = align256(sizeof(int) * ((size_t)num_segments + 1));
  const size_t cap = (size_t)feat_redo_cap(m);
  w.redo_list = align256(sizeof(int) * cap);
  w.redo_tau = align256(sizeof(float) * cap);
  w.hit_count = align256(sizeof(int) * cap);
  w.hits = align256(sizeof(double) * cap * feat_hit_cap(k));
  w.pack = feat_pack_bytes(n, d);
  if (feat_wide_applies(m, d, num_segments, k)) {
    const FeatWidePlan wp = feat_wide_plan(n, m, num_segments, k);
    w.wide_plan = align256(sizeof(int) * ((size_t)num_segments + 1)) +
                  align256(sizeof(long long) * ((size_t)num_segments + 1));
    w.wide_buf =
        align256(sizeof(uint2) * wp.pieces * kWideQueries * 2 * wp.cap);
    w.wide_count = align256(sizeof(int) * wp.pieces * 2 * kWideQueries);
    w.wide_owners =
        align256(sizeof(WideOwner) * (size_t)wp.grid * kWideQueries);
    w.wide_lists = align256(sizeof(float) * (size_t)wp.grid *
                            feat_wide_width(k) * kWideQueries);
    w.partial = w.wide_plan + w.wide_buf + w.wide_count + w.wide_lists +
                w.wide_owners;
  } else {
    w.partial = align256(sizeof(double) * tiles * chunks * kk * kFeatQueries);
  }
  w.cand = align256(sizeof(double) * (size_t)m * kk);
  w.second = second_pass_on_matrix_cores(d, k)
                 ? knn_mfma_scratch_bytes(n, m, d, num_segments, k,
                                          kSecondPassChunks)
                 : knn_generic_scratch_bytes(n, m, num_segments, k);
  return w;
}

size_t knn_feat_scratch_bytes(int n, int m, int d, int num_segments, int k) {
  return feat_layout(n, m, d, num_segments, k).total();
}

namespace {

// fp16 / bf16 rows of d components as fp32 (exact) and, for the filter (kept
// or null), with every component times chain_keep (exact as well)
template <bool BF16>
__global__ __launch_bounds__(kBlock) void widen16_kernel(
    const uint16_t *__restrict__ src, size_t count, int d,
    float *__restrict__ dst, float *__restrict__ kept) {
  const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= count)
    return;
  const uint16_t v = src[i];
  const float wide = BF16 ? __uint_as_float((uint32_t)v << 16)
                          : (float)__builtin_bit_cast(_Float16, v);
  dst[i] = wide;
  if (kept != nullptr)
    kept[i] = wide * chain_keep<BF16 ? 2 : 1>(d, (int)(i % (size_t)d));
}

void launch_widen16(const void *src, size_t count, int d, bool bf16,
                    float *dst, float *kept, hipStream_t stream) {
  const unsigned grid = (unsigned)((count + kBlock - 1) / kBlock);
  if (bf16)
    hipLaunchKernelGGL(widen16_kernel<true>, dim3(grid), dim3(kBlock), 0,
                       stream, static_cast<const uint16_t *>(src), count, d,
                       dst, kept);
  else
    hipLaunchKernelGGL(widen16_kernel<false>, dim3(grid), dim3(kBlock), 0,
                       stream, static_cast<const uint16_t *>(src), count, d,
                       dst, kept);
}

} // namespace

bool knn_feat_one_kernel(int n, int m, int d, int num_segments, int k,
                         bool cosine) {
  return knn_feat_supported(d, k, cosine) &&
         feat_small_applies(n, m, d, num_segments, k, cosine);
}

bool radius_feat_supported(int n, int m, int d, int num_segments, int slots,
                           int r16) {
  // (fp32 points of up to eight dimensions have kernels of their own; 16-bit
  // ones have none but the exhaustive scan)
  const bool fits =
      (r16 != 0 ? d >= 1 : d > 8) && d <= 128 && slots >= 1 && slots <= 32;
  if (const char *env = std::getenv("PCA_RADIUS_FEAT")) {
    if (env[0] == '0')
      return false;
    if (env[0] == '1')
      return fits;
  }
  // (the preparation is half a dozen launches: small searches are quicker
  // with the plain scan)
  const double work = (double)n / (num_segments > 0 ? num_segments : 1) *
                      (double)m * (double)d;
  return fits && work >= 16.0e6;
}

bool knn_feat16_supported(int n, int d, int num_segments, int k, bool cosine,
                          bool bf16) {
  if (const char *env = std::getenv("PCA_KNN_FEAT_16BIT"))
    if (env[0] == '0')
      return false;
  (void)bf16; // (both types up to 128 components)
  return !cosine && d >= 1 && d <= 128 && k <= kFeatSmallMaxK &&
         n >= 1 &&
         num_segments >= 1;
}

size_t knn_feat16_scratch_bytes(int n, int m, int d, int num_segments,
                                int k) {
  // (x twice: as it is, and as the filter takes it)
  return 2 * align256(sizeof(float) * (size_t)n * d) +
         align256(sizeof(float) * (size_t)m * d) +
         knn_feat_scratch_bytes(n, m, d, num_segments, k);
}

hipError_t launch_knn_feat(const SearchInput &in_given, int k, bool cosine,
                           const int *work_start, void *scratch,
                           const DenseResult &out, hipEvent_t time_start,
                           hipEvent_t time_stop, hipStream_t stream,
                           int r16, const FeatRadius *radius) {
  SearchInput in = in_given;
  if (radius != nullptr && cosine)
    return hipErrorInvalidValue;
  // the rows of x the filter is made from (16-bit rows: scaled, see
  // chain_keep; else the rows themselves)
  const float *x_for_filter = nullptr;
  if (r16 != 0) {
    // 16-bit rows: searched as fp32 rows (the widening is exact) by the one
    // kernel that can compute the exact distances in the 16-bit arithmetic
    if (cosine || in.d > 128 || k > kFeatSmallMaxK)
      return hipErrorInvalidValue;
    char *at = static_cast<char *>(scratch);
    float *x32 = reinterpret_cast<float *>(at);
    at += align256(sizeof(float) * (size_t)in.n * in.d);
    float *x_kept = reinterpret_cast<float *>(at);
    at += align256(sizeof(float) * (size_t)in.n * in.d);
    float *y32 = reinterpret_cast<float *>(at);
    at += align256(sizeof(float) * (size_t)in.m * in.d);
    scratch = at;
    const bool y_is_x = in.y == in.x && in.m == in.n;
    launch_widen16(in.x, (size_t)in.n * in.d, in.d, r16 == 2, x32, x_kept,
                   stream);
    // (the search kernel scales the queries itself)
    if (!y_is_x)
      launch_widen16(in.y, (size_t)in.m * in.d, in.d, r16 == 2, y32, nullptr,
                     stream);
    in.x = x32;
    in.y = y_is_x ? x32 : y32;
    x_for_filter = x_kept;
  }
  const FeatLayout lay =
      feat_layout(in.n, in.m, in.d, in.num_segments, k);
  const int tiles_bound =
      plan_upper_bound(in.m, in.num_segments, kFeatQueries);
  const int chunks = knn_feat_slices(in.n, in.m, in.d, in.num_segments);
  char *base = static_cast<char *>(scratch);
  auto take = [&base](size_t bytes) {
    char *piece = base;
    base += bytes;
    return piece;
  };
  FeatGlobals *globals = reinterpret_cast<FeatGlobals *>(take(lay.globals));
  float *x_norm = reinterpret_cast<float *>(take(lay.x_norm));
  float *x_class_buf = reinterpret_cast<float *>(take(lay.x_class));
  float *y_norm = reinterpret_cast<float *>(take(lay.y_norm));
  float *tau = reinterpret_cast<float *>(take(lay.tau));
  int *redo_q = reinterpret_cast<int *>(take(lay.redo));
  int *overflow = reinterpret_cast<int *>(take(lay.over));
  int *plan256 = reinterpret_cast<int *>(take(lay.plan256));
  int *redo_list = reinterpret_cast<int *>(take(lay.redo_list));
  float *redo_tau = reinterpret_cast<float *>(take(lay.redo_tau));
  int *hit_count = reinterpret_cast<int *>(take(lay.hit_count));
  double *hits = reinterpret_cast<double *>(take(lay.hits));
  const int redo_cap = feat_redo_cap(in.m);
  char *first_pass = base;
  uint4 *x_pack = reinterpret_cast<uint4 *>(take(lay.pack));
  double *partial = reinterpret_cast<double *>(take(lay.partial));
  double *cand = reinterpret_cast<double *>(take(lay.cand));

  const float *xf = static_cast<const float *>(in.x);
  const float *xp = x_for_filter != nullptr ? x_for_filter : xf;
  const float *yf = static_cast<const float *>(in.y);
  const int nb = feat_blocks(in.d);

  const bool small = r16 != 0 || radius != nullptr ||
                     feat_small_applies(in.n, in.m, in.d, in.num_segments, k,
                                        cosine);
  hipLaunchKernelGGL(feat_init_kernel, dim3((in.m + kBlock - 1) / kBlock),
                     dim3(kBlock), 0, stream, globals, tau, in.m, hit_count,
                     redo_cap, overflow, small ? out.edge_sums : nullptr,
                     (in.m + kCompactBlockQueries - 1) / kCompactBlockQueries +
                         1);
  // squared norms that only classify the rows (NaN: a non-finite component);
  // for the Euclidean distance they also enter the filter
  float *x_class = cosine ? x_class_buf : x_norm;
  unsigned *x_big = nullptr;
  const int rows_per_block = kBlock / 16;
  if (cosine) {
    // |x|, |y| as the reference's Cosine::norm computes them: they enter the
    // exact distances
    (void)launch_row_norms(xf, in.n, in.d, x_norm, stream);
    (void)launch_row_norms(yf, in.m, in.d, y_norm, stream);
    // (no scale to make: the rows are normalised one by one)
    hipLaunchKernelGGL(feat_rows_kernel,
                       dim3((in.n + rows_per_block - 1) / rows_per_block),
                       dim3(kBlock), 0, stream, xf, in.n, in.d, x_class,
                       static_cast<FeatGlobals *>(nullptr),
                       static_cast<unsigned *>(nullptr),
                       static_cast<unsigned *>(nullptr));
  } else {
    // (the classification buffer is free here: it holds every row's largest
    // component)
    x_big = reinterpret_cast<unsigned *>(x_class_buf);
    hipLaunchKernelGGL(feat_rows_kernel,
                       dim3((in.n + rows_per_block - 1) / rows_per_block),
                       dim3(kBlock), 0, stream, xp, in.n, in.d, x_norm,
                       globals, x_big, globals->hist_x);
    // (a cloud searched in itself: one pass over the rows serves both)
    const bool y_is_x = yf == xf && in.m == in.n;
    if (!y_is_x)
      hipLaunchKernelGGL(feat_rows_kernel,
                         dim3((in.m + rows_per_block - 1) / rows_per_block),
                         dim3(kBlock), 0, stream, yf, in.m, in.d,
                         static_cast<float *>(nullptr), globals,
                         static_cast<unsigned *>(nullptr), globals->hist_y);
    hipLaunchKernelGGL(feat_scale_kernel, dim3(1), dim3(256), 0, stream,
                       globals, in.n, in.m, y_is_x);
  }
  {
    hipError_t perr;
    switch (nb) {
    case 3:
      perr = launch_feat_pack<3>(xp, x_norm, x_class, x_big, in.n, in.d,
                                 cosine, globals, x_pack, stream);
      break;
    case 5:
      perr = launch_feat_pack<5>(xp, x_norm, x_class, x_big, in.n, in.d,
                                 cosine, globals, x_pack, stream);
      break;
    case 9:
      perr = launch_feat_pack<9>(xp, x_norm, x_class, x_big, in.n, in.d,
                                 cosine, globals, x_pack, stream);
      break;
    case 17:
      perr = launch_feat_pack<17>(xp, x_norm, x_class, x_big, in.n, in.d,
                                  cosine, globals, x_pack, stream);
      break;
    default:
      perr = launch_feat_pack<33>(xp, x_norm, x_class, x_big, in.n, in.d,
                                  cosine, globals, x_pack, stream);
      break;
    }
    if (perr != hipSuccess)
      return perr;
  }

  KnnFeatParams p;
  p.x = xf;
  p.y = yf;
  p.ptr_x = in.ptr_x;
  p.ptr_y = in.ptr_y;
  p.x_norm = x_norm;
  p.y_norm = y_norm;
  p.x_pack = x_pack;
  p.globals = globals;
  p.n = in.n;
  p.m = in.m;
  p.d = in.d;
  p.num_segments = in.num_segments;
  p.k = k;
  p.work_start = work_start;
  p.num_chunks = chunks;
  // (tiles of 32 rows, from 129 components on: every 4 tiles measured 2-4 %
  // faster than every 8 at 256 components; tiles of 64 rows: the other way)
  p.round_period = feat_tile_rows(in.d) == 64 ? kFeatRoundPeriod
                                              : kFeatRoundPeriod / 2;
  if (const char *env = std::getenv("PCA_FEAT_ROUND_PERIOD")) {
    const int v = std::atoi(env);
    if (v >= 1 && v <= 64)
      p.round_period = v;
  }
  p.tau = tau;
  p.partial = partial;
  p.cand = cand;
  p.redo_q = redo_q;
  p.redo_list = redo_list;
  p.redo_tau = redo_tau;
  p.hit_count = hit_count;
  p.hits = hits;
  p.redo_cap = redo_cap;
  p.hit_cap = feat_hit_cap(k);
  p.overflow = nullptr;
  p.out_idx = out.idx;
  p.out_dist = out.dist;
  p.out_count = out.count;

  const int kp = feat_width(k);
  hipError_t err;
  if (small) {
    p.edge_sums = out.edge_sums;
    p.self_pos = out.self_pos;
    p.kept = out.kept;
    // one exact kernel: nothing is listed, merged, refined or searched again
    // (in steps of 8: the lists' padding in front is at most 7 entries)
    const int kbucket = (k + 7) / 8 * 8;
    if (radius != nullptr) {
      p.r2 = radius->r2;
      p.ignore_same = radius->ignore_same ? 1 : 0;
    }
    if (time_start)
      (void)hipEventRecord(time_start, stream);
#define PCA_SMALL_CASE(NB)                                                     \
  err = radius                                                                 \
            ? (r16 == 0   ? launch_radius_feat_blocks<NB, 0>(                  \
                                p, kbucket, tiles_bound, stream)               \
               : r16 == 1 ? launch_radius_feat_blocks<NB, 1>(                  \
                                p, kbucket, tiles_bound, stream)               \
                          : launch_radius_feat_blocks<NB, 2>(                  \
                                p, kbucket, tiles_bound, stream))              \
        : cosine   ? launch_knn_feat_small_blocks<NB, 3>(p, kbucket,           \
                                                         tiles_bound, stream)  \
        : r16 == 0 ? launch_knn_feat_small_blocks<NB, 0>(p, kbucket,           \
                                                         tiles_bound, stream)  \
        : r16 == 1 ? launch_knn_feat_small_blocks<NB, 1>(p, kbucket,           \
                                                         tiles_bound, stream)  \
                   : launch_knn_feat_small_blocks<NB, 2>(p, kbucket,           \
                                                         tiles_bound, stream)
    switch (nb) {
    case 3:
      PCA_SMALL_CASE(3);
      break;
    case 5:
      PCA_SMALL_CASE(5);
      break;
    default:
      PCA_SMALL_CASE(9);
      break;
    }
#undef PCA_SMALL_CASE
    if (time_stop)
      (void)hipEventRecord(time_stop, stream);
    return err;
  } else if (lay.wide_buf != 0) {
    // eight-wave first stage: plan, filter, gather
    const FeatWidePlan wp = feat_wide_plan(in.n, in.m, in.num_segments, k);
    char *wb = reinterpret_cast<char *>(partial);
    KnnFeatWideParams wpar;
    p.overflow = overflow;
    wpar.base = p;
    int *tile_start = reinterpret_cast<int *>(wb);
    long long *unit_start = reinterpret_cast<long long *>(
        wb + align256(sizeof(int) * ((size_t)in.num_segments + 1)));
    wb += lay.wide_plan;
    wpar.tile_start = tile_start;
    wpar.unit_start = unit_start;
    wpar.cap = wp.cap;
    wpar.ckpt_growth = 32;
    if (const char *env = std::getenv("PCA_FEAT_WIDE_CKPT")) {
      const int v = std::atoi(env);
      if (v >= 17 && v <= 64)
        wpar.ckpt_growth = v;
    }
    wpar.buf = reinterpret_cast<uint2 *>(wb);
    wb += lay.wide_buf;
    wpar.buf_count = reinterpret_cast<int *>(wb);
    wb += lay.wide_count;
    wpar.lists = reinterpret_cast<float *>(wb);
    wb += lay.wide_lists;
    wpar.owners = reinterpret_cast<WideOwner *>(wb);
    wpar.overflow = overflow;
    hipLaunchKernelGGL(feat_wide_plan_kernel, dim3(1), dim3(kPlanThreads), 0,
                       stream, in.ptr_x, in.ptr_y, in.n, in.m,
                       in.num_segments, tile_start, unit_start);
    if (time_start)
      (void)hipEventRecord(time_start, stream);
    const int kw = feat_wide_width(k);
    switch (nb) {
    case 3:
      err = launch_knn_feat_wide_blocks<3>(wpar, kw, cosine, wp.grid, stream);
      break;
    case 5:
      err = launch_knn_feat_wide_blocks<5>(wpar, kw, cosine, wp.grid, stream);
      break;
    default:
      err = launch_knn_feat_wide_blocks<9>(wpar, kw, cosine, wp.grid, stream);
      break;
    }
    if (time_stop)
      (void)hipEventRecord(time_stop, stream);
    if (err != hipSuccess)
      return err;
    const int ggrid = wp.tiles * (kWideQueries / kBlock);
    switch (kp) {
    case 24:
      hipLaunchKernelGGL((feat_wide_gather_kernel<24>), dim3(ggrid),
                         dim3(kBlock), 0, stream, wpar, wp.grid);
      break;
    case 32:
      hipLaunchKernelGGL((feat_wide_gather_kernel<32>), dim3(ggrid),
                         dim3(kBlock), 0, stream, wpar, wp.grid);
      break;
    case 48:
      hipLaunchKernelGGL((feat_wide_gather_kernel<48>), dim3(ggrid),
                         dim3(kBlock), 0, stream, wpar, wp.grid);
      break;
    case 64:
      hipLaunchKernelGGL((feat_wide_gather_kernel<64>), dim3(ggrid),
                         dim3(kBlock), 0, stream, wpar, wp.grid);
      break;
    case 80:
      hipLaunchKernelGGL((feat_wide_gather_kernel<80>), dim3(ggrid),
                         dim3(kBlock), 0, stream, wpar, wp.grid);
      break;
    default:
      hipLaunchKernelGGL((feat_wide_gather_kernel<116>), dim3(ggrid),
                         dim3(kBlock), 0, stream, wpar, wp.grid);
      break;
    }
  } else {
  const int grid = tiles_bound * chunks;
  if (time_start)
    (void)hipEventRecord(time_start, stream);
  switch (nb) {
  case 3:
    err = launch_knn_feat_blocks<3>(p, kp, cosine, grid, stream);
    break;
  case 5:
    err = launch_knn_feat_blocks<5>(p, kp, cosine, grid, stream);
    break;
  case 9:
    err = launch_knn_feat_blocks<9>(p, kp, cosine, grid, stream);
    break;
  case 17:
    err = launch_knn_feat_blocks<17>(p, kp, cosine, grid, stream);
    break;
  default:
    err = launch_knn_feat_blocks<33>(p, kp, cosine, grid, stream);
    break;
  }
  if (time_stop)
    (void)hipEventRecord(time_stop, stream);
  if (err != hipSuccess)
    return err;

  switch (kp) {
  case 24:
    launch_feat_merge<24>(p, tiles_bound, stream);
    break;
  case 32:
    launch_feat_merge<32>(p, tiles_bound, stream);
    break;
  case 48:
    launch_feat_merge<48>(p, tiles_bound, stream);
    break;
  case 64:
    launch_feat_merge<64>(p, tiles_bound, stream);
    break;
  case 80:
    launch_feat_merge<80>(p, tiles_bound, stream);
    break;
  default:
    launch_feat_merge<116>(p, tiles_bound, stream);
    break;
  }
  }
  {
    const int waves = kBlock / kWave;
    const int rgrid = (in.m + waves - 1) / waves;
    if (cosine)
      hipLaunchKernelGGL((feat_refine_kernel<true>), dim3(rgrid),
                         dim3(kBlock), 0, stream, p);
    else
      hipLaunchKernelGGL((feat_refine_kernel<false>), dim3(rgrid),
                         dim3(kBlock), 0, stream, p);
  }
  err = hipGetLastError();
  if (err != hipSuccess)
    return err;

  // The flagged queries: the kernels are queued in any case and leave at once
  // while nothing is flagged (no host read in between).  First the scan that
  // collects the rows at or below a query's k-th listed distance, then --
  // only for what that scan could not take -- the full second pass.
  {
    const int waves = kBlock / kWave;
    const int sgrid =
        (redo_cap + kFeatRedoGroup - 1) / kFeatRedoGroup * kFeatRedoSlices;
    if (cosine)
      hipLaunchKernelGGL((feat_redo_scan_kernel<true>), dim3(sgrid),
                         dim3(kBlock), 0, stream, p);
    else
      hipLaunchKernelGGL((feat_redo_scan_kernel<false>), dim3(sgrid),
                         dim3(kBlock), 0, stream, p);
    hipLaunchKernelGGL(feat_redo_select_kernel,
                       dim3((redo_cap + waves - 1) / waves), dim3(kBlock), 0,
                       stream, p);
    err = hipGetLastError();
    if (err != hipSuccess)
      return err;
  }
  const int *gate = &globals->unresolved;
  if (second_pass_on_matrix_cores(in.d, k)) {
    MfmaSecondPass second{gate, redo_q, x_norm, y_norm, kSecondPassChunks};
    return launch_knn_mfma(in, k, cosine, work_start, first_pass, out, nullptr,
                           nullptr, stream, nullptr, &second);
  }
  err = launch_plan(in.ptr_y, in.m, in.num_segments, kBlock, plan256, stream);
  if (err != hipSuccess)
    return err;
  return launch_knn_generic(
      in, k, cosine, x_norm, plan256,
      plan_upper_bound(in.m, in.num_segments, kBlock), out, stream,
      lay.second ? first_pass : nullptr, gate, redo_q);
}

} // namespace pca
