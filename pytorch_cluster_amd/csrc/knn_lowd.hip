// Dispatch of the low-dimensional kNN kernels (see knn_lowd_impl.hpp) and of
// the any-dimension kernel (knn_generic_impl.hpp).
#include "knn_generic_impl.hpp"
#include "knn_lowd_impl.hpp"
#include "knn_lowd_mc_impl.hpp"

#include <algorithm>
#include <cstdlib>

namespace pca {

namespace {

// Points are padded with zero components up to the next compiled width; a
// zero component adds fma(0, 0, acc) = acc, so results do not change.
int padded_dim(int d) {
  if (d <= 2)
    return 2;
  if (d <= 4)
    return d;
  return 8;
}

int k_bucket(int k) {
  static const int buckets[] = {8, 16, 24, 32, 48, 64, 100};
  for (int b : buckets)
    if (k <= b)
      return b;
  return 0;
}

int env_int(const char *name, int fallback) {
  const char *v = std::getenv(name);
  return v ? std::atoi(v) : fallback;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

__global__ __launch_bounds__(kBlock) void fill_f32_kernel(float *p, int n,
                                                          float v) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n)
    p[i] = v;
}

template <int KB>
void launch_merge(const KnnLowdParams &p, int tile_queries, int tiles_bound,
                  hipStream_t stream) {
  if (tile_queries == kMcQueries) {
    hipLaunchKernelGGL((knn_merge_kernel<KB, kMcQueries>), dim3(tiles_bound),
                       dim3(kBlock), 0, stream, p);
    return;
  }
  if constexpr (KB <= 32) {
    if (tile_queries == 2 * kBlock) {
      hipLaunchKernelGGL((knn_merge_kernel<KB, 2 * kBlock>), dim3(tiles_bound),
                         dim3(kBlock), 0, stream, p);
      return;
    }
  }
  hipLaunchKernelGGL((knn_merge_kernel<KB, kBlock>), dim3(tiles_bound),
                     dim3(kBlock), 0, stream, p);
}

} // namespace

bool knn_lowd_supported(int d, int k, bool /*cosine*/) {
  return d >= 1 && d <= 8 && k >= 1 && k <= 100;
}

KnnLowdConfig knn_lowd_config(int /*d*/, int k, int n, int m,
                              int num_segments, bool cosine) {
  KnnLowdConfig cfg;
  cfg.kbucket = k_bucket(k);
  // One query per lane keeps four waves per SIMD resident and measures
  // fastest; two per lane (half the LDS reads per distance, more registers)
  // stay available for experiments.
  int qpt = 1;
  const int forced_qpt = env_int("PCA_KNN_QUERIES_PER_LANE", 0);
  if (forced_qpt == 1 || (forced_qpt == 2 && cfg.kbucket <= 32 && !cosine))
    qpt = forced_qpt;
  (void)m;
  cfg.queries_per_lane = qpt;
  cfg.tile_queries = kBlock * qpt;
  // Euclidean lists of up to 32 entries: pre-filter on the matrix cores
  // (longer lists were tried there too: three to four times slower than the
  // vector-ALU kernel, whose queues hold single candidates)
  cfg.matrix_cores = !cosine && cfg.kbucket <= 32 &&
                     env_int("PCA_KNN_LOWD_MATRIX_CORES", 1) != 0;
  if (cfg.matrix_cores) {
    cfg.queries_per_lane = 1;
    cfg.tile_queries = kMcQueries;
  }

  // Slices of x per segment: enough work items (~32 per CU) to even out
  // ragged segments, but slices of at least ~4 LDS tiles on average -- every
  // slice pays the start-up phase of its candidate lists again.
  const int tiles = plan_upper_bound(m, num_segments, cfg.tile_queries);
  // (about 6,000 items for the matrix-core kernel, whose workgroups hold
  // half as many queries.  On 8 scans of 60,000-200,000 points 2, 3 and 4
  // slices run equally fast -- 2.77 / 2.76 / 2.77 ms; 2.83 / 2.87 / 2.94 ms with
  // 5 / 6 / 8 --, but with 2 the slices outgrow the L2s: 443 MB read + 119 MB
  // written per launch against 312 + 175 MB with 4)
  const int target = cfg.matrix_cores ? 6144 : 8192;
  const int want = (target + tiles - 1) / tiles;
  const int by_length = (n / num_segments) / (4 * kLowdTileX);
  int chunks = std::max(1, std::min(std::min(want, 16), by_length));
  const int forced_chunks = env_int("PCA_KNN_SLICES", 0);
  if (forced_chunks >= 1 && forced_chunks <= 64)
    chunks = forced_chunks;
  cfg.num_chunks = chunks;
  cfg.nearest = false;
  return cfg;
}

KnnLowdConfig nearest_lowd_config(int d, int n, int m, int num_segments) {
  // the slices of a one-neighbour kNN search on the matrix cores
  KnnLowdConfig cfg = knn_lowd_config(d, 1, n, m, num_segments, false);
  if (!cfg.matrix_cores) {
    cfg.matrix_cores = true; // the only kernel with the `nearest` rules
    cfg.queries_per_lane = 1;
    cfg.tile_queries = kMcQueries;
  }
  cfg.kbucket = 1;
  cfg.nearest = true;
  return cfg;
}

// packed operand rows of the matrix-core kernel
size_t mc_split_bytes(const KnnLowdConfig &cfg, int n, int d) {
  if (!cfg.matrix_cores)
    return 0;
  const int dim = padded_dim(d);
  // McShape<dim>::REC: operand quads + coordinate quads
  const int per_row = (dim + 1 + 3) / 4 + (dim <= 4 ? 1 : 2);
  return align256(sizeof(uint4) * (size_t)n * per_row);
}

// shared bounds [m]
size_t lowd_bounds_bytes(int m) {
  return align256(sizeof(float) * (size_t)m);
}

size_t knn_lowd_scratch_bytes(const KnnLowdConfig &cfg, int n, int m, int d,
                              int num_segments, int k) {
  size_t bytes = lowd_bounds_bytes(m);
  bytes += mc_split_bytes(cfg, n, d);
  if (cfg.num_chunks > 1) {
    const size_t tiles = plan_upper_bound(m, num_segments, cfg.tile_queries);
    bytes += align256(sizeof(double) * tiles * cfg.num_chunks * (size_t)k *
                      cfg.tile_queries);
  }
  return bytes;
}

// One launch of knn_lowd_kernel for the padded dimension and metric.
hipError_t launch_lowd_pass(const KnnLowdParams &p, const KnnLowdConfig &cfg,
                            int dim, bool cosine, int tiles_bound,
                            hipStream_t stream) {
  if (cfg.matrix_cores) {
    const int grid = tiles_bound * p.num_chunks;
    switch (dim) {
    case 2:
      return launch_knn_lowd_mc_dim<2>(p, cfg.kbucket, grid, stream);
    case 3:
      return launch_knn_lowd_mc_dim<3>(p, cfg.kbucket, grid, stream);
    case 4:
      return launch_knn_lowd_mc_dim<4>(p, cfg.kbucket, grid, stream);
    case 8:
      return launch_knn_lowd_mc_dim<8>(p, cfg.kbucket, grid, stream);
    }
    return hipErrorInvalidValue;
  }
#define PCA_DIM_CASE(D)                                                        \
  case D:                                                                      \
    return cosine ? launch_knn_lowd_dim<D, true>(p, cfg, tiles_bound, stream)  \
                  : launch_knn_lowd_dim<D, false>(p, cfg, tiles_bound,         \
                                                  stream);
  switch (dim) {
    PCA_DIM_CASE(2)
    PCA_DIM_CASE(3)
    PCA_DIM_CASE(4)
    PCA_DIM_CASE(8)
  }
#undef PCA_DIM_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_knn_lowd(const SearchInput &in, int k, bool cosine,
                           const KnnLowdConfig &cfg, int *work_start,
                           void *scratch, const DenseResult &out,
                           hipEvent_t time_start, hipEvent_t time_stop,
                           hipStream_t stream, int64_t *nearest_out,
                           const SegmentSource *src) {
  const int tiles_bound =
      plan_upper_bound(in.m, in.num_segments, cfg.tile_queries);
  KnnLowdParams p;
  p.x = static_cast<const float *>(in.x);
  p.y = static_cast<const float *>(in.y);
  p.ptr_x = in.ptr_x;
  p.ptr_y = in.ptr_y;
  p.n = in.n;
  p.m = in.m;
  p.d_in = in.d;
  p.num_segments = in.num_segments;
  p.k = k;
  p.work_start = work_start;
  p.num_chunks = cfg.num_chunks;
  p.tau = nullptr;
  p.partial = nullptr;
  p.out_idx = out.idx;
  p.out_dist = out.dist;
  p.out_count = out.count;
  p.out_nearest = nearest_out;
  p.x_split = nullptr;
  char *base = static_cast<char *>(scratch);
  const size_t tau_bytes = lowd_bounds_bytes(in.m);
  // tiles between two exchanges of bounds among the slices of a query
  // (a power of two; PCA_KNN_SYNC_PERIOD overrides)
  int period = env_int("PCA_KNN_SYNC_PERIOD", 4);
  if (period < 1 || period > 64 || (period & (period - 1)) != 0)
    period = 4;
  p.sync_mask = period - 1;
  const size_t split_bytes = mc_split_bytes(cfg, in.n, in.d);
  if (cfg.num_chunks > 1) {
    p.tau = reinterpret_cast<float *>(base);
    p.partial = reinterpret_cast<double *>(base + tau_bytes + split_bytes);
  }
  const float tau_start = cfg.nearest ? kNearestLimit : kKnnSentinel;
  if (cfg.matrix_cores) {
    // one launch: pointers (when the caller passed example ids), plan, packed
    // rows, start value of the shared bounds
    uint4 *split = reinterpret_cast<uint4 *>(base + tau_bytes);
    p.x_split = split;
    // (only this set-up clears the compaction's block sums: the other path
    // leaves the counting to the compaction)
    p.edge_sums = nearest_out ? nullptr : out.edge_sums;
    p.self_pos = out.self_pos;
    p.kept = out.kept;
    McSetup a;
    a.edge_sums = p.edge_sums;
    a.edge_blocks =
        (in.m + kCompactBlockQueries - 1) / kCompactBlockQueries + 1;
    a.x = p.x;
    a.n = in.n;
    a.d_in = in.d;
    a.out = split;
    a.tau = p.tau;
    a.m = in.m;
    a.tau_value = tau_start;
    a.ptr_y = in.ptr_y;
    a.num_segments = in.num_segments;
    a.per_item = cfg.tile_queries;
    a.work_start = work_start;
    if (src)
      a.src = *src;
    hipError_t perr = hipErrorInvalidValue;
    switch (padded_dim(in.d)) {
    case 2:
      perr = launch_mc_setup<2>(a, stream);
      break;
    case 3:
      perr = launch_mc_setup<3>(a, stream);
      break;
    case 4:
      perr = launch_mc_setup<4>(a, stream);
      break;
    case 8:
      perr = launch_mc_setup<8>(a, stream);
      break;
    }
    if (perr != hipSuccess)
      return perr;
  } else {
    const hipError_t perr =
        launch_plan(in.ptr_y, in.m, in.num_segments, cfg.tile_queries,
                    work_start, stream, src);
    if (perr != hipSuccess)
      return perr;
    if (cfg.num_chunks > 1)
      hipLaunchKernelGGL(fill_f32_kernel, dim3((in.m + kBlock - 1) / kBlock),
                         dim3(kBlock), 0, stream, p.tau, in.m, tau_start);
  }

  if (time_start)
    (void)hipEventRecord(time_start, stream);
  const hipError_t err = launch_lowd_pass(p, cfg, padded_dim(in.d), cosine,
                                          tiles_bound, stream);
  if (err != hipSuccess)
    return err;
  if (time_stop)
    (void)hipEventRecord(time_stop, stream);
  if (cfg.num_chunks <= 1)
    return err;

  switch (cfg.kbucket) {
  case 1:
    hipLaunchKernelGGL((knn_merge_kernel<1, kMcQueries, true>),
                       dim3(tiles_bound), dim3(kBlock), 0, stream, p);
    break;
  case 8:
    launch_merge<8>(p, cfg.tile_queries, tiles_bound, stream);
    break;
  case 16:
    launch_merge<16>(p, cfg.tile_queries, tiles_bound, stream);
    break;
  case 24:
    launch_merge<24>(p, cfg.tile_queries, tiles_bound, stream);
    break;
  case 32:
    launch_merge<32>(p, cfg.tile_queries, tiles_bound, stream);
    break;
  case 48:
    launch_merge<48>(p, cfg.tile_queries, tiles_bound, stream);
    break;
  case 64:
    launch_merge<64>(p, cfg.tile_queries, tiles_bound, stream);
    break;
  case 100:
    launch_merge<100>(p, cfg.tile_queries, tiles_bound, stream);
    break;
  default:
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

int knn_generic_slices(int n, int m, int num_segments) {
  // enough work items for four workgroups per CU, slices of at least 16 LDS
  // tiles on average
  const int tiles = plan_upper_bound(m, num_segments, kBlock);
  const int want = (1024 + tiles - 1) / tiles;
  const int by_length = (n / num_segments) / (16 * kGenTile);
  int chunks = std::max(1, std::min(std::min(want, 64), by_length));
  const int forced = env_int("PCA_KNN_SLICES", 0);
  if (forced >= 1 && forced <= 64)
    chunks = forced;
  return chunks;
}

size_t knn_generic_scratch_bytes(int n, int m, int num_segments, int k) {
  const int chunks = knn_generic_slices(n, m, num_segments);
  if (chunks <= 1)
    return 0;
  const size_t tiles = plan_upper_bound(m, num_segments, kBlock);
  return align256(sizeof(double) * tiles * chunks * (size_t)k * kBlock);
}

hipError_t launch_knn_generic(const SearchInput &in, int k, bool cosine,
                              const float *x_norm, const int *work_start,
                              int grid_bound, const DenseResult &out,
                              hipStream_t stream, void *scratch,
                              const int *gate, const int *redo_q) {
  const int kb = k_bucket(k);
  const int chunks =
      scratch ? knn_generic_slices(in.n, in.m, in.num_segments) : 1;
  double *partial = static_cast<double *>(scratch);
  const hipError_t err =
      cosine ? launch_knn_generic_metric<true>(in, k, kb, x_norm, work_start,
                                               grid_bound, out, stream, gate,
                                               redo_q, chunks, partial)
             : launch_knn_generic_metric<false>(in, k, kb, x_norm, work_start,
                                                grid_bound, out, stream, gate,
                                                redo_q, chunks, partial);
  if (err != hipSuccess || chunks <= 1)
    return err;
  // the slices' lists -> dense results
  KnnLowdParams p;
  p.x = static_cast<const float *>(in.x);
  p.y = static_cast<const float *>(in.y);
  p.ptr_x = in.ptr_x;
  p.ptr_y = in.ptr_y;
  p.n = in.n;
  p.m = in.m;
  p.d_in = in.d;
  p.num_segments = in.num_segments;
  p.k = k;
  p.work_start = work_start;
  p.num_chunks = chunks;
  p.tau = nullptr;
  p.partial = partial;
  p.out_idx = out.idx;
  p.out_dist = out.dist;
  p.out_count = out.count;
  p.out_nearest = nullptr;
  p.x_split = nullptr;
  p.gate = gate;
  p.redo_q = redo_q;
  switch (kb) {
  case 8:
    launch_merge<8>(p, kBlock, grid_bound, stream);
    break;
  case 16:
    launch_merge<16>(p, kBlock, grid_bound, stream);
    break;
  case 24:
    launch_merge<24>(p, kBlock, grid_bound, stream);
    break;
  case 32:
    launch_merge<32>(p, kBlock, grid_bound, stream);
    break;
  case 48:
    launch_merge<48>(p, kBlock, grid_bound, stream);
    break;
  case 64:
    launch_merge<64>(p, kBlock, grid_bound, stream);
    break;
  case 100:
    launch_merge<100>(p, kBlock, grid_bound, stream);
    break;
  default:
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

} // namespace pca
