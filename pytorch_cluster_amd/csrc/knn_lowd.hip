// Dispatch of the low-dimensional kNN kernels (see knn_lowd_impl.hpp).
#include "knn_generic_impl.hpp"
#include "knn_lowd_impl.hpp"

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

} // namespace

bool knn_lowd_supported(int d, int k, bool /*cosine*/) {
  return d >= 1 && d <= 8 && k >= 1 && k <= 100;
}

KnnLowdConfig knn_lowd_config(int /*d*/, int k, int m) {
  KnnLowdConfig cfg;
  cfg.kbucket = k_bucket(k);
  // Two queries per lane halve the LDS reads per distance but need twice the
  // queries to fill the 256 CUs; worth it once there are enough query tiles.
  int qpt = (cfg.kbucket <= 32 && m >= 2 * kBlock * 256) ? 2 : 1;
  if (const char *env = std::getenv("PCA_KNN_QUERIES_PER_LANE")) {
    const int v = std::atoi(env);
    if ((v == 1 || v == 2) && (v == 1 || cfg.kbucket <= 32))
      qpt = v;
  }
  cfg.queries_per_lane = qpt;
  cfg.tile_queries = kBlock * qpt;
  return cfg;
}

hipError_t launch_knn_lowd(const SearchInput &in, int k, bool cosine,
                           const KnnLowdConfig &cfg, const int *work_start,
                           int grid_bound, const DenseResult &out,
                           hipStream_t stream) {
  KnnLowdConfig c = cfg;
  if (cosine) {
    c.queries_per_lane = 1;
  }
#define PCA_DIM_CASE(D)                                                        \
  case D:                                                                      \
    return cosine ? launch_knn_lowd_dim<D, true>(in, k, c, work_start,         \
                                                 grid_bound, out, stream)      \
                  : launch_knn_lowd_dim<D, false>(in, k, c, work_start,        \
                                                  grid_bound, out, stream);
  switch (padded_dim(in.d)) {
    PCA_DIM_CASE(2)
    PCA_DIM_CASE(3)
    PCA_DIM_CASE(4)
    PCA_DIM_CASE(8)
  }
#undef PCA_DIM_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_knn_generic(const SearchInput &in, int k, bool cosine,
                              const float *x_norm, const int *work_start,
                              int grid_bound, const DenseResult &out,
                              hipStream_t stream) {
  const int kb = k_bucket(k);
  return cosine ? launch_knn_generic_metric<true>(in, k, kb, x_norm,
                                                  work_start, grid_bound, out,
                                                  stream)
                : launch_knn_generic_metric<false>(in, k, kb, x_norm,
                                                   work_start, grid_bound, out,
                                                   stream);
}

} // namespace pca
