// Low-dimensional kNN with the pre-filter on the matrix cores: Euclidean
// distance, 3 components per point.
#include "knn_lowd_mc_impl.hpp"

namespace pca {
PCA_LOWD_MC_DEFINE(3)
} // namespace pca

#ifdef PCA_MC_STATS
// (instrumented builds only) reads and clears the counters
extern "C" int pca_mc_stats(unsigned long long *out) {
  unsigned long long zero[8] = {0};
  if (hipMemcpyFromSymbol(out, HIP_SYMBOL(pca::g_mc_stats), sizeof(zero)) !=
      hipSuccess)
    return -1;
  return hipMemcpyToSymbol(HIP_SYMBOL(pca::g_mc_stats), zero, sizeof(zero)) ==
                 hipSuccess
             ? 0
             : -1;
}
#endif
