// Low-dimensional kNN with the pre-filter on the matrix cores: Euclidean
// distance, 8 components per point.
#include "knn_lowd_mc_impl.hpp"

namespace pca {
PCA_LOWD_MC_DEFINE(8)
} // namespace pca
