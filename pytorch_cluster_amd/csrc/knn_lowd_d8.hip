// Low-dimensional kNN kernels: Euclidean distance, 8 components per point.
#include "knn_lowd_impl.hpp"

namespace pca {
PCA_LOWD_DEFINE_SLICE(8, false)
} // namespace pca
