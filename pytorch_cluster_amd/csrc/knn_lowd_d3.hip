// Low-dimensional kNN kernels: Euclidean distance, 3 components per point.
#include "knn_lowd_impl.hpp"

namespace pca {
PCA_LOWD_DEFINE_SLICE(3, false)
} // namespace pca
