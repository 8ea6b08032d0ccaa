// Low-dimensional kNN kernels: cosine distance, 2 components per point.
#include "knn_lowd_impl.hpp"

namespace pca {
PCA_LOWD_DEFINE_SLICE(2, true)
} // namespace pca
