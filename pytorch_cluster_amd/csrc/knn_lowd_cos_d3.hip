// Low-dimensional kNN kernels: cosine distance, 3 components per point.
#include "knn_lowd_impl.hpp"

namespace pca {
PCA_LOWD_DEFINE_SLICE(3, true)
} // namespace pca
