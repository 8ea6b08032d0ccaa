// Low-dimensional kNN kernels: cosine distance, 4 components per point.
#include "knn_lowd_impl.hpp"

namespace pca {
PCA_LOWD_DEFINE_SLICE(4, true)
} // namespace pca
