// Any-dimension kNN kernels, squared Euclidean distance.
#include "knn_generic_impl.hpp"

namespace pca {
PCA_GENERIC_DEFINE(false)
} // namespace pca
