// Feature-space kNN of small examples in one exact kernel: 9 blocks of 16
// components (up to 128 features).
#include "knn_feat_small_impl.hpp"

namespace pca {
PCA_KNN_FEAT_SMALL_DEFINE(9)
} // namespace pca
