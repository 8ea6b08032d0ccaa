// Feature-space kNN of small examples in one exact kernel: 3 blocks of 16
// components (up to 32 features).
#include "knn_feat_small_impl.hpp"

namespace pca {
PCA_KNN_FEAT_SMALL_DEFINE(3)
} // namespace pca
