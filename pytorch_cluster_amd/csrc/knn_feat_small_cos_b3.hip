// Feature-space kNN of moderate examples in one exact kernel: 3 blocks of 16 components (up to 32 features),
// cosine distance of fp32 rows.
#include "knn_feat_small_impl.hpp"

namespace pca {
PCA_KNN_FEAT_SMALL_DEFINE(3, 3)
} // namespace pca
