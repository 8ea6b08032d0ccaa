// Feature-space radius search in one kernel: 5 blocks of 16 components (up to 64 features),
// bf16 rows.
#include "knn_feat_small_impl.hpp"

namespace pca {
PCA_RADIUS_FEAT_DEFINE(5, 2)
} // namespace pca
