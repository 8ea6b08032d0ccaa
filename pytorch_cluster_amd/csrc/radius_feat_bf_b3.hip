// Feature-space radius search in one kernel: 3 blocks of 16 components (up to 32 features),
// bf16 rows.
#include "knn_feat_small_impl.hpp"

namespace pca {
PCA_RADIUS_FEAT_DEFINE(3, 2)
} // namespace pca
