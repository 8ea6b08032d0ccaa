// Feature-space radius search in one kernel: 9 blocks of 16 components (up to 128 features),
// fp32 rows.
#include "knn_feat_small_impl.hpp"

namespace pca {
PCA_RADIUS_FEAT_DEFINE(9, 0)
} // namespace pca
