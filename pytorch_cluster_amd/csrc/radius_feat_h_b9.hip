// Feature-space radius search in one kernel: 9 blocks of 16 components (up to 128 features),
// fp16 rows.
#include "knn_feat_small_impl.hpp"

namespace pca {
PCA_RADIUS_FEAT_DEFINE(9, 1)
} // namespace pca
