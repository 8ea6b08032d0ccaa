// Feature-space kNN kernels (fp16 filter) for points of up to 256 components
// (17 blocks of 16: the coordinates and one block that carries the norms).
#include "knn_feat_impl.hpp"

namespace pca {

PCA_KNN_FEAT_DEFINE(17)

} // namespace pca
