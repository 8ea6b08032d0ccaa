// Feature-space kNN kernels (fp16 filter) for points of up to 512 components
// (33 blocks of 16: the coordinates and one block that carries the norms).
#include "knn_feat_impl.hpp"

namespace pca {

PCA_KNN_FEAT_DEFINE(33)

} // namespace pca
