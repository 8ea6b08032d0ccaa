// Feature-space kNN, eight-wave first stage (fp16 filter with the cut inside
// the matrix product) for points of up to 128 components.
#include "knn_feat_wide_impl.hpp"

namespace pca {

PCA_KNN_FEAT_WIDE_DEFINE(9)

} // namespace pca
