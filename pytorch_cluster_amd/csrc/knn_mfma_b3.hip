// Matrix-core kNN kernels for points of up to 32 components (3 blocks
// of 16: the coordinates and one block of augmented components).
#include "knn_mfma_impl.hpp"

namespace pca {

template <int NB>
hipError_t launch_knn_mfma_blocks(const KnnMfmaParams &p, int kbucket,
                                  bool cosine, int grid, hipStream_t stream);
template <int NB>
hipError_t launch_mfma_pack_rows(const float *x, const float *norms, int n,
                                 int d, bool cosine, uint4 *out,
                                 hipStream_t stream, const int *gate);

PCA_KNN_MFMA_DEFINE(3)

} // namespace pca
