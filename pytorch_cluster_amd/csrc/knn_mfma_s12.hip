// Matrix-core kNN kernels for up to 22 components per point.
#include "knn_mfma_impl.hpp"

namespace pca {

template <int STEPS>
hipError_t launch_knn_mfma_steps(const KnnMfmaParams &p, int kbucket,
                                 bool cosine, int grid, hipStream_t stream);

template <int STEPS, int KB>
void launch_one(const KnnMfmaParams &p, bool cosine, int grid,
                hipStream_t stream) {
  if (cosine)
    hipLaunchKernelGGL((knn_mfma_kernel<STEPS, KB, true>), dim3(grid),
                       dim3(kBlock), 0, stream, p);
  else
    hipLaunchKernelGGL((knn_mfma_kernel<STEPS, KB, false>), dim3(grid),
                       dim3(kBlock), 0, stream, p);
}

template <>
hipError_t launch_knn_mfma_steps<12>(const KnnMfmaParams &p, int kbucket,
                                     bool cosine, int grid,
                                     hipStream_t stream) {
  switch (kbucket) {
  case 8:
    launch_one<12, 8>(p, cosine, grid, stream);
    break;
  case 16:
    launch_one<12, 16>(p, cosine, grid, stream);
    break;
  case 24:
    launch_one<12, 24>(p, cosine, grid, stream);
    break;
  case 32:
    launch_one<12, 32>(p, cosine, grid, stream);
    break;
  default:
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

} // namespace pca
