// Matrix-core kNN kernels for up to 32 components per point.
#include "knn_mfma_impl.hpp"

namespace pca {

template <int STEPS>
hipError_t launch_knn_mfma_steps(const KnnMfmaParams &p, int kbucket,
                                 int grid, hipStream_t stream);

template <>
hipError_t launch_knn_mfma_steps<16>(const KnnMfmaParams &p, int kbucket,
                                     int grid, hipStream_t stream) {
  switch (kbucket) {
  case 8:
    hipLaunchKernelGGL((knn_mfma_kernel<16, 8>), dim3(grid), dim3(kBlock), 0,
                       stream, p);
    break;
  case 16:
    hipLaunchKernelGGL((knn_mfma_kernel<16, 16>), dim3(grid), dim3(kBlock), 0,
                       stream, p);
    break;
  case 24:
    hipLaunchKernelGGL((knn_mfma_kernel<16, 24>), dim3(grid), dim3(kBlock), 0,
                       stream, p);
    break;
  case 32:
    hipLaunchKernelGGL((knn_mfma_kernel<16, 32>), dim3(grid), dim3(kBlock), 0,
                       stream, p);
    break;
  default:
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

} // namespace pca
