// Matrix-core kNN kernels for up to 64 components per point.
#include "knn_mfma_impl.hpp"

namespace pca {

template <int STEPS>
hipError_t launch_knn_mfma_steps(const KnnMfmaParams &p, int kbucket,
                                 int grid, hipStream_t stream);

template <>
hipError_t launch_knn_mfma_steps<32>(const KnnMfmaParams &p, int kbucket,
                                     int grid, hipStream_t stream) {
  switch (kbucket) {
  case 8:
    hipLaunchKernelGGL((knn_mfma_kernel<32, 8>), dim3(grid), dim3(kBlock), 0,
                       stream, p);
    break;
  case 16:
    hipLaunchKernelGGL((knn_mfma_kernel<32, 16>), dim3(grid), dim3(kBlock), 0,
                       stream, p);
    break;
  case 24:
    hipLaunchKernelGGL((knn_mfma_kernel<32, 24>), dim3(grid), dim3(kBlock), 0,
                       stream, p);
    break;
  case 32:
    hipLaunchKernelGGL((knn_mfma_kernel<32, 32>), dim3(grid), dim3(kBlock), 0,
                       stream, p);
    break;
  default:
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

} // namespace pca
