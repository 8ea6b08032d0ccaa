// Any-dimension kNN kernels, cosine distance.
#include "knn_generic_impl.hpp"

namespace pca {
PCA_GENERIC_DEFINE(true)

// |row| = sqrt(sum of squares accumulated with one FMA per component in
// ascending order), as Cosine::norm in the reference computes it.
__global__ __launch_bounds__(kBlock) void row_norm_kernel(
    const float *__restrict__ x, int n, int d, float *__restrict__ norm) {
  const int row = blockIdx.x * kBlock + threadIdx.x;
  if (row >= n)
    return;
  const float *p = x + (size_t)row * d;
  float s = 0.0f;
  for (int c = 0; c < d; ++c)
    s = __builtin_fmaf(p[c], p[c], s);
  norm[row] = __builtin_sqrtf(s);
}


hipError_t launch_row_norms(const float *x, int n, int d, float *norm,
                            hipStream_t stream) {
  const int grid = (n + kBlock - 1) / kBlock;
  hipLaunchKernelGGL(row_norm_kernel, dim3(grid), dim3(kBlock), 0, stream, x,
                     n, d, norm);
  return hipGetLastError();
}
} // namespace pca
