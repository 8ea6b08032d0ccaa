// Dispatch of the matrix-core radius search (see radius_mc_impl.hpp).
#include "radius_mc_impl.hpp"

#include <cstdlib>

namespace pca {

namespace {

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

int padded_dim(int d) {
  if (d <= 2)
    return 2;
  if (d <= 4)
    return d;
  return 8;
}

template <int DIM>
hipError_t launch_dim(RadiusMcParams p, const float *x, uint4 *packed,
                      int grid, hipStream_t stream) {
  hipLaunchKernelGGL((mc_pack_rows_kernel<DIM>),
                     dim3((p.n + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     stream, x, p.n, p.d_in, packed);
  hipLaunchKernelGGL((radius_mc_kernel<DIM>), dim3(grid), dim3(kBlock), 0,
                     stream, p);
  return hipGetLastError();
}

} // namespace

bool radius_mc_supported(int d, int n, int m, int num_segments) {
  if (d < 1 || d > 8)
    return false;
  // PCA_RADIUS_MATRIX_CORES=0 / 1 switches the path off / on regardless of
  // the problem size (tests use it)
  if (const char *env = std::getenv("PCA_RADIUS_MATRIX_CORES")) {
    if (env[0] == '0')
      return false;
    if (env[0] == '1')
      return true;
  }
  // one workgroup per 128 queries scans a whole segment; measured faster
  // than the wave-per-query kernel of radius.hip from 128 workgroups on
  // (half a workgroup per CU), the small problems below stay there
  (void)n;
  return plan_upper_bound(m, num_segments, kRadiusMcTileQueries) >= 64;
}

size_t radius_mc_scratch_bytes(int n, int d) {
  const int dim = padded_dim(d);
  const int per_row = (dim + 1 + 3) / 4 + (dim <= 4 ? 1 : 2); // McShape::REC
  return align256(sizeof(uint4) * (size_t)n * per_row);
}

hipError_t launch_radius_mc(const SearchInput &in, float r2,
                            bool ignore_same_index, const int *work_start,
                            int tiles_bound, void *scratch,
                            const DenseResult &out, hipStream_t stream) {
  if (tiles_bound <= 0)
    return hipSuccess;
  RadiusMcParams p;
  p.y = static_cast<const float *>(in.y);
  p.ptr_x = in.ptr_x;
  p.ptr_y = in.ptr_y;
  p.x_split = static_cast<const uint4 *>(scratch);
  p.n = in.n;
  p.m = in.m;
  p.d_in = in.d;
  p.num_segments = in.num_segments;
  p.r2 = r2;
  p.slots = out.slots;
  p.ignore_same_index = ignore_same_index ? 1 : 0;
  p.work_start = work_start;
  p.out_idx = out.idx;
  p.out_count = out.count;
  const float *x = static_cast<const float *>(in.x);
  uint4 *packed = static_cast<uint4 *>(scratch);
  switch (padded_dim(in.d)) {
  case 2:
    return launch_dim<2>(p, x, packed, tiles_bound, stream);
  case 3:
    return launch_dim<3>(p, x, packed, tiles_bound, stream);
  case 4:
    return launch_dim<4>(p, x, packed, tiles_bound, stream);
  case 8:
    return launch_dim<8>(p, x, packed, tiles_bound, stream);
  }
  return hipErrorInvalidValue;
}

} // namespace pca
