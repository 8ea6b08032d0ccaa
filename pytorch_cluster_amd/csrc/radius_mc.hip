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

// Two launches: the preparation (segment pointers from example ids when src
// is used, the plan, the packed rows) and the search.
template <int DIM>
hipError_t launch_dim(RadiusMcParams p, const McSetup &setup, int grid,
                      hipEvent_t time_start, hipStream_t stream) {
  const int rows = setup.n > setup.m ? setup.n : setup.m;
  hipLaunchKernelGGL((mc_setup_kernel<DIM>),
                     dim3((rows + kPlanThreads - 1) / kPlanThreads),
                     dim3(kPlanThreads), 0, stream, setup);
  if (time_start)
    (void)hipEventRecord(time_start, stream);
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
                            bool ignore_same_index, int *work_start,
                            int tiles_bound, void *scratch,
                            const DenseResult &out, hipEvent_t time_start,
                            hipStream_t stream, const SegmentSource *src) {
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
  p.edge_sums = out.edge_sums;
  McSetup a;
  a.edge_sums = out.edge_sums;
  a.edge_blocks = (in.m + kCompactBlockQueries - 1) / kCompactBlockQueries + 1;
  a.x = static_cast<const float *>(in.x);
  a.n = in.n;
  a.d_in = in.d;
  a.out = static_cast<uint4 *>(scratch);
  a.tau = nullptr;
  a.m = in.m;
  a.tau_value = 0.0f;
  a.ptr_y = in.ptr_y;
  a.num_segments = in.num_segments;
  a.per_item = kRadiusMcTileQueries;
  a.work_start = work_start;
  if (src)
    a.src = *src;
  switch (padded_dim(in.d)) {
  case 2:
    return launch_dim<2>(p, a, tiles_bound, time_start, stream);
  case 3:
    return launch_dim<3>(p, a, tiles_bound, time_start, stream);
  case 4:
    return launch_dim<4>(p, a, tiles_bound, time_start, stream);
  case 8:
    return launch_dim<8>(p, a, tiles_bound, time_start, stream);
  }
  return hipErrorInvalidValue;
}

} // namespace pca
