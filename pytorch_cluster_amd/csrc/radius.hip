// Fixed-radius neighbour search for fp32 points on gfx950.
//
// Computes what radius_kernel of the reference computes
// (csrc/cuda/radius_cuda.cu:9-42: one thread per query scans its segment of x
// in ascending row order, keeps the first max_num_neighbors rows with
// dist < r^2, stops as soon as it has them), with a different machine
// mapping chosen for the early exit:
//
//   * a WAVE, not a lane, owns a query: the 64 lanes take 64 consecutive x
//     rows, compute their distances to the query, and the hits are compacted
//     with a wavefront ballot + mbcnt prefix count into the query's slot row,
//     in ascending x row order by construction;
//   * the stop test (count >= max_num_neighbors) is wave-uniform, so a query
//     that has its neighbours costs nothing more -- no lane waits for the
//     slowest of 64 unrelated queries;
//   * each wave carries QW queries of one segment at once: the 64 candidate
//     rows are loaded once (coalesced) and reused for every query still open,
//     the queries' coordinates are wave-uniform (scalar registers).
//
// Distances are direct differences with one fused multiply-add per dimension
// in ascending dimension order, as in the kNN kernels.
#include "device_utils.hpp"
#include "launchers.hpp"

namespace pca {

namespace {

constexpr int QW = kRadiusQueriesPerWave;
constexpr int kWavesPerBlock = kBlock / kWave;

__device__ __forceinline__ int lane_prefix_count(uint64_t mask) {
  // number of set bits of `mask` below this lane
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
}

// DIM > 0: compile-time number of components; DIM == 0: runtime d.
template <int DIM>
__global__ __launch_bounds__(kBlock) void radius_kernel(
    const float *__restrict__ x, const float *__restrict__ y,
    const int64_t *__restrict__ ptr_x, const int64_t *__restrict__ ptr_y,
    int n, int m, int d_rt, int num_segments, float r2, int slots,
    int ignore_same_index, const int *__restrict__ work_start,
    int *__restrict__ out_idx, int *__restrict__ out_count) {
  const int lane = threadIdx.x & (kWave - 1);
  // wave-uniform by construction; readfirstlane lets the compiler keep the
  // bookkeeping in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int task = blockIdx.x * kWavesPerBlock + wave;
  if (task >= work_start[num_segments])
    return;
  const int d = DIM > 0 ? DIM : d_rt;
  const int seg = find_segment(work_start, num_segments, task);
  const int x_begin = ptr_x ? (int)ptr_x[seg] : 0;
  const int x_end = ptr_x ? (int)ptr_x[seg + 1] : n;
  const int y_begin = ptr_y ? (int)ptr_y[seg] : 0;
  const int y_end = ptr_y ? (int)ptr_y[seg + 1] : m;
  const int q0 = y_begin + (task - work_start[seg]) * QW;
  const int nq = min(QW, y_end - q0);

  int count[QW];
  bool open[QW];
#pragma unroll
  for (int qi = 0; qi < QW; ++qi) {
    count[qi] = 0;
    open[qi] = qi < nq;
  }
  int num_open = nq;

  for (int base = x_begin; base < x_end && num_open > 0; base += kWave) {
    const int row = base + lane;
    const bool in_range = row < x_end;

    float acc[QW];
    if (DIM > 0) {
      float cx[DIM > 0 ? DIM : 1];
#pragma unroll
      for (int c = 0; c < DIM; ++c)
        cx[c] = in_range ? x[(size_t)row * DIM + c] : __builtin_inff();
#pragma unroll
      for (int qi = 0; qi < QW; ++qi) {
        if (!open[qi])
          continue;
        const float *yq = y + (size_t)(q0 + qi) * DIM;
        const float d0 = cx[0] - yq[0];
        float a = d0 * d0;
#pragma unroll
        for (int c = 1; c < DIM; ++c) {
          const float dc = cx[c] - yq[c];
          a = __builtin_fmaf(dc, dc, a);
        }
        acc[qi] = a;
      }
    } else {
#pragma unroll
      for (int qi = 0; qi < QW; ++qi)
        acc[qi] = 0.0f;
      for (int c = 0; c < d; ++c) {
        const float xv = in_range ? x[(size_t)row * d + c] : __builtin_inff();
#pragma unroll
        for (int qi = 0; qi < QW; ++qi) {
          if (!open[qi])
            continue;
          const float dc = xv - y[(size_t)(q0 + qi) * d + c];
          acc[qi] = __builtin_fmaf(dc, dc, acc[qi]);
        }
      }
    }

#pragma unroll
    for (int qi = 0; qi < QW; ++qi) {
      if (!open[qi])
        continue;
      const int q = q0 + qi;
      // rows past the segment end are +inf: inf or NaN, never < r2
      bool hit = acc[qi] < r2;
      if (ignore_same_index)
        hit = hit && row != q;
      const uint64_t mask = __ballot(hit);
      if (mask != 0) {
        const int pos = count[qi] + lane_prefix_count(mask);
        if (hit && pos < slots)
          out_idx[(size_t)q * slots + pos] = row;
        count[qi] += __builtin_popcountll(mask);
        if (count[qi] >= slots) {
          open[qi] = false;
          --num_open;
        }
      }
    }
  }

  if (lane < nq) {
    int c = 0;
#pragma unroll
    for (int qi = 0; qi < QW; ++qi)
      if (lane == qi)
        c = min(count[qi], slots);
    out_count[q0 + lane] = c;
  }
}

} // namespace

hipError_t launch_radius(const SearchInput &in, float r2,
                         bool ignore_same_index, const int *work_start,
                         int task_bound, const DenseResult &out,
                         hipStream_t stream) {
  const int grid = (task_bound + kWavesPerBlock - 1) / kWavesPerBlock;
  if (grid <= 0)
    return hipSuccess;
#define PCA_RADIUS_LAUNCH(DIM)                                                 \
  hipLaunchKernelGGL((radius_kernel<DIM>), dim3(grid), dim3(kBlock), 0,        \
                     stream, (const float *)in.x, (const float *)in.y,         \
                     in.ptr_x, in.ptr_y, in.n, in.m, in.d, in.num_segments,    \
                     r2, out.slots, ignore_same_index ? 1 : 0, work_start,     \
                     out.idx, out.count)
  switch (in.d) {
  case 1:
    PCA_RADIUS_LAUNCH(1);
    break;
  case 2:
    PCA_RADIUS_LAUNCH(2);
    break;
  case 3:
    PCA_RADIUS_LAUNCH(3);
    break;
  case 4:
    PCA_RADIUS_LAUNCH(4);
    break;
  default:
    PCA_RADIUS_LAUNCH(0);
    break;
  }
#undef PCA_RADIUS_LAUNCH
  return hipGetLastError();
}

} // namespace pca
