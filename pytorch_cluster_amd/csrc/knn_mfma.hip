// Dispatch of the matrix-core kNN kernels (see knn_mfma_impl.hpp).
#include "knn_mfma_impl.hpp"

#include <algorithm>
#include <cstdlib>

namespace pca {

// One number of component blocks per translation unit (knn_mfma_b*.hip):
// the search kernels and the kernel that packs the x rows for them.
template <int NB>
hipError_t launch_knn_mfma_blocks(const KnnMfmaParams &p, int kbucket,
                                  bool cosine, int grid, hipStream_t stream);
template <int NB>
hipError_t launch_mfma_pack_rows(const float *x, const float *norms, int n,
                                 int d, bool cosine, uint4 *out,
                                 hipStream_t stream, const int *gate);
#define PCA_DECLARE_BLOCKS(NB)                                                 \
  template <>                                                                  \
  hipError_t launch_knn_mfma_blocks<NB>(const KnnMfmaParams &, int, bool,      \
                                        int, hipStream_t);                     \
  template <>                                                                  \
  hipError_t launch_mfma_pack_rows<NB>(const float *, const float *, int,      \
                                       int, bool, uint4 *, hipStream_t,        \
                                       const int *);
PCA_DECLARE_BLOCKS(2)
PCA_DECLARE_BLOCKS(3)
PCA_DECLARE_BLOCKS(5)
PCA_DECLARE_BLOCKS(9)
#undef PCA_DECLARE_BLOCKS

// csrc/knn_generic_cos.hip
hipError_t launch_row_norms(const float *x, int n, int d, float *norm,
                            hipStream_t stream);

__global__ __launch_bounds__(kBlock) void row_sqnorm_kernel(
    const float *__restrict__ x, int n, int d, float *__restrict__ out) {
  const int row = blockIdx.x * kBlock + threadIdx.x;
  if (row >= n)
    return;
  const float *p = x + (size_t)row * d;
  float s = 0.0f;
  for (int c = 0; c < d; ++c)
    s = __builtin_fmaf(p[c], p[c], s);
  out[row] = s;
}

namespace {

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

int k_bucket(int k) {
  static const int buckets[] = {8, 16, 24, 32, 48, 64};
  for (int b : buckets)
    if (k <= b)
      return b;
  return 0;
}

__global__ __launch_bounds__(kBlock) void fill_tau_kernel(float *p, int n,
                                                          float v) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n)
    p[i] = v;
}

template <int KB>
void launch_mfma_merge(const KnnLowdParams &p, int tiles_bound,
                       hipStream_t stream) {
  hipLaunchKernelGGL((knn_merge_kernel<KB, kMfmaQueries>), dim3(tiles_bound),
                     dim3(kBlock), 0, stream, p);
}

// blocks of 16 components: the coordinates and one augmented block
int mfma_blocks(int d) {
  if (d <= 16)
    return 2;
  if (d <= 32)
    return 3;
  if (d <= 64)
    return 5;
  return 9;
}

size_t mfma_pack_bytes(int n, int d) {
  const int nb = mfma_blocks(d);
  const size_t units = 2 * nb + 2 * (nb - 1) + 1; // MfmaShape<nb>::RSU
  // (one tile of spare rows: the last tile of a slice is read in full)
  return align256(sizeof(uint4) * units * ((size_t)n + kMfmaRows));
}

} // namespace

bool knn_mfma_supported(int d, int k, bool cosine) {
  if (const char *env = std::getenv("PCA_KNN_NO_MFMA"))
    if (env[0] == '1')
      return false;
  (void)cosine;
  return d > 8 && d <= 128 && k >= 1 && k <= 64;
}

int knn_mfma_slices(int n, int m, int num_segments) {
  const int tiles = plan_upper_bound(m, num_segments, kMfmaQueries);
  const int want = (3072 + tiles - 1) / tiles;
  const int by_length = (n / num_segments) / 4096;
  int chunks = std::max(1, std::min(std::min(want, 16), by_length));
  if (const char *env = std::getenv("PCA_KNN_SLICES")) {
    const int v = std::atoi(env);
    if (v >= 1 && v <= 64)
      chunks = v;
  }
  return chunks;
}

size_t knn_mfma_scratch_bytes(int n, int m, int d, int num_segments, int k,
                              int forced_chunks) {
  const size_t tiles = plan_upper_bound(m, num_segments, kMfmaQueries);
  // the largest slice count a call may choose
  const int chunks = forced_chunks > 0
                         ? forced_chunks
                         : std::max(knn_mfma_slices(n, m, num_segments), 1);
  return mfma_pack_bytes(n, d) + align256(sizeof(float) * (size_t)n) +
         2 * align256(sizeof(float) * (size_t)m) +
         align256(sizeof(double) * tiles * chunks * (size_t)k *
                  kMfmaQueries);
}

hipError_t launch_knn_mfma(const SearchInput &in, int k, bool cosine,
                           const int *work_start, void *scratch,
                           const DenseResult &out, hipEvent_t time_start,
                           hipEvent_t time_stop, hipStream_t stream,
                           int64_t *nearest_out, const MfmaSecondPass *second) {
  const bool nearest = nearest_out != nullptr;
  const int tiles_bound =
      plan_upper_bound(in.m, in.num_segments, kMfmaQueries);
  const int chunks = second ? second->chunks
                            : knn_mfma_slices(in.n, in.m, in.num_segments);
  const int *gate = second ? second->gate : nullptr;
  char *base = static_cast<char *>(scratch);
  uint4 *x_pack = reinterpret_cast<uint4 *>(base);
  base += mfma_pack_bytes(in.n, in.d);
  float *x_sq = reinterpret_cast<float *>(base);
  base += align256(sizeof(float) * (size_t)in.n);
  float *tau = reinterpret_cast<float *>(base);
  base += align256(sizeof(float) * (size_t)in.m);
  float *y_norm = reinterpret_cast<float *>(base);
  base += align256(sizeof(float) * (size_t)in.m);
  double *partial = reinterpret_cast<double *>(base);

  if (second) {
    // the first pass has the norms already
    x_sq = const_cast<float *>(second->x_norm);
    y_norm = const_cast<float *>(second->y_norm);
  } else if (cosine) {
    (void)launch_row_norms(static_cast<const float *>(in.x), in.n, in.d, x_sq,
                           stream);
    (void)launch_row_norms(static_cast<const float *>(in.y), in.m, in.d,
                           y_norm, stream);
  } else
    hipLaunchKernelGGL(row_sqnorm_kernel, dim3((in.n + kBlock - 1) / kBlock),
                       dim3(kBlock), 0, stream,
                       static_cast<const float *>(in.x), in.n, in.d, x_sq);
  hipLaunchKernelGGL(fill_tau_kernel, dim3((in.m + kBlock - 1) / kBlock),
                     dim3(kBlock), 0, stream, tau, in.m,
                     nearest ? kNearestLimit : kKnnSentinel);
  {
    const float *xf = static_cast<const float *>(in.x);
    hipError_t perr;
    switch (mfma_blocks(in.d)) {
    case 2:
      perr = launch_mfma_pack_rows<2>(xf, x_sq, in.n, in.d, cosine, x_pack,
                                      stream, gate);
      break;
    case 3:
      perr = launch_mfma_pack_rows<3>(xf, x_sq, in.n, in.d, cosine, x_pack,
                                      stream, gate);
      break;
    case 5:
      perr = launch_mfma_pack_rows<5>(xf, x_sq, in.n, in.d, cosine, x_pack,
                                      stream, gate);
      break;
    default:
      perr = launch_mfma_pack_rows<9>(xf, x_sq, in.n, in.d, cosine, x_pack,
                                      stream, gate);
      break;
    }
    if (perr != hipSuccess)
      return perr;
  }

  KnnMfmaParams p;
  p.x = static_cast<const float *>(in.x);
  p.y = static_cast<const float *>(in.y);
  p.ptr_x = in.ptr_x;
  p.ptr_y = in.ptr_y;
  p.x_sq = x_sq;
  p.y_norm = y_norm;
  p.x_pack = x_pack;
  p.n = in.n;
  p.m = in.m;
  p.d = in.d;
  p.num_segments = in.num_segments;
  p.k = k;
  p.work_start = work_start;
  p.num_chunks = chunks;
  p.tau = tau;
  p.partial = partial;
  p.gate = gate;
  p.redo_q = second ? second->redo_q : nullptr;

  const int kb = nearest ? 1 : k_bucket(k);
  const int grid = tiles_bound * chunks;
  auto launch = [&](const KnnMfmaParams &pp, int g) {
    switch (mfma_blocks(in.d)) {
    case 2:
      return launch_knn_mfma_blocks<2>(pp, kb, cosine, g, stream);
    case 3:
      return launch_knn_mfma_blocks<3>(pp, kb, cosine, g, stream);
    case 5:
      return launch_knn_mfma_blocks<5>(pp, kb, cosine, g, stream);
    default:
      return launch_knn_mfma_blocks<9>(pp, kb, cosine, g, stream);
    }
  };
  if (time_start)
    (void)hipEventRecord(time_start, stream);
  const hipError_t err = launch(p, grid);
  if (time_stop)
    (void)hipEventRecord(time_stop, stream);
  if (err != hipSuccess)
    return err;

  // one list per query and slice
  KnnLowdParams mp;
  mp.x = p.x;
  mp.y = p.y;
  mp.ptr_x = in.ptr_x;
  mp.ptr_y = in.ptr_y;
  mp.n = in.n;
  mp.m = in.m;
  mp.d_in = in.d;
  mp.num_segments = in.num_segments;
  mp.k = k;
  mp.work_start = work_start;
  mp.num_chunks = chunks;
  mp.tau = nullptr;
  mp.partial = partial;
  mp.out_idx = out.idx;
  mp.out_dist = out.dist;
  mp.out_count = out.count;
  mp.out_nearest = nearest_out;
  mp.x_split = nullptr;
  mp.gate = gate;
  mp.redo_q = second ? second->redo_q : nullptr;
  switch (kb) {
  case 1:
    hipLaunchKernelGGL((knn_merge_kernel<8, kMfmaQueries, true>),
                       dim3(tiles_bound), dim3(kBlock), 0, stream, mp);
    break;
  case 8:
    launch_mfma_merge<8>(mp, tiles_bound, stream);
    break;
  case 16:
    launch_mfma_merge<16>(mp, tiles_bound, stream);
    break;
  case 24:
    launch_mfma_merge<24>(mp, tiles_bound, stream);
    break;
  case 32:
    launch_mfma_merge<32>(mp, tiles_bound, stream);
    break;
  case 48:
    launch_mfma_merge<48>(mp, tiles_bound, stream);
    break;
  case 64:
    launch_mfma_merge<64>(mp, tiles_bound, stream);
    break;
  default:
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

} // namespace pca
