// C ABI of the neighbour-search library (declared in include/pca_neighbors.h).
//
// Validates sizes on the host, carves the caller's workspace and queues the
// kernels on the caller's stream.  No allocation, no synchronisation, no
// state: the operator-level behaviour of the reference's host wrappers
// (csrc/cuda/knn_cuda.cu:86-135, csrc/cuda/radius_cuda.cu:44-96) minus tensor
// handling, which belongs to the binding above this layer.
#include "../../include/pca_neighbors.h"

#include "device_utils.hpp"
#include "launchers.hpp"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <mutex>

namespace {

thread_local char g_last_error[256] = "";

int fail(int status, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return status;
}

// one-shot request of pca_time_next_search
// pca_report_examples: where the next call that derives pointers from ids
// leaves the number of examples those ids speak of
thread_local int64_t *g_examples_out = nullptr;
thread_local hipEvent_t g_time_start = nullptr;
thread_local hipEvent_t g_time_stop = nullptr;

struct SearchTimer {
  hipStream_t stream;
  hipEvent_t start, stop;
  explicit SearchTimer(hipStream_t s)
      : stream(s), start(g_time_start), stop(g_time_stop) {
    // consumed by this call whether or not it reaches its search kernel
    g_time_start = g_time_stop = nullptr;
  }
  void begin() {
    if (start)
      (void)hipEventRecord(start, stream);
  }
  void done() {
    if (stop)
      (void)hipEventRecord(stop, stream);
    stop = nullptr;
  }
};

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct Carver {
  char *base;
  size_t offset = 0;
  explicit Carver(void *p) : base(static_cast<char *>(p)) {}
  template <typename T> T *take(size_t count) {
    T *p = reinterpret_cast<T *>(base + offset);
    offset += align256(sizeof(T) * count);
    return p;
  }
};

__global__ void set_i64_kernel(int64_t *p, int64_t v) { *p = v; }

__global__ void fill_i64_kernel(int64_t *p, int64_t count, int64_t v) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count)
    p[i] = v;
}

constexpr int64_t kMaxRows = 2147483646; // n, m < 2^31 - 1

// Segments a call works with: one when no pointers are given.
int64_t segments_in_use(const int64_t *ptr_x, int64_t num_segments) {
  return ptr_x == nullptr ? 1 : num_segments;
}

bool sizes_ok(int64_t n, int64_t m, int64_t d, int64_t num_segments) {
  return n >= 0 && m >= 0 && n <= kMaxRows && m <= kMaxRows && d >= 1 &&
         d <= (1 << 20) && num_segments >= 1 && num_segments <= kMaxRows;
}

// two arrays of num_segments + 1 pointers (PCA_SEGMENTS_BY_ID)
size_t segment_pointer_bytes(int64_t num_segments) {
  return 2 * align256(sizeof(int64_t) * (size_t)(num_segments + 1));
}

// With PCA_SEGMENTS_BY_ID the caller's ptr_x / ptr_y are sorted example ids;
// the pointers the kernels read live in `area` (segment_pointer_bytes) and are
// written by the launch that plans the work.  Returns the source description
// for that launch and redirects ptr_x / ptr_y.
pca::SegmentSource segments_by_id(const int64_t *&ptr_x, const int64_t *&ptr_y,
                                  int64_t n, int64_t m, int64_t num_segments,
                                  void *area) {
  pca::SegmentSource src;
  src.ids_x = ptr_x;
  src.ids_y = ptr_y;
  src.n = (int)n;
  src.m = (int)m;
  src.ptr_x = static_cast<int64_t *>(area);
  src.ptr_y = reinterpret_cast<int64_t *>(
      static_cast<char *>(area) +
      align256(sizeof(int64_t) * (size_t)(num_segments + 1)));
  ptr_x = src.ptr_x;
  ptr_y = src.ptr_y;
  src.examples_out = g_examples_out;
  g_examples_out = nullptr;
  return src;
}

// Sizes of the pieces pca_knn carves out of the workspace, in carving order.
struct KnnLayout {
  size_t x_norm = 0;  // |x| (any-dimension kernel, cosine)
  size_t sliced = 0;  // shared bounds + partial key lists of sliced segments
  size_t work_start, idx, dist, count, compact;
  size_t ptrs = 0;    // segment pointers derived from example ids, both sides
  size_t total() const {
    return x_norm + sliced + work_start + idx + dist + count + compact + ptrs;
  }
};

KnnLayout knn_layout(int64_t n, int64_t m, int64_t d, int64_t num_segments,
                     int64_t k, int dtype) {
  KnnLayout w;
  if (dtype != PCA_F32) {
    w.x_norm = align256(pca::anytype_norm_bytes((int)n));
    w.sliced = pca::knn_anytype_scratch_bytes((int)n, (int)m,
                                              (int)num_segments, (int)k);
    // (16-bit rows through the matrix-core filter: the Euclidean metric only,
    // but one size query serves both)
    if ((dtype == PCA_F16 || dtype == PCA_BF16) &&
        pca::knn_feat16_supported((int)n, (int)d, (int)num_segments, (int)k,
                                  false, dtype == PCA_BF16))
      w.sliced = std::max(w.sliced,
                          pca::knn_feat16_scratch_bytes((int)n, (int)m, (int)d,
                                                        (int)num_segments,
                                                        (int)k));
  } else if (d > 8) {
    w.x_norm = align256(sizeof(float) * (size_t)n);
    if (pca::knn_feat_supported((int)d, (int)k, false))
      w.sliced = pca::knn_feat_scratch_bytes((int)n, (int)m, (int)d,
                                             (int)num_segments, (int)k);
    else if (pca::knn_mfma_supported((int)d, (int)k, false))
      w.sliced = pca::knn_mfma_scratch_bytes((int)n, (int)m, (int)d,
                                             (int)num_segments, (int)k);
    else
      w.sliced = pca::knn_generic_scratch_bytes((int)n, (int)m,
                                                (int)num_segments, (int)k);
  } else {
    // the larger of the two metrics' needs, so one size query serves both
    for (int cosine = 0; cosine < 2; ++cosine) {
      const pca::KnnLowdConfig cfg = pca::knn_lowd_config(
          (int)d, (int)k, (int)n, (int)m, (int)num_segments, cosine != 0);
      w.sliced = std::max(w.sliced,
                          pca::knn_lowd_scratch_bytes(cfg, (int)n, (int)m,
                                                      (int)d,
                                                      (int)num_segments,
                                                      (int)k));
    }
  }
  w.work_start = align256(sizeof(int) * (size_t)(num_segments + 1));
  w.idx = align256(sizeof(int) * (size_t)m * (size_t)k);
  w.dist = align256(sizeof(float) * (size_t)m * (size_t)k);
  w.count = align256(sizeof(int) * (size_t)m);
  w.compact = pca::compact_workspace_bytes((int)m);
  w.ptrs = segment_pointer_bytes(num_segments);
  return w;
}

size_t knn_workspace(int64_t n, int64_t m, int64_t d, int64_t num_segments,
                     int64_t k, int dtype) {
  return knn_layout(n, m, d, num_segments, k, dtype).total();
}

size_t binned_workspace(int64_t n, int64_t m, int64_t num_segments,
                        int64_t k) {
  return align256(pca::knn_binned_scratch_bytes((int)n, (int)m,
                                                (int)num_segments)) +
         align256(sizeof(int) * (size_t)m * (size_t)k) +
         align256(sizeof(float) * (size_t)m * (size_t)k) +
         align256(sizeof(int) * (size_t)m) +
         pca::compact_workspace_bytes((int)m);
}

size_t radius_binned_workspace(int64_t n, int64_t m, int64_t num_segments,
                               int64_t slots) {
  return align256(pca::knn_binned_scratch_bytes((int)n, (int)m,
                                                (int)num_segments)) +
         align256(sizeof(int) * (size_t)m * (size_t)slots) +
         align256(sizeof(int) * (size_t)m) +
         pca::compact_workspace_bytes((int)m);
}

bool dtype_ok(int dtype) {
  return dtype == PCA_F32 || dtype == PCA_F64 || dtype == PCA_F16 ||
         dtype == PCA_BF16;
}

size_t radius_workspace(int64_t n, int64_t m, int64_t d, int64_t num_segments,
                        int64_t slots, int dtype) {
  size_t bytes = 0;
  if (dtype == PCA_F32 &&
      pca::radius_mc_supported((int)d, (int)n, (int)m, (int)num_segments))
    bytes += pca::radius_mc_scratch_bytes((int)n, (int)d);
  else if (dtype == PCA_F32 &&
           pca::radius_feat_supported((int)n, (int)m, (int)d,
                                      (int)num_segments, (int)slots))
    bytes += pca::knn_feat_scratch_bytes((int)n, (int)m, (int)d,
                                         (int)num_segments, (int)slots);
  else if ((dtype == PCA_F16 || dtype == PCA_BF16) &&
           pca::radius_feat_supported((int)n, (int)m, (int)d,
                                      (int)num_segments, (int)slots,
                                      dtype == PCA_F16 ? 1 : 2))
    bytes += pca::knn_feat16_scratch_bytes((int)n, (int)m, (int)d,
                                           (int)num_segments, (int)slots);
  bytes += align256(sizeof(int) * (size_t)(num_segments + 1));
  bytes += align256(sizeof(int) * (size_t)m * (size_t)slots);
  bytes += align256(sizeof(int) * (size_t)m);
  bytes += pca::compact_workspace_bytes((int)m);
  bytes += segment_pointer_bytes(num_segments);
  return bytes;
}

// by_id: the entry point takes example ids in place of pointers
bool edge_flags_ok(int flags, bool by_id = false) {
  const int known = PCA_EDGES_DROP_SELF | PCA_EDGES_X_FIRST |
                    (by_id ? PCA_SEGMENTS_BY_ID : 0);
  return (flags & ~known) == 0;
}

bool nearest_dtype_ok(int dtype) {
  return dtype == PCA_F32 || dtype == PCA_F64 || dtype == PCA_F16;
}

// (searching rows n, candidates m)
bool nearest_low_d(int64_t d, int dtype) { return dtype == PCA_F32 && d <= 8; }

// fp32, 8 < d <= 128: the matrix-core kernel of the feature-space kNN
bool nearest_mfma(int64_t d, int dtype) {
  return dtype == PCA_F32 && d > 8 &&
         pca::knn_mfma_supported((int)d, 1, false);
}

size_t nearest_workspace(int64_t n, int64_t m, int64_t d,
                         int64_t num_segments, int dtype) {
  size_t bytes = align256(sizeof(int) * (size_t)(num_segments + 1));
  if (nearest_mfma(d, dtype))
    bytes += pca::knn_mfma_scratch_bytes((int)m, (int)n, (int)d,
                                         (int)num_segments, 1);
  if (nearest_low_d(d, dtype)) {
    const pca::KnnLowdConfig cfg =
        pca::nearest_lowd_config((int)d, (int)m, (int)n, (int)num_segments);
    bytes += pca::knn_lowd_scratch_bytes(cfg, (int)m, (int)n, (int)d,
                                         (int)num_segments, 1);
  }
  return bytes;
}

// The binned entry points sort with rocPRIM, whose clears of histograms are
// memset nodes in a captured graph: they are refused while `stream` is being
// captured (the scanning entry points can be captured).
bool being_captured(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

int refuse_capture(const char *entry) {
  return fail(PCA_ERR_UNSUPPORTED,
              "%s cannot be captured into a graph (its sorts clear their "
              "buffers with memset nodes); use the scanning entry point",
              entry);
}

int check_launch(hipError_t err, const char *what) {
  if (err != hipSuccess)
    return fail(PCA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
  return PCA_OK;
}

int knn_call(const void *x, const void *y, const int64_t *ptr_x,
             const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
             int64_t num_segments, int64_t k, int cosine, int dtype,
             int edge_flags, int64_t *edges, int64_t *num_edges, void *dist,
             void *workspace, size_t workspace_bytes, void *stream_);

} // namespace

// Scratch of pca_knn_fixed_scratch: device memory of the library itself, one
// copy per GPU the library runs on, held until the process ends.  In host code
// the array's name is only a handle for hipGetSymbolAddress; kernels and copies
// take the per-device address kept in g_fixed_scratch.
static __device__ __align__(256) unsigned char scratch[PCA_FIXED_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_fixed_scratch_mutex;
void *g_fixed_scratch[kMaxDevices] = {};

// The address of `scratch` on the device that is current on this thread
// (looked up once per device; nothing is allocated).
int fixed_scratch_of_current_device(void **out) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess || device < 0 || device >= kMaxDevices)
    return fail(PCA_ERR_NO_DEVICE, "hipGetDevice: %s (device %d)",
                hipGetErrorString(err), device);
  std::lock_guard<std::mutex> lock(g_fixed_scratch_mutex);
  if (g_fixed_scratch[device] == nullptr) {
    void *ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr)
      return fail(PCA_ERR_NO_DEVICE, "hipGetSymbolAddress(scratch): %s",
                  hipGetErrorString(err));
    if (((uintptr_t)ptr & 255) != 0)
      return fail(PCA_ERR_WORKSPACE, "the fixed scratch is not 256-aligned");
    g_fixed_scratch[device] = ptr;
  }
  *out = g_fixed_scratch[device];
  return PCA_OK;
}

} // namespace

extern "C" {

int pca_abi_version(void) { return PCA_ABI_VERSION; }

const char *pca_status_string(int status) {
  switch (status) {
  case PCA_OK:
    return "ok";
  case PCA_ERR_INVALID_ARGUMENT:
    return "invalid argument";
  case PCA_ERR_K_TOO_LARGE:
    return "`k` needs to smaller than or equal to 100";
  case PCA_ERR_WORKSPACE:
    return "workspace too small or misaligned";
  case PCA_ERR_LAUNCH:
    return "HIP launch failed";
  case PCA_ERR_UNSUPPORTED:
    return "combination not supported";
  case PCA_ERR_NO_DEVICE:
    return "no usable device";
  default:
    return "unknown status";
  }
}

const char *pca_last_error(void) { return g_last_error; }

int pca_time_next_search(void *start_event, void *stop_event) {
  if ((start_event == nullptr) != (stop_event == nullptr))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "start and stop events must both be given or both be NULL");
  g_time_start = static_cast<hipEvent_t>(start_event);
  g_time_stop = static_cast<hipEvent_t>(stop_event);
  return PCA_OK;
}

int pca_report_examples(int64_t *examples_in_use) {
  g_examples_out = examples_in_use;
  return PCA_OK;
}

int pca_segment_pointers(const int64_t *ids_x, int64_t n, const int64_t *ids_y,
                         int64_t m, int64_t num_segments, int64_t *ptr_x,
                         int64_t *ptr_y, void *stream_) {
  g_last_error[0] = 0;
  if (n < 0 || m < 0 || n > kMaxRows || m > kMaxRows || num_segments < 1 ||
      num_segments > kMaxRows)
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "bad sizes n=%lld m=%lld num_segments=%lld", (long long)n,
                (long long)m, (long long)num_segments);
  if (ptr_x == nullptr || ptr_y == nullptr || (n > 0 && ids_x == nullptr) ||
      (m > 0 && ids_y == nullptr))
    return fail(PCA_ERR_INVALID_ARGUMENT, "ids or pointers are NULL");
  pca::SegmentSource src;
  src.ids_x = ids_x;
  src.ids_y = ids_y;
  src.n = (int)n;
  src.m = (int)m;
  src.ptr_x = ptr_x;
  src.ptr_y = ptr_y;
  src.examples_out = g_examples_out;
  g_examples_out = nullptr;
  return check_launch(
      pca::launch_segment_pointers(src, (int)num_segments,
                                   static_cast<hipStream_t>(stream_)),
      "segment_pointers_kernel");
}

size_t pca_knn_workspace_bytes(int64_t n, int64_t m, int64_t d,
                               int64_t num_segments, int64_t k, int dtype) {
  if (num_segments < 1)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments) || k < 1 || k > PCA_KNN_MAX_K ||
      !dtype_ok(dtype))
    return 0;
  return knn_workspace(n, m, d, num_segments, k, dtype);
}

int pca_knn(const void *x, const void *y, const int64_t *ptr_x,
            const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
            int64_t num_segments, int64_t k, int cosine, int dtype,
            int edge_flags, int64_t *edges, int64_t *num_edges, void *dist,
            void *workspace, size_t workspace_bytes, void *stream_) {
  return knn_call(x, y, ptr_x, ptr_y, n, m, d, num_segments, k, cosine, dtype,
                  edge_flags, edges, num_edges, dist, workspace,
                  workspace_bytes, stream_);
}

int pca_knn_fixed_scratch(const void *x, const void *y, const int64_t *ptr_x,
                          const int64_t *ptr_y, int64_t n, int64_t m,
                          int64_t d, int64_t num_segments, int64_t k,
                          int cosine, int dtype, int edge_flags,
                          int64_t *edges, int64_t *num_edges, void *dist,
                          void *stream_) {
  g_last_error[0] = 0;
  // (the size test sees what the search will use: knn_call sizes its
  // workspace by the same two functions; invalid sizes are reported by
  // knn_call itself)
  const int64_t segs = segments_in_use(ptr_x, num_segments);
  if (sizes_ok(n, m, d, segs) && k >= 1 && k <= PCA_KNN_MAX_K &&
      dtype_ok(dtype) && n > 0 && m > 0) {
    const size_t need = knn_workspace(n, m, d, segs, k, dtype);
    if (need > PCA_FIXED_SCRATCH_BYTES)
      return fail(PCA_ERR_WORKSPACE,
                  "pca_knn_fixed_scratch: this search needs %zu bytes of "
                  "scratch, the library's fixed buffer holds %zu; use pca_knn "
                  "with a workspace of the caller",
                  need, (size_t)PCA_FIXED_SCRATCH_BYTES);
  }
  void *buffer = nullptr;
  const int rc = fixed_scratch_of_current_device(&buffer);
  if (rc != PCA_OK)
    return rc;
  return knn_call(x, y, ptr_x, ptr_y, n, m, d, num_segments, k, cosine, dtype,
                  edge_flags, edges, num_edges, dist, buffer,
                  PCA_FIXED_SCRATCH_BYTES, stream_);
}

} // extern "C"

namespace {

int knn_call(const void *x, const void *y, const int64_t *ptr_x,
             const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
             int64_t num_segments, int64_t k, int cosine, int dtype,
             int edge_flags, int64_t *edges, int64_t *num_edges, void *dist,
             void *workspace, size_t workspace_bytes, void *stream_) {
  g_last_error[0] = 0;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  SearchTimer timer(stream);
  if ((ptr_x == nullptr) != (ptr_y == nullptr))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "ptr_x and ptr_y must both be given or both be NULL");
  num_segments = segments_in_use(ptr_x, num_segments);
  if (!sizes_ok(n, m, d, num_segments))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "bad sizes n=%lld m=%lld d=%lld num_segments=%lld",
                (long long)n, (long long)m, (long long)d,
                (long long)num_segments);
  if (k < 1)
    return fail(PCA_ERR_INVALID_ARGUMENT, "k must be >= 1, got %lld",
                (long long)k);
  if (k > PCA_KNN_MAX_K)
    return fail(PCA_ERR_K_TOO_LARGE, "%s",
                pca_status_string(PCA_ERR_K_TOO_LARGE));
  if (num_edges == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "num_edges is NULL");
  if (!dtype_ok(dtype))
    return fail(PCA_ERR_UNSUPPORTED, "element type %d is not built", dtype);
  if (dtype != PCA_F32 && dist != nullptr)
    return fail(PCA_ERR_UNSUPPORTED,
                "per-edge distances are returned for fp32 points only");
  if (!edge_flags_ok(edge_flags, true))
    return fail(PCA_ERR_INVALID_ARGUMENT, "unknown edge flags %d", edge_flags);

  if (n == 0 || m == 0) {
    hipLaunchKernelGGL(set_i64_kernel, dim3(1), dim3(1), 0, stream, num_edges,
                       (int64_t)0);
    return check_launch(hipGetLastError(), "set_i64_kernel");
  }
  if (x == nullptr || y == nullptr || edges == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "x, y or edges is NULL");
  if (workspace == nullptr || ((uintptr_t)workspace & 255) != 0 ||
      workspace_bytes < knn_workspace(n, m, d, num_segments, k, dtype))
    return fail(PCA_ERR_WORKSPACE, "workspace needs %zu bytes, 256-aligned",
                knn_workspace(n, m, d, num_segments, k, dtype));

  const bool f32 = dtype == PCA_F32;
  const bool low_d =
      f32 && pca::knn_lowd_supported((int)d, (int)k, cosine != 0);

  const KnnLayout lay = knn_layout(n, m, d, num_segments, k, dtype);
  char *cursor = static_cast<char *>(workspace);
  auto take = [&cursor](size_t bytes) {
    char *piece = cursor;
    cursor += bytes;
    return static_cast<void *>(piece);
  };
  float *x_norm = static_cast<float *>(take(lay.x_norm));
  void *lowd_scratch = take(lay.sliced);
  int *work_start = static_cast<int *>(take(lay.work_start));
  pca::DenseResult dense;
  dense.idx = static_cast<int *>(take(lay.idx));
  dense.dist = static_cast<float *>(take(lay.dist));
  dense.count = static_cast<int *>(take(lay.count));
  dense.slots = (int)k;
  void *compact_ws = take(lay.compact);
  if (dist == nullptr)
    dense.dist = nullptr;
  pca::SegmentSource src;
  const bool by_id = (edge_flags & PCA_SEGMENTS_BY_ID) != 0 && ptr_x != nullptr;
  if (by_id)
    src = segments_by_id(ptr_x, ptr_y, n, m, num_segments, take(lay.ptrs));
  pca::KnnLowdConfig cfg = pca::knn_lowd_config(
      (int)d, (int)k, (int)n, (int)m, (int)num_segments, cosine != 0);
  // (the matrix-core kernels count the edges while they write their lists)
  if (low_d && cfg.matrix_cores)
    pca::compact_hints(dense, (int)m, compact_ws,
                       (edge_flags & PCA_EDGES_DROP_SELF) != 0);

  pca::SearchInput in{x,      y,      ptr_x,  ptr_y,
                      (int)n, (int)m, (int)d, (int)num_segments};
  const bool feat =
      f32 && !low_d && pca::knn_feat_supported((int)d, (int)k, cosine != 0);
  const bool mfma = f32 && !low_d && !feat &&
                    pca::knn_mfma_supported((int)d, (int)k, cosine != 0);
  const int r16 = dtype == PCA_F16 ? 1 : (dtype == PCA_BF16 ? 2 : 0);
  const bool feat16 =
      r16 != 0 && pca::knn_feat16_supported((int)n, (int)d, (int)num_segments,
                                            (int)k, cosine != 0, r16 == 2);
  // (so does the one-kernel feature-space search)
  if (feat16 || (feat && pca::knn_feat_one_kernel((int)n, (int)m, (int)d,
                                                   (int)num_segments, (int)k,
                                                   cosine != 0)))
    pca::compact_hints(dense, (int)m, compact_ws,
                       (edge_flags & PCA_EDGES_DROP_SELF) != 0);
  if (mfma || feat || feat16)
    cfg.tile_queries = pca::kMfmaTileQueries;
  else if (!low_d)
    cfg.tile_queries = pca::kBlock; // any-dimension kernel: one query per lane
  int rc = PCA_OK;
  // (the low-dimensional path plans its work inside its own first launch)
  if (!low_d)
    rc = check_launch(pca::launch_plan(ptr_y, (int)m, (int)num_segments,
                                       cfg.tile_queries, work_start, stream,
                                       by_id ? &src : nullptr),
                      "plan_kernel");
  if (rc != PCA_OK)
    return rc;
  const int bound =
      pca::plan_upper_bound((int)m, (int)num_segments, cfg.tile_queries);
  if (low_d) {
    // the events bracket the search kernel itself, not the preparation and
    // the merge around it
    rc = check_launch(pca::launch_knn_lowd(in, (int)k, cosine != 0, cfg,
                                           work_start, lowd_scratch, dense,
                                           timer.start, timer.stop, stream,
                                           nullptr, by_id ? &src : nullptr),
                      "knn_lowd_kernel");
    timer.stop = nullptr;
  } else if (feat) {
    rc = check_launch(pca::launch_knn_feat(in, (int)k, cosine != 0, work_start,
                                           lowd_scratch, dense, timer.start,
                                           timer.stop, stream),
                      "knn_feat_kernel");
    timer.stop = nullptr;
  } else if (feat16) {
    rc = check_launch(pca::launch_knn_feat(in, (int)k, false, work_start,
                                           lowd_scratch, dense, timer.start,
                                           timer.stop, stream, r16),
                      "knn_feat_small_kernel");
    timer.stop = nullptr;
  } else if (mfma) {
    rc = check_launch(pca::launch_knn_mfma(in, (int)k, cosine != 0, work_start,
                                           lowd_scratch, dense, timer.start,
                                           timer.stop, stream),
                      "knn_mfma_kernel");
    timer.stop = nullptr;
  } else if (!f32) {
    timer.begin();
    rc = check_launch(pca::launch_knn_anytype(dtype, in, (int)k, cosine != 0,
                                              x_norm, work_start, bound,
                                              dense, stream,
                                              lay.sliced ? lowd_scratch
                                                         : nullptr),
                      "knn_any_kernel");
    timer.done();
  } else {
    if (cosine) {
      rc = check_launch(pca::launch_row_norms(static_cast<const float *>(x),
                                              (int)n, (int)d, x_norm, stream),
                        "row_norm_kernel");
      if (rc != PCA_OK)
        return rc;
    }
    timer.begin();
    rc = check_launch(pca::launch_knn_generic(
                          in, (int)k, cosine != 0, x_norm, work_start, bound,
                          dense, stream, lay.sliced ? lowd_scratch : nullptr),
                      "knn_generic_kernel");
    timer.done();
  }
  if (rc != PCA_OK)
    return rc;
  return check_launch(
      pca::launch_compact(dense, (int)m, edges, num_edges,
                          static_cast<float *>(dist), compact_ws, stream,
                          (edge_flags & PCA_EDGES_DROP_SELF) != 0,
                          (edge_flags & PCA_EDGES_X_FIRST) != 0),
      "compaction kernels");
}

} // namespace

extern "C" {

size_t pca_knn_binned_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                      int64_t num_segments, int64_t k) {
  if (num_segments < 1)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments) || n == 0 || m == 0 ||
      !pca::knn_binned_supported((int)d, (int)k, false))
    return 0;
  return binned_workspace(n, m, num_segments, k);
}

int pca_knn_binned(const void *x, const void *y, const int64_t *ptr_x,
                   const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                   int64_t num_segments, int64_t k, int edge_flags,
                   int64_t *edges, int64_t *num_edges, void *dist,
                   void *workspace, size_t workspace_bytes, void *stream_) {
  g_last_error[0] = 0;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (being_captured(stream))
    return refuse_capture("pca_knn_binned");
  SearchTimer timer(stream);
  if ((ptr_x == nullptr) != (ptr_y == nullptr))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "ptr_x and ptr_y must both be given or both be NULL");
  if (ptr_x == nullptr)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "bad sizes n=%lld m=%lld d=%lld num_segments=%lld",
                (long long)n, (long long)m, (long long)d,
                (long long)num_segments);
  if (k < 1)
    return fail(PCA_ERR_INVALID_ARGUMENT, "k must be >= 1, got %lld",
                (long long)k);
  if (k > PCA_KNN_MAX_K)
    return fail(PCA_ERR_K_TOO_LARGE, "%s",
                pca_status_string(PCA_ERR_K_TOO_LARGE));
  if (!pca::knn_binned_supported((int)d, (int)k, false))
    return fail(PCA_ERR_UNSUPPORTED,
                "binned search: fp32 points of up to 3 dimensions and k <= 64, "
                "got d=%lld k=%lld",
                (long long)d, (long long)k);
  if (num_edges == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "num_edges is NULL");
  if (!edge_flags_ok(edge_flags))
    return fail(PCA_ERR_INVALID_ARGUMENT, "unknown edge flags %d", edge_flags);
  if (n == 0 || m == 0) {
    hipLaunchKernelGGL(set_i64_kernel, dim3(1), dim3(1), 0, stream, num_edges,
                       (int64_t)0);
    return check_launch(hipGetLastError(), "set_i64_kernel");
  }
  if (x == nullptr || y == nullptr || edges == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "x, y or edges is NULL");
  const size_t need = binned_workspace(n, m, num_segments, k);
  if (workspace == nullptr || ((uintptr_t)workspace & 255) != 0 ||
      workspace_bytes < need)
    return fail(PCA_ERR_WORKSPACE, "workspace needs %zu bytes, 256-aligned",
                need);

  Carver carve(workspace);
  void *scratch = carve.take<char>(pca::knn_binned_scratch_bytes(
      (int)n, (int)m, (int)num_segments));
  pca::DenseResult dense;
  dense.idx = carve.take<int>((size_t)m * (size_t)k);
  dense.dist = carve.take<float>((size_t)m * (size_t)k);
  dense.count = carve.take<int>((size_t)m);
  dense.slots = (int)k;
  void *compact_ws = carve.take<char>(pca::compact_workspace_bytes((int)m));
  if (dist == nullptr)
    dense.dist = nullptr;

  pca::SearchInput in{x,      y,      ptr_x,  ptr_y,
                      (int)n, (int)m, (int)d, (int)num_segments};
  int rc = check_launch(pca::launch_knn_binned(in, (int)k, scratch, dense,
                                               timer.start, timer.stop, stream),
                        "binned search");
  timer.stop = nullptr;
  if (rc != PCA_OK)
    return rc;
  return check_launch(
      pca::launch_compact(dense, (int)m, edges, num_edges,
                          static_cast<float *>(dist), compact_ws, stream,
                          (edge_flags & PCA_EDGES_DROP_SELF) != 0,
                          (edge_flags & PCA_EDGES_X_FIRST) != 0),
      "compaction kernels");
}

int64_t pca_radius_slots(int64_t n, int64_t max_num_neighbors) {
  if (n < 0 || max_num_neighbors < 0)
    return 0;
  return max_num_neighbors < n ? max_num_neighbors : n;
}

size_t pca_radius_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                  int64_t num_segments,
                                  int64_t max_num_neighbors, int dtype) {
  if (num_segments < 1)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments) || max_num_neighbors < 1 ||
      !dtype_ok(dtype))
    return 0;
  return radius_workspace(n, m, d, num_segments,
                          pca_radius_slots(n, max_num_neighbors), dtype);
}

int pca_radius(const void *x, const void *y, const int64_t *ptr_x,
               const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
               int64_t num_segments, double r, int64_t max_num_neighbors,
               int ignore_same_index, int dtype, int edge_flags,
               int64_t *edges, int64_t *num_edges, void *workspace,
               size_t workspace_bytes, void *stream_) {
  g_last_error[0] = 0;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  SearchTimer timer(stream);
  if ((ptr_x == nullptr) != (ptr_y == nullptr))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "ptr_x and ptr_y must both be given or both be NULL");
  if (ptr_x == nullptr)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "bad sizes n=%lld m=%lld d=%lld num_segments=%lld",
                (long long)n, (long long)m, (long long)d,
                (long long)num_segments);
  if (max_num_neighbors < 1)
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "max_num_neighbors must be >= 1, got %lld",
                (long long)max_num_neighbors);
  if (!edge_flags_ok(edge_flags, true))
    return fail(PCA_ERR_INVALID_ARGUMENT, "unknown edge flags %d", edge_flags);
  // (the search itself skips the row; it must not count towards the limit)
  if (edge_flags & PCA_EDGES_DROP_SELF)
    ignore_same_index = 1;
  if (num_edges == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "num_edges is NULL");
  if (!dtype_ok(dtype))
    return fail(PCA_ERR_UNSUPPORTED, "element type %d is not built", dtype);

  if (n == 0 || m == 0) {
    hipLaunchKernelGGL(set_i64_kernel, dim3(1), dim3(1), 0, stream, num_edges,
                       (int64_t)0);
    return check_launch(hipGetLastError(), "set_i64_kernel");
  }
  if (x == nullptr || y == nullptr || edges == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "x, y or edges is NULL");
  const int64_t slots = pca_radius_slots(n, max_num_neighbors);
  if (workspace == nullptr || ((uintptr_t)workspace & 255) != 0 ||
      workspace_bytes <
          radius_workspace(n, m, d, num_segments, slots, dtype))
    return fail(PCA_ERR_WORKSPACE, "workspace needs %zu bytes, 256-aligned",
                radius_workspace(n, m, d, num_segments, slots, dtype));

  const bool matrix_cores =
      dtype == PCA_F32 &&
      pca::radius_mc_supported((int)d, (int)n, (int)m, (int)num_segments);
  const int r16 = dtype == PCA_F16 ? 1 : (dtype == PCA_BF16 ? 2 : 0);
  const bool feature_space =
      !matrix_cores && (dtype == PCA_F32 || r16 != 0) &&
      pca::radius_feat_supported((int)n, (int)m, (int)d, (int)num_segments,
                                 (int)slots, r16);
  Carver ws(workspace);
  void *packed_rows = nullptr;
  if (matrix_cores)
    packed_rows =
        ws.take<char>(pca::radius_mc_scratch_bytes((int)n, (int)d));
  else if (feature_space)
    packed_rows = ws.take<char>(
        r16 != 0 ? pca::knn_feat16_scratch_bytes((int)n, (int)m, (int)d,
                                                 (int)num_segments, (int)slots)
                 : pca::knn_feat_scratch_bytes((int)n, (int)m, (int)d,
                                               (int)num_segments, (int)slots));
  int *work_start = ws.take<int>((size_t)num_segments + 1);
  pca::DenseResult dense;
  dense.idx = ws.take<int>((size_t)m * slots);
  dense.dist = nullptr;
  dense.count = ws.take<int>((size_t)m);
  dense.slots = (int)slots;
  void *compact_ws = ws.take<char>(pca::compact_workspace_bytes((int)m));
  pca::SegmentSource src;
  const bool by_id = (edge_flags & PCA_SEGMENTS_BY_ID) != 0 && ptr_x != nullptr;
  if (by_id)
    src = segments_by_id(ptr_x, ptr_y, n, m, num_segments,
                         ws.take<char>(segment_pointer_bytes(num_segments)));

  // r * r in double, narrowed to the element type at the launch
  // (csrc/cuda/radius_cuda.cu:90)
  const float r2 = (float)(r * r);

  pca::SearchInput in{x,      y,      ptr_x,  ptr_y,
                      (int)n, (int)m, (int)d, (int)num_segments};
  const int per_item = matrix_cores    ? pca::kRadiusMcTileQueries
                       : feature_space ? pca::kMfmaTileQueries
                                       : pca::kRadiusQueriesPerWave;
  int rc = PCA_OK;
  // (the matrix-core path plans its work in the launch that packs the rows)
  if (!matrix_cores)
    rc = check_launch(pca::launch_plan(ptr_y, (int)m, (int)num_segments,
                                       per_item, work_start, stream,
                                       by_id ? &src : nullptr),
                      "plan_kernel");
  if (rc != PCA_OK)
    return rc;
  const int bound =
      pca::plan_upper_bound((int)m, (int)num_segments, per_item);
  if (!matrix_cores && !feature_space)
    timer.begin();
  if (matrix_cores || feature_space)
    pca::compact_hints(dense, (int)m, compact_ws, false);
  if (feature_space) {
    const pca::FeatRadius radius{
        r16 != 0 ? pca::narrow_r2_16bit(r * r, r16 == 2) : r2,
        ignore_same_index != 0};
    rc = check_launch(pca::launch_knn_feat(in, (int)slots, false, work_start,
                                           packed_rows, dense, timer.start,
                                           timer.stop, stream, r16, &radius),
                      "knn_feat_small_kernel (radius)");
    timer.stop = nullptr;
  } else if (matrix_cores)
    rc = check_launch(pca::launch_radius_mc(in, r2, ignore_same_index != 0,
                                            work_start, bound, packed_rows,
                                            dense, timer.start, stream,
                                            by_id ? &src : nullptr),
                      "radius_mc_kernel");
  else if (dtype == PCA_F32)
    rc = check_launch(pca::launch_radius(in, r2, ignore_same_index != 0,
                                         work_start, bound, dense, stream),
                      "radius_kernel");
  else
    rc = check_launch(pca::launch_radius_anytype(dtype, in, r,
                                                 ignore_same_index != 0,
                                                 work_start, bound, dense,
                                                 stream),
                      "radius_any_kernel");
  timer.done();
  if (rc != PCA_OK)
    return rc;
  return check_launch(
      pca::launch_compact(dense, (int)m, edges, num_edges, nullptr,
                          compact_ws, stream, false,
                          (edge_flags & PCA_EDGES_X_FIRST) != 0),
      "compaction kernels");
}

size_t pca_radius_binned_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                         int64_t num_segments,
                                         int64_t max_num_neighbors) {
  if (num_segments < 1)
    num_segments = 1;
  const int64_t slots = pca_radius_slots(n, max_num_neighbors);
  if (!sizes_ok(n, m, d, num_segments) || n == 0 || m == 0 ||
      !pca::radius_binned_supported((int)d, (int)slots))
    return 0;
  return radius_binned_workspace(n, m, num_segments, slots);
}

int pca_radius_binned(const void *x, const void *y, const int64_t *ptr_x,
                      const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                      int64_t num_segments, double r,
                      int64_t max_num_neighbors, int ignore_same_index,
                      int edge_flags, int64_t *edges, int64_t *num_edges,
                      void *workspace, size_t workspace_bytes, void *stream_) {
  g_last_error[0] = 0;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (being_captured(stream))
    return refuse_capture("pca_radius_binned");
  SearchTimer timer(stream);
  if ((ptr_x == nullptr) != (ptr_y == nullptr))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "ptr_x and ptr_y must both be given or both be NULL");
  if (ptr_x == nullptr)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "bad sizes n=%lld m=%lld d=%lld num_segments=%lld",
                (long long)n, (long long)m, (long long)d,
                (long long)num_segments);
  if (max_num_neighbors < 1)
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "max_num_neighbors must be >= 1, got %lld",
                (long long)max_num_neighbors);
  if (!edge_flags_ok(edge_flags))
    return fail(PCA_ERR_INVALID_ARGUMENT, "unknown edge flags %d", edge_flags);
  if (edge_flags & PCA_EDGES_DROP_SELF)
    ignore_same_index = 1;
  if (num_edges == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "num_edges is NULL");
  if (n == 0 || m == 0) {
    hipLaunchKernelGGL(set_i64_kernel, dim3(1), dim3(1), 0, stream, num_edges,
                       (int64_t)0);
    return check_launch(hipGetLastError(), "set_i64_kernel");
  }
  const int64_t slots = pca_radius_slots(n, max_num_neighbors);
  if (!pca::radius_binned_supported((int)d, (int)slots))
    return fail(PCA_ERR_UNSUPPORTED,
                "binned search: fp32 points of up to 3 dimensions and at most "
                "64 neighbours per query, got d=%lld slots=%lld",
                (long long)d, (long long)slots);
  if (x == nullptr || y == nullptr || edges == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "x, y or edges is NULL");
  const size_t need = radius_binned_workspace(n, m, num_segments, slots);
  if (workspace == nullptr || ((uintptr_t)workspace & 255) != 0 ||
      workspace_bytes < need)
    return fail(PCA_ERR_WORKSPACE, "workspace needs %zu bytes, 256-aligned",
                need);

  Carver carve(workspace);
  void *scratch = carve.take<char>(pca::knn_binned_scratch_bytes(
      (int)n, (int)m, (int)num_segments));
  pca::DenseResult dense;
  dense.idx = carve.take<int>((size_t)m * (size_t)slots);
  dense.dist = nullptr;
  dense.count = carve.take<int>((size_t)m);
  dense.slots = (int)slots;
  void *compact_ws = carve.take<char>(pca::compact_workspace_bytes((int)m));

  // r * r in double, narrowed to the element type at the launch
  // (csrc/cuda/radius_cuda.cu:90)
  const float r2 = (float)(r * r);
  pca::SearchInput in{x,      y,      ptr_x,  ptr_y,
                      (int)n, (int)m, (int)d, (int)num_segments};
  timer.begin();
  int rc = check_launch(pca::launch_radius_binned(in, r2,
                                                  ignore_same_index != 0,
                                                  scratch, dense, stream),
                        "binned search");
  timer.done();
  if (rc != PCA_OK)
    return rc;
  return check_launch(
      pca::launch_compact(dense, (int)m, edges, num_edges, nullptr,
                          compact_ws, stream, false,
                          (edge_flags & PCA_EDGES_X_FIRST) != 0),
      "compaction kernels");
}

size_t pca_nearest_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                   int64_t num_segments, int dtype) {
  if (num_segments < 1)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments) || !nearest_dtype_ok(dtype))
    return 0;
  return nearest_workspace(n, m, d, num_segments, dtype);
}

int pca_nearest(const void *x, const void *y, const int64_t *ptr_x,
                const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                int64_t num_segments, int dtype, int64_t *out,
                void *workspace, size_t workspace_bytes, void *stream_) {
  g_last_error[0] = 0;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  SearchTimer timer(stream);
  if ((ptr_x == nullptr) != (ptr_y == nullptr))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "ptr_x and ptr_y must both be given or both be NULL");
  if (ptr_x == nullptr)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "bad sizes n=%lld m=%lld d=%lld num_segments=%lld",
                (long long)n, (long long)m, (long long)d,
                (long long)num_segments);
  if (!dtype_ok(dtype))
    return fail(PCA_ERR_INVALID_ARGUMENT, "unknown element type %d", dtype);
  if (!nearest_dtype_ok(dtype))
    return fail(PCA_ERR_UNSUPPORTED,
                "nearest is built for fp32, fp64 and fp16 points");
  if (n == 0)
    return PCA_OK;
  if (out == nullptr || x == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "x or out is NULL");
  if (m == 0) {
    // no candidate anywhere: every row keeps the reference's initial index
    hipLaunchKernelGGL(fill_i64_kernel, dim3((unsigned)((n + 255) / 256)),
                       dim3(256), 0, stream, out, n, (int64_t)0);
    return check_launch(hipGetLastError(), "fill_i64_kernel");
  }
  if (y == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "y is NULL");
  const size_t need = nearest_workspace(n, m, d, num_segments, dtype);
  if (workspace == nullptr || ((uintptr_t)workspace & 255) != 0 ||
      workspace_bytes < need)
    return fail(PCA_ERR_WORKSPACE, "workspace needs %zu bytes, 256-aligned",
                need);

  // the search kernels call the searched rows x and the searching rows y
  pca::SearchInput in{y,      x,      ptr_y,  ptr_x,
                      (int)m, (int)n, (int)d, (int)num_segments};
  Carver ws(workspace);
  int *work_start = ws.take<int>((size_t)num_segments + 1);
  const bool low_d = nearest_low_d(d, dtype);
  const bool mfma = nearest_mfma(d, dtype);
  pca::KnnLowdConfig cfg;
  int per_item = mfma ? pca::kMfmaTileQueries : pca::kBlock;
  if (low_d) {
    cfg = pca::nearest_lowd_config((int)d, (int)m, (int)n, (int)num_segments);
    per_item = cfg.tile_queries;
  }
  int rc = PCA_OK;
  if (!low_d)
    rc = check_launch(pca::launch_plan(ptr_x, (int)n, (int)num_segments,
                                       per_item, work_start, stream),
                      "plan_kernel");
  if (rc != PCA_OK)
    return rc;
  if (low_d) {
    void *scratch = ws.take<char>(pca::knn_lowd_scratch_bytes(
        cfg, (int)m, (int)n, (int)d, (int)num_segments, 1));
    const pca::DenseResult none{nullptr, nullptr, nullptr, 1};
    rc = check_launch(pca::launch_knn_lowd(in, 1, false, cfg, work_start,
                                           scratch, none, timer.start,
                                           timer.stop, stream, out),
                      "knn_lowd_mc_kernel (nearest)");
    timer.stop = nullptr;
    return rc;
  }
  if (mfma) {
    void *scratch = ws.take<char>(pca::knn_mfma_scratch_bytes(
        (int)m, (int)n, (int)d, (int)num_segments, 1));
    const pca::DenseResult none{nullptr, nullptr, nullptr, 1};
    rc = check_launch(pca::launch_knn_mfma(in, 1, false, work_start, scratch,
                                           none, timer.start, timer.stop,
                                           stream, out),
                      "knn_mfma_kernel (nearest)");
    timer.stop = nullptr;
    return rc;
  }
  const int bound =
      pca::plan_upper_bound((int)n, (int)num_segments, per_item);
  timer.begin();
  rc = check_launch(pca::launch_nearest_any(dtype, in, work_start, bound, out,
                                            stream),
                    "nearest_any_kernel");
  timer.done();
  return rc;
}

size_t pca_nearest_binned_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                          int64_t num_segments) {
  if (num_segments < 1)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments) || n == 0 || m == 0 || d > 3)
    return 0;
  // (the searched rows, m of them, are the ones that get binned)
  return align256(
      pca::knn_binned_scratch_bytes((int)m, (int)n, (int)num_segments));
}

int pca_nearest_binned(const void *x, const void *y, const int64_t *ptr_x,
                       const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                       int64_t num_segments, int64_t *out, void *workspace,
                       size_t workspace_bytes, void *stream_) {
  g_last_error[0] = 0;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (being_captured(stream))
    return refuse_capture("pca_nearest_binned");
  SearchTimer timer(stream);
  if ((ptr_x == nullptr) != (ptr_y == nullptr))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "ptr_x and ptr_y must both be given or both be NULL");
  if (ptr_x == nullptr)
    num_segments = 1;
  if (!sizes_ok(n, m, d, num_segments))
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "bad sizes n=%lld m=%lld d=%lld num_segments=%lld",
                (long long)n, (long long)m, (long long)d,
                (long long)num_segments);
  if (d > 3)
    return fail(PCA_ERR_UNSUPPORTED,
                "binned search: fp32 points of up to 3 dimensions, got d=%lld",
                (long long)d);
  if (n == 0)
    return PCA_OK;
  if (out == nullptr || x == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "x or out is NULL");
  if (m == 0) {
    // no candidate anywhere: every row keeps the reference's initial index
    hipLaunchKernelGGL(fill_i64_kernel, dim3((unsigned)((n + 255) / 256)),
                       dim3(256), 0, stream, out, n, (int64_t)0);
    return check_launch(hipGetLastError(), "fill_i64_kernel");
  }
  if (y == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "y is NULL");
  const size_t need = align256(
      pca::knn_binned_scratch_bytes((int)m, (int)n, (int)num_segments));
  if (workspace == nullptr || ((uintptr_t)workspace & 255) != 0 ||
      workspace_bytes < need)
    return fail(PCA_ERR_WORKSPACE, "workspace needs %zu bytes, 256-aligned",
                need);
  // the search kernels call the searched rows x and the searching rows y
  pca::SearchInput in{y,      x,      ptr_y,  ptr_x,
                      (int)m, (int)n, (int)d, (int)num_segments};
  const int rc = check_launch(
      pca::launch_nearest_binned(in, workspace, out, timer.start, timer.stop,
                                 stream),
      "binned search (nearest)");
  timer.stop = nullptr;
  return rc;
}

size_t pca_fps_workspace_bytes(int64_t n, int64_t d, int64_t num_segments,
                               int64_t max_segment_rows, int dtype) {
  if (n < 0 || n > kMaxRows || d < 1 || d > (1 << 20) || num_segments < 1 ||
      !nearest_dtype_ok(dtype))
    return 0;
  if (pca::fps_in_registers(dtype, (int)d, max_segment_rows))
    return 256;
  return align256(pca::fps_dist_bytes(n)) + 256;
}

int pca_fps(const void *src, const int64_t *ptr, const int64_t *out_ptr,
            const int64_t *start, int64_t n, int64_t d, int64_t num_segments,
            int64_t max_segment_rows, int dtype, int64_t *out, void *workspace,
            size_t workspace_bytes, void *stream_) {
  g_last_error[0] = 0;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (n < 0 || n > kMaxRows || d < 1 || d > (1 << 20) || num_segments < 1 ||
      num_segments > kMaxRows)
    return fail(PCA_ERR_INVALID_ARGUMENT,
                "bad sizes n=%lld d=%lld num_segments=%lld", (long long)n,
                (long long)d, (long long)num_segments);
  if (!dtype_ok(dtype))
    return fail(PCA_ERR_INVALID_ARGUMENT, "unknown element type %d", dtype);
  if (!nearest_dtype_ok(dtype))
    return fail(PCA_ERR_UNSUPPORTED,
                "fps is built for fp32, fp64 and fp16 points");
  if (ptr == nullptr || out_ptr == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "ptr or out_ptr is NULL");
  if (n == 0)
    return PCA_OK;
  if (src == nullptr || out == nullptr)
    return fail(PCA_ERR_INVALID_ARGUMENT, "src or out is NULL");
  const size_t need =
      pca_fps_workspace_bytes(n, d, num_segments, max_segment_rows, dtype);
  if (workspace == nullptr || ((uintptr_t)workspace & 255) != 0 ||
      workspace_bytes < need)
    return fail(PCA_ERR_WORKSPACE, "workspace needs %zu bytes, 256-aligned",
                need);
  return check_launch(pca::launch_fps(dtype, src, ptr, out_ptr, start, (int)d,
                                      (int)num_segments, max_segment_rows,
                                      workspace, out, stream),
                      "fps kernel");
}

} // extern "C"
