// TorchScript operator binding: registers `torch_cluster::knn`,
// `torch_cluster::radius`, `torch_cluster::nearest` and `torch_cluster::fps`
// with the reference's operator signatures (csrc/knn.cpp:22-40,
// csrc/radius.cpp:22-39, csrc/nearest.cpp:22-39, csrc/fps.cpp:22-41) on top of
// the C ABI in
// include/pca_neighbors.h.  Tensor validation, allocation through PyTorch's
// caching allocator, the current HIP stream and the single host read of the
// edge count live here; the kernels never see a torch type.
//
// Validation and error texts follow the reference's GPU host wrappers
// (csrc/cuda/knn_cuda.cu:91-114, csrc/cuda/radius_cuda.cu:49-73,
// csrc/cuda/utils.cuh:5-9).  Tensors that are not on a GPU take the host
// searches (pca_knn_host / pca_radius_host), as the reference's dispatchers
// send them to knn_cpu / radius_cpu (csrc/knn.cpp:26-36,
// csrc/radius.cpp:27-35); `nearest` and `fps` are GPU-only here.
#include <ATen/ATen.h>
#include <ATen/Parallel.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <hip/hip_version.h>
#include <torch/library.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <optional>
#include <string>

#include "../../include/pca_neighbors.h"

namespace {

#define PCA_CHECK_GPU(x)                                                       \
  TORCH_CHECK((x).device().is_cuda(), #x " must be CUDA tensor")
#define PCA_CHECK_CONTIGUOUS(x)                                                \
  TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define PCA_CHECK_INPUT(cond) TORCH_CHECK(cond, "Input mismatch")

int dtype_code(const at::Tensor &x) {
  switch (x.scalar_type()) {
  case at::kFloat:
    return PCA_F32;
  case at::kDouble:
    return PCA_F64;
  case at::kHalf:
    return PCA_F16;
  case at::kBFloat16:
    return PCA_BF16;
  default:
    TORCH_CHECK(false, "unsupported element type ", x.scalar_type());
  }
}

// Restores the previously current device when it goes out of scope
// (the reference calls c10::cuda::MaybeSetDevice, knn_cuda.cu:116).
struct DeviceScope {
  int previous = -1;
  explicit DeviceScope(int device) {
    TORCH_CHECK(hipGetDevice(&previous) == hipSuccess, "hipGetDevice failed");
    if (previous != device) {
      TORCH_CHECK(hipSetDevice(device) == hipSuccess, "hipSetDevice failed");
    } else {
      previous = -1;
    }
  }
  ~DeviceScope() {
    if (previous >= 0)
      (void)hipSetDevice(previous);
  }
};

void check_status(int status) {
  if (status == PCA_OK)
    return;
  const char *detail = pca_last_error();
  TORCH_CHECK(false, (detail && detail[0]) ? detail
                                           : pca_status_string(status));
}

struct Segments {
  const int64_t *ptr_x = nullptr;
  const int64_t *ptr_y = nullptr;
  int64_t count = 1;
  at::Tensor keep_x, keep_y;
};

// One missing pointer is replaced by [0, N] like the reference does
// (knn_cuda.cu:100-112); both missing = one segment, no device array needed.
Segments resolve_segments(const at::Tensor &x, const at::Tensor &y,
                          std::optional<at::Tensor> ptr_x,
                          std::optional<at::Tensor> ptr_y) {
  Segments s;
  if (ptr_x.has_value()) {
    PCA_CHECK_GPU(ptr_x.value());
    PCA_CHECK_INPUT(ptr_x.value().dim() == 1);
  }
  if (ptr_y.has_value()) {
    PCA_CHECK_GPU(ptr_y.value());
    PCA_CHECK_INPUT(ptr_y.value().dim() == 1);
  }
  if (!ptr_x.has_value() && !ptr_y.has_value())
    return s;
  if (!ptr_x.has_value())
    ptr_x = at::arange(0, x.size(0) + 1, x.size(0),
                       x.options().dtype(at::kLong));
  if (!ptr_y.has_value())
    ptr_y = at::arange(0, y.size(0) + 1, y.size(0),
                       y.options().dtype(at::kLong));
  PCA_CHECK_INPUT(ptr_x.value().numel() == ptr_y.value().numel());
  PCA_CHECK_INPUT(ptr_x.value().numel() >= 2);
  s.keep_x = ptr_x.value().to(at::kLong).contiguous();
  s.keep_y = ptr_y.value().to(at::kLong).contiguous();
  s.ptr_x = s.keep_x.data_ptr<int64_t>();
  s.ptr_y = s.keep_y.data_ptr<int64_t>();
  s.count = s.keep_x.numel() - 1;
  return s;
}

// Segments given as the sorted example ids of the rows (what the Python entry
// points receive as batch_x / batch_y) with the number of examples: the
// pointers are derived on the device, in the launch that prepares the search
// (PCA_SEGMENTS_BY_ID), instead of by two bucketize calls before it
// (torch_cluster/knn.py:75-79).
Segments segments_by_id(const at::Tensor &x, const at::Tensor &y,
                        const at::Tensor &batch_x, const at::Tensor &batch_y,
                        int64_t batch_size) {
  PCA_CHECK_GPU(batch_x);
  PCA_CHECK_GPU(batch_y);
  PCA_CHECK_INPUT(batch_x.dim() == 1 && batch_x.numel() == x.size(0));
  PCA_CHECK_INPUT(batch_y.dim() == 1 && batch_y.numel() == y.size(0));
  TORCH_CHECK(batch_size >= 1, "`batch_size` needs to be positive");
  Segments s;
  s.keep_x = batch_x.to(at::kLong).contiguous();
  s.keep_y = batch_y.to(at::kLong).contiguous();
  s.ptr_x = s.keep_x.data_ptr<int64_t>();
  s.ptr_y = s.keep_y.data_ptr<int64_t>();
  s.count = batch_size;
  return s;
}

// For the entry points that take pointers only: the pointers of `ids` in a
// tensor of their own (one small launch).
void pointers_for(Segments &s, int64_t n, int64_t m, hipStream_t stream) {
  auto both = at::empty({2, s.count + 1}, s.keep_x.options());
  int64_t *px = both.data_ptr<int64_t>();
  int64_t *py = px + (s.count + 1);
  check_status(
      pca_segment_pointers(s.ptr_x, n, s.ptr_y, m, s.count, px, py, stream));
  s.keep_x = both;
  s.keep_y = both;
  s.ptr_x = px;
  s.ptr_y = py;
}

// The edge count in pinned host memory (PyTorch keeps such blocks for reuse):
// the kernel that knows E writes it there, and the operator waits for the
// stream instead of queueing a copy behind it.
at::Tensor edge_count_slot() {
  return at::empty({1}, at::TensorOptions().dtype(at::kLong).pinned_memory(
                            true));
}

// Waits of the host for the device that the operators of this library have
// made (for tests and profiles: the default calls are meant to make one).
std::atomic<int64_t> g_host_waits{0};
int64_t host_waits() { return g_host_waits.load(); }

// Until an operator has waited for its stream the kernels it queued may still
// write the edge count: on every way out before that wait -- an exception
// after some kernels were queued -- the stream is waited for here, so that
// the pinned slot is not handed to a later call while a kernel of this one
// can still write it.
struct SlotGuard {
  hipStream_t stream;
  bool armed = true;
  explicit SlotGuard(hipStream_t s) : stream(s) {}
  ~SlotGuard() {
    if (armed)
      (void)hipStreamSynchronize(stream);
  }
};

// The size of an edge list depends on the data: the operators read it from
// the device before they return, which a stream that is being captured into
// a graph cannot do.
void refuse_capture(hipStream_t stream, const char *op) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  TORCH_CHECK(status == hipStreamCaptureStatusNone, op,
              " cannot be captured into a graph: the size of its result "
              "depends on the data (call pca_knn / pca_radius of the C ABI "
              "with buffers of the largest size instead)");
}

at::Tensor finish(const at::Tensor &edges, const at::Tensor &num_edges,
                  hipStream_t stream) {
  // the only host synchronisation of the operator: the edge count sizes the
  // result (the reference synchronises in its masked_selects)
  TORCH_CHECK(hipStreamSynchronize(stream) == hipSuccess,
              "hipStreamSynchronize failed");
  g_host_waits += 1;
  const int64_t E = *num_edges.data_ptr<int64_t>();
  at::Tensor out = edges.narrow(0, 0, 2 * E).view({2, E});
  // (a view keeps the whole slot buffer alive: a result that fills less than
  // half of it gets storage of its own, like the reference's [2, E])
  if (4 * E < edges.numel())
    out = out.clone();
  return out;
}

// ---- tensors that are not on a GPU ---------------------------------------

#define PCA_CHECK_CPU(x)                                                       \
  TORCH_CHECK((x).device().is_cpu(), #x " must be CPU tensor")

struct HostPoints {
  at::Tensor x, y, ptr_x, ptr_y;
  const int64_t *px = nullptr, *py = nullptr;
  int64_t segments = 1;
  int dtype = PCA_F32;
};

// Checks of csrc/cpu/knn_cpu.cpp:12-24 / radius_cpu.cpp:13-25; integer points
// are searched as doubles (their squared distances are exact there).
HostPoints host_points(at::Tensor x, at::Tensor y,
                       std::optional<at::Tensor> ptr_x,
                       std::optional<at::Tensor> ptr_y) {
  PCA_CHECK_CPU(x);
  PCA_CHECK_INPUT(x.dim() == 2);
  PCA_CHECK_CPU(y);
  PCA_CHECK_INPUT(y.dim() == 2);
  PCA_CHECK_INPUT(x.size(1) == y.size(1));
  PCA_CHECK_INPUT(x.scalar_type() == y.scalar_type());
  HostPoints h;
  if (ptr_x.has_value()) {
    PCA_CHECK_CPU(ptr_x.value());
    PCA_CHECK_INPUT(ptr_x.value().dim() == 1);
  }
  if (ptr_y.has_value()) {
    PCA_CHECK_CPU(ptr_y.value());
    PCA_CHECK_INPUT(ptr_y.value().dim() == 1);
  }
  if (!at::isFloatingType(x.scalar_type())) {
    x = x.to(at::kDouble);
    y = y.to(at::kDouble);
  }
  h.x = x.contiguous();
  h.y = y.contiguous();
  h.dtype = dtype_code(h.x);
  if (ptr_x.has_value() || ptr_y.has_value()) {
    if (!ptr_x.has_value())
      ptr_x = at::arange(0, x.size(0) + 1, x.size(0), at::kLong);
    if (!ptr_y.has_value())
      ptr_y = at::arange(0, y.size(0) + 1, y.size(0), at::kLong);
    PCA_CHECK_INPUT(ptr_x.value().numel() == ptr_y.value().numel());
    PCA_CHECK_INPUT(ptr_x.value().numel() >= 2);
    h.ptr_x = ptr_x.value().to(at::kLong).contiguous();
    h.ptr_y = ptr_y.value().to(at::kLong).contiguous();
    h.px = h.ptr_x.data_ptr<int64_t>();
    h.py = h.ptr_y.data_ptr<int64_t>();
    h.segments = h.ptr_x.numel() - 1;
  }
  return h;
}

int host_threads(int64_t num_workers) {
  return (int)std::max<int64_t>(std::max<int64_t>(num_workers, 1),
                                at::get_num_threads());
}

void check_host_status(int status) {
  if (status == PCA_OK)
    return;
  const char *detail = pca_host_last_error();
  TORCH_CHECK(false, (detail && detail[0]) ? detail
                                           : pca_status_string(status));
}

at::Tensor host_result(const at::Tensor &edges, int64_t E) {
  at::Tensor out = edges.narrow(0, 0, 2 * E).view({2, E});
  return 4 * E < edges.numel() ? out.clone() : out;
}

at::Tensor knn_host(at::Tensor x, at::Tensor y,
                    std::optional<at::Tensor> ptr_x,
                    std::optional<at::Tensor> ptr_y, int64_t k, bool cosine,
                    int flags, int64_t num_workers) {
  // csrc/knn.cpp:33-34
  TORCH_CHECK(!cosine, "`cosine` argument not supported on CPU");
  TORCH_CHECK(k >= 1, "`k` needs to be positive");
  HostPoints h = host_points(x, y, ptr_x, ptr_y);
  const int64_t n = h.x.size(0), m = h.y.size(0), d = h.x.size(1);
  auto long_opts = at::TensorOptions().dtype(at::kLong);
  if (n == 0 || m == 0)
    return at::empty({2, 0}, long_opts);
  auto edges = at::empty({2 * m * std::min(k, n)}, long_opts);
  int64_t E = 0;
  check_host_status(pca_knn_host(
      h.x.data_ptr(), h.y.data_ptr(), h.px, h.py, n, m, d, h.segments, k,
      h.dtype, flags, host_threads(num_workers), edges.data_ptr<int64_t>(),
      &E, nullptr));
  return host_result(edges, E);
}

at::Tensor radius_host(at::Tensor x, at::Tensor y,
                       std::optional<at::Tensor> ptr_x,
                       std::optional<at::Tensor> ptr_y, double r,
                       int64_t max_num_neighbors, bool ignore_same_index,
                       int flags, int64_t num_workers) {
  TORCH_CHECK(max_num_neighbors >= 1,
              "`max_num_neighbors` needs to be positive");
  HostPoints h = host_points(x, y, ptr_x, ptr_y);
  const int64_t n = h.x.size(0), m = h.y.size(0), d = h.x.size(1);
  auto long_opts = at::TensorOptions().dtype(at::kLong);
  if (n == 0 || m == 0)
    return at::empty({2, 0}, long_opts);
  auto edges =
      at::empty({2 * m * pca_radius_slots(n, max_num_neighbors)}, long_opts);
  int64_t E = 0;
  check_host_status(pca_radius_host(
      h.x.data_ptr(), h.y.data_ptr(), h.px, h.py, n, m, d, h.segments, r,
      max_num_neighbors, ignore_same_index ? 1 : 0, h.dtype, flags,
      host_threads(num_workers), edges.data_ptr<int64_t>(), &E));
  return host_result(edges, E);
}

int edge_flags(bool drop_self, bool x_first) {
  return (drop_self ? PCA_EDGES_DROP_SELF : 0) |
         (x_first ? PCA_EDGES_X_FIRST : 0);
}

// How a search over fp32 points of up to 3 dimensions goes about it: "scan"
// looks at every row of the segment (pca_knn, pca_radius), "binned" at the
// rows near the query (pca_knn_binned: Euclidean, k <= 64; pca_radius_binned:
// at most 64 neighbours per query - anything else is scanned).  Same edges
// either way.  "auto" - the default - bins when that is expected to pay off
// (bins_wanted).  Process-wide; the environment variable PCA_SEARCH_STRATEGY
// sets the initial value.
enum Strategy { kScan = 0, kBinned = 1, kAuto = 2 };

int strategy_code(const std::string &name) {
  if (name == "scan")
    return kScan;
  if (name == "binned")
    return kBinned;
  if (name == "auto")
    return kAuto;
  return -1;
}

std::atomic<int> g_strategy{[] {
  const char *e = std::getenv("PCA_SEARCH_STRATEGY");
  const int code = e != nullptr ? strategy_code(e) : kAuto;
  return code < 0 ? (int)kAuto : code;
}()};

void set_search_strategy(std::string name) {
  const int code = strategy_code(name);
  TORCH_CHECK(code >= 0, "search strategy is 'scan', 'binned' or 'auto', got '",
              name, "'");
  g_strategy.store(code);
}

std::string get_search_strategy() {
  const int code = g_strategy.load();
  return code == kBinned ? "binned" : code == kAuto ? "auto" : "scan";
}

// The estimates of "auto" per operator, fitted to whole calls on an MI355X
// (`python bench.py --extras-only --case crossover` measures both strategies
// over uniform clouds of 2,048 - 262,144 points in 1 and 8 examples and
// reports where the pick loses).
struct SearchCost {
  double scan_rate;   // pairs per ms the scan looks at
  double query_us;    // binned search: us per searching row
  double binned_base; // binned search: ms before the first row counts
};
// kNN ~3 G pairs/ms (between its small-cloud and large-cloud rates); radius and
// nearest ~10 G (the radius scan stops at max_num_neighbors, nearest keeps one
// neighbour); a binned radius call starts sooner than a binned kNN call (no
// tasks to order).
constexpr SearchCost kKnnCost{3e9, 2e-3, 0.2};
constexpr SearchCost kRadiusCost{1e10, 0.5e-3, 0.13};
constexpr SearchCost kNearestCost{1e10, 0.5e-3, 0.2};

// searched: rows that get binned (x of knn / radius, y of nearest);
// searching: the rows that look for neighbours.  "auto" compares two rough
// estimates in ms: the scan looks at every pair of a segment (segments taken
// as equal) at scan_rate pairs per ms, binning costs a sort of both sides and
// a search that grows with their sizes.  It picks the scan for clouds of a few
// thousand points and for a handful of queries against many rows, bins from
// some ten thousand rows per segment on.
bool bins_wanted(int64_t searched, int64_t searching, int64_t num_segments,
                 const SearchCost &cost) {
  const int code = g_strategy.load();
  if (code != kAuto)
    return code == kBinned;
  const double pairs = (double)searched * (double)searching /
                       (double)std::max<int64_t>(num_segments, 1);
  const double scan_ms = 0.1 + pairs / cost.scan_rate;
  const double binned_ms = cost.binned_base + 1e-6 * (double)searched +
                           1e-3 * cost.query_us * (double)searching;
  return scan_ms > binned_ms;
}

// A stream that is being captured into a graph takes the scanning kernels:
// the binned entry points refuse capture.
bool being_captured(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

// What the current strategy picks for an operator ("knn", "radius",
// "nearest") and these sizes, when the points qualify for binning at all
// (fp32, up to 3 dimensions, Euclidean): "scan" or "binned".
std::string strategy_for(std::string op, int64_t searched, int64_t searching,
                         int64_t num_segments) {
  const SearchCost *cost = op == "knn"       ? &kKnnCost
                           : op == "radius"  ? &kRadiusCost
                           : op == "nearest" ? &kNearestCost
                                             : nullptr;
  TORCH_CHECK(cost != nullptr, "operator is 'knn', 'radius' or 'nearest', got '",
              op, "'");
  return bins_wanted(searched, searching, num_segments, *cost)
             ? "binned"
             : "scan";
}

at::Tensor knn_search(at::Tensor x, at::Tensor y,
                      std::optional<at::Tensor> ptr_x,
                      std::optional<at::Tensor> ptr_y, int64_t k, bool cosine,
                      int flags, int64_t num_workers = 1,
                      int64_t ids_examples = 0,
                      int64_t *examples_report = nullptr) {
  // ids_examples > 0: ptr_x / ptr_y hold the rows' example ids, that many
  // examples (GPU tensors only); examples_report: where the launch that
  // derives the pointers leaves the largest id + 1 (pinned host memory)
  // the device branch of csrc/knn.cpp:26-36
  if (!x.device().is_cuda()) {
    TORCH_CHECK(ids_examples == 0, "example ids are taken for GPU tensors");
    return knn_host(x, y, ptr_x, ptr_y, k, cosine, flags, num_workers);
  }
  PCA_CHECK_GPU(x);
  PCA_CHECK_CONTIGUOUS(x);
  PCA_CHECK_INPUT(x.dim() == 2);
  PCA_CHECK_GPU(y);
  PCA_CHECK_CONTIGUOUS(y);
  PCA_CHECK_INPUT(y.dim() == 2);
  PCA_CHECK_INPUT(x.size(1) == y.size(1));
  PCA_CHECK_INPUT(x.scalar_type() == y.scalar_type());
  PCA_CHECK_INPUT(x.get_device() == y.get_device());
  TORCH_CHECK(k <= PCA_KNN_MAX_K, "`k` needs to smaller than or equal to 100");
  TORCH_CHECK(k >= 1, "`k` needs to be positive");

  Segments seg = ids_examples > 0
                     ? segments_by_id(x, y, ptr_x.value(), ptr_y.value(),
                                      ids_examples)
                     : resolve_segments(x, y, ptr_x, ptr_y);
  DeviceScope scope(x.get_device());
  auto long_opts = x.options().dtype(at::kLong);
  const int64_t n = x.size(0), m = y.size(0), d = x.size(1);
  if (n == 0 || m == 0)
    return at::empty({2, 0}, long_opts);

  refuse_capture(c10::hip::getCurrentHIPStream(x.get_device()).stream(),
                 "knn");
  const int dtype = dtype_code(x);
  const bool binned = bins_wanted(n, m, seg.count, kKnnCost) &&
                      dtype == PCA_F32 && !cosine && d <= 3 && k <= 64;
  const size_t ws_bytes =
      binned ? pca_knn_binned_workspace_bytes(n, m, d, seg.count, k)
             : pca_knn_workspace_bytes(n, m, d, seg.count, k, dtype);
  TORCH_CHECK(ws_bytes > 0, "problem size not supported");
  auto workspace =
      at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
  auto edges = at::empty({2 * m * k}, long_opts);
  auto num_edges = edge_count_slot();

  hipStream_t stream = c10::hip::getCurrentHIPStream(x.get_device()).stream();
  SlotGuard guard(stream);
  if (ids_examples > 0) {
    (void)pca_report_examples(examples_report);
    if (binned)
      pointers_for(seg, n, m, stream);
    else
      flags |= PCA_SEGMENTS_BY_ID;
  }
  if (binned) {
    check_status(pca_knn_binned(x.data_ptr(), y.data_ptr(), seg.ptr_x,
                                seg.ptr_y, n, m, d, seg.count, k, flags,
                                edges.data_ptr<int64_t>(),
                                num_edges.data_ptr<int64_t>(), nullptr,
                                workspace.data_ptr(), ws_bytes, stream));
    guard.armed = false; // (finish waits for the stream itself)
    return finish(edges, num_edges, stream);
  }
  check_status(pca_knn(x.data_ptr(), y.data_ptr(), seg.ptr_x, seg.ptr_y, n, m,
                       d, seg.count, k, cosine ? 1 : 0, dtype, flags,
                       edges.data_ptr<int64_t>(),
                       num_edges.data_ptr<int64_t>(), nullptr,
                       workspace.data_ptr(), ws_bytes, stream));
  guard.armed = false;
  return finish(edges, num_edges, stream);
}

at::Tensor knn(at::Tensor x, at::Tensor y, std::optional<at::Tensor> ptr_x,
               std::optional<at::Tensor> ptr_y, int64_t k, bool cosine,
               int64_t num_workers) {
  // (num_workers: unused by the reference, csrc/cpu/knn_cpu.cpp; here the
  // host search runs on at least that many threads)
  return knn_search(x, y, ptr_x, ptr_y, k, cosine, 0, num_workers);
}

// The search of knn_graph with its epilogue (torch_cluster/knn.py:135-144)
// folded into the pass that writes the edges: no pairs of a row with itself
// (drop_self), neighbour row first (x_first).
at::Tensor knn_edges(at::Tensor x, at::Tensor y,
                     std::optional<at::Tensor> ptr_x,
                     std::optional<at::Tensor> ptr_y, int64_t k, bool cosine,
                     bool drop_self, bool x_first) {
  return knn_search(x, y, ptr_x, ptr_y, k, cosine,
                    edge_flags(drop_self, x_first));
}

// The number of examples of a call that was not told (batch_size < 1): the
// reference's wrappers read it from the device before they can start
// (torch_cluster/knn.py:62-72, two reductions with a host wait each).  Here
// the search starts with the number the previous call of the process met, the
// launch that derives the pointers reports the number the ids really speak
// of into pinned host memory, and the operator looks at it after the one wait
// it has anyway (for the edge count): equal or smaller, the edges are right
// (examples without rows); larger, the search runs once more with the right
// number.  Only the first call of a process reads the ids' last entries up
// front.
std::atomic<int64_t> g_examples_hint{0};

template <typename Run>
at::Tensor with_examples(const at::Tensor &batch_x, const at::Tensor &batch_y,
                         int64_t batch_size, Run run) {
  if (batch_size >= 1)
    return run(batch_size, nullptr);
  int64_t guess = g_examples_hint.load();
  if (guess < 1) {
    // (sorted ids: the last ones are the largest)
    int64_t last = -1;
    if (batch_x.numel() > 0)
      last = std::max(last, batch_x[-1].item<int64_t>());
    if (batch_y.numel() > 0 && !batch_y.is_same(batch_x))
      last = std::max(last, batch_y[-1].item<int64_t>());
    g_host_waits += 1;
    guess = std::max<int64_t>(last + 1, 1);
    g_examples_hint.store(guess);
    return run(guess, nullptr);
  }
  auto slot = at::empty({1}, at::TensorOptions().dtype(at::kLong).pinned_memory(
                                 true));
  int64_t *in_use = slot.data_ptr<int64_t>();
  *in_use = 0;
  at::Tensor out = run(guess, in_use);
  // (run has waited for the stream: the number is there)
  const int64_t met = std::max<int64_t>(*in_use, 1);
  g_examples_hint.store(met);
  if (met > guess)
    out = run(met, nullptr);
  return out;
}

// knn_edges with the segments given as the rows' sorted example ids and the
// number of examples (the prologue of torch_cluster/knn.py:62-79 folded into
// the launch that prepares the search); batch_size < 1: not known, see
// with_examples.
at::Tensor knn_batched(at::Tensor x, at::Tensor y, at::Tensor batch_x,
                       at::Tensor batch_y, int64_t batch_size, int64_t k,
                       bool cosine, bool drop_self, bool x_first) {
  return with_examples(
      batch_x, batch_y, batch_size, [&](int64_t examples, int64_t *report) {
        return knn_search(x, y, batch_x, batch_y, k, cosine,
                          edge_flags(drop_self, x_first), 1, examples, report);
      });
}

at::Tensor radius_search(at::Tensor x, at::Tensor y,
                         std::optional<at::Tensor> ptr_x,
                         std::optional<at::Tensor> ptr_y, double r,
                         int64_t max_num_neighbors, bool ignore_same_index,
                         int flags, int64_t num_workers = 1,
                         int64_t ids_examples = 0,
                         int64_t *examples_report = nullptr) {
  // (ids_examples, examples_report: as for knn_search)
  // the device branch of csrc/radius.cpp:27-35
  if (!x.device().is_cuda()) {
    TORCH_CHECK(ids_examples == 0, "example ids are taken for GPU tensors");
    return radius_host(x, y, ptr_x, ptr_y, r, max_num_neighbors,
                       ignore_same_index, flags, num_workers);
  }
  PCA_CHECK_GPU(x);
  PCA_CHECK_CONTIGUOUS(x);
  PCA_CHECK_INPUT(x.dim() == 2);
  PCA_CHECK_GPU(y);
  PCA_CHECK_CONTIGUOUS(y);
  PCA_CHECK_INPUT(y.dim() == 2);
  PCA_CHECK_INPUT(x.size(1) == y.size(1));
  PCA_CHECK_INPUT(x.scalar_type() == y.scalar_type());
  PCA_CHECK_INPUT(x.get_device() == y.get_device());
  TORCH_CHECK(max_num_neighbors >= 1,
              "`max_num_neighbors` needs to be positive");

  Segments seg = ids_examples > 0
                     ? segments_by_id(x, y, ptr_x.value(), ptr_y.value(),
                                      ids_examples)
                     : resolve_segments(x, y, ptr_x, ptr_y);
  DeviceScope scope(x.get_device());
  auto long_opts = x.options().dtype(at::kLong);
  const int64_t n = x.size(0), m = y.size(0), d = x.size(1);
  if (n == 0 || m == 0)
    return at::empty({2, 0}, long_opts);

  refuse_capture(c10::hip::getCurrentHIPStream(x.get_device()).stream(),
                 "radius");
  const int dtype = dtype_code(x);
  const int64_t slots = pca_radius_slots(n, max_num_neighbors);
  const bool binned = bins_wanted(n, m, seg.count, kRadiusCost) &&
                      dtype == PCA_F32 && d <= 3 && slots <= 64;
  const size_t ws_bytes =
      binned ? pca_radius_binned_workspace_bytes(n, m, d, seg.count,
                                                 max_num_neighbors)
             : pca_radius_workspace_bytes(n, m, d, seg.count,
                                          max_num_neighbors, dtype);
  TORCH_CHECK(ws_bytes > 0, "problem size not supported");
  auto workspace =
      at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
  auto edges = at::empty({2 * m * slots}, long_opts);
  auto num_edges = edge_count_slot();

  hipStream_t stream = c10::hip::getCurrentHIPStream(x.get_device()).stream();
  SlotGuard guard(stream);
  if (ids_examples > 0) {
    (void)pca_report_examples(examples_report);
    if (binned)
      pointers_for(seg, n, m, stream);
    else
      flags |= PCA_SEGMENTS_BY_ID;
  }
  if (binned) {
    check_status(pca_radius_binned(
        x.data_ptr(), y.data_ptr(), seg.ptr_x, seg.ptr_y, n, m, d, seg.count,
        r, max_num_neighbors, ignore_same_index ? 1 : 0, flags,
        edges.data_ptr<int64_t>(), num_edges.data_ptr<int64_t>(),
        workspace.data_ptr(), ws_bytes, stream));
    guard.armed = false; // (finish waits for the stream itself)
    return finish(edges, num_edges, stream);
  }
  check_status(pca_radius(x.data_ptr(), y.data_ptr(), seg.ptr_x, seg.ptr_y, n,
                          m, d, seg.count, r, max_num_neighbors,
                          ignore_same_index ? 1 : 0, dtype, flags,
                          edges.data_ptr<int64_t>(),
                          num_edges.data_ptr<int64_t>(), workspace.data_ptr(),
                          ws_bytes, stream));
  guard.armed = false;
  return finish(edges, num_edges, stream);
}

at::Tensor radius(at::Tensor x, at::Tensor y, std::optional<at::Tensor> ptr_x,
                  std::optional<at::Tensor> ptr_y, double r,
                  int64_t max_num_neighbors, int64_t num_workers,
                  bool ignore_same_index) {
  return radius_search(x, y, ptr_x, ptr_y, r, max_num_neighbors,
                       ignore_same_index, 0, num_workers);
}

// The search of radius_graph with the flow flip of
// torch_cluster/radius.py:143-148 folded in.
at::Tensor radius_edges(at::Tensor x, at::Tensor y,
                        std::optional<at::Tensor> ptr_x,
                        std::optional<at::Tensor> ptr_y, double r,
                        int64_t max_num_neighbors, bool ignore_same_index,
                        bool x_first) {
  return radius_search(x, y, ptr_x, ptr_y, r, max_num_neighbors,
                       ignore_same_index, edge_flags(false, x_first));
}

// radius_edges with the segments given as example ids (see knn_batched).
at::Tensor radius_batched(at::Tensor x, at::Tensor y, at::Tensor batch_x,
                          at::Tensor batch_y, int64_t batch_size, double r,
                          int64_t max_num_neighbors, bool ignore_same_index,
                          bool x_first) {
  return with_examples(
      batch_x, batch_y, batch_size, [&](int64_t examples, int64_t *report) {
        return radius_search(x, y, batch_x, batch_y, r, max_num_neighbors,
                             ignore_same_index, edge_flags(false, x_first), 1,
                             examples, report);
      });
}

// csrc/nearest.cpp:22-36 -> nearest_cuda (csrc/cuda/nearest_cuda.cu:68-94):
// both pointer tensors are required, x and y are flattened to [N, -1].
// Points that are not on a GPU: the package's own host search (the reference
// has no operator for them: its Python entry point goes through
// scipy.cluster.vq.vq, torch_cluster/nearest.py:93-124).
at::Tensor nearest_host(at::Tensor x, at::Tensor y, at::Tensor ptr_x,
                        at::Tensor ptr_y) {
  PCA_CHECK_CPU(x);
  PCA_CHECK_CPU(y);
  PCA_CHECK_CPU(ptr_x);
  PCA_CHECK_CPU(ptr_y);
  PCA_CHECK_INPUT(x.dim() >= 1 && y.dim() >= 1);
  x = x.view({x.size(0), -1});
  y = y.view({y.size(0), -1});
  PCA_CHECK_INPUT(x.size(1) == y.size(1));
  PCA_CHECK_INPUT(ptr_x.dim() == 1 && ptr_y.dim() == 1);
  PCA_CHECK_INPUT(ptr_x.numel() == ptr_y.numel() && ptr_x.numel() >= 2);
  // (half and bfloat16 points are searched as float, integers as double)
  const auto type = x.scalar_type() == at::kDouble || !x.is_floating_point()
                        ? at::kDouble
                        : at::kFloat;
  x = x.to(type).contiguous();
  y = y.to(type).contiguous();
  ptr_x = ptr_x.to(at::kLong).contiguous();
  ptr_y = ptr_y.to(at::kLong).contiguous();
  auto out = at::empty({x.size(0)}, ptr_x.options());
  const int rc = pca_nearest_host(
      x.data_ptr(), y.size(0) > 0 ? y.data_ptr() : nullptr,
      ptr_x.data_ptr<int64_t>(), ptr_y.data_ptr<int64_t>(), x.size(0),
      y.size(0), x.size(1), ptr_x.numel() - 1,
      type == at::kDouble ? PCA_F64 : PCA_F32, at::get_num_threads(),
      out.data_ptr<int64_t>());
  TORCH_CHECK(rc == PCA_OK, pca_host_last_error());
  return out;
}

at::Tensor nearest(at::Tensor x, at::Tensor y, at::Tensor ptr_x,
                   at::Tensor ptr_y) {
  if (!x.device().is_cuda())
    return nearest_host(x, y, ptr_x, ptr_y);
  PCA_CHECK_GPU(x);
  PCA_CHECK_GPU(y);
  PCA_CHECK_GPU(ptr_x);
  PCA_CHECK_GPU(ptr_y);
  PCA_CHECK_INPUT(x.dim() >= 1 && y.dim() >= 1);
  PCA_CHECK_INPUT(x.scalar_type() == y.scalar_type());
  PCA_CHECK_INPUT(x.get_device() == y.get_device());
  PCA_CHECK_INPUT(ptr_x.dim() == 1 && ptr_y.dim() == 1);
  PCA_CHECK_INPUT(ptr_x.numel() == ptr_y.numel() && ptr_x.numel() >= 2);
  DeviceScope scope(x.get_device());
  x = x.view({x.size(0), -1}).contiguous();
  y = y.view({y.size(0), -1}).contiguous();
  PCA_CHECK_INPUT(x.size(0) == 0 || y.size(0) == 0 ||
                  x.size(1) == y.size(1));
  auto out = at::empty({x.size(0)}, ptr_x.options().dtype(at::kLong));
  const int64_t n = x.size(0), m = y.size(0);
  if (n == 0)
    return out;
  const int64_t d = x.size(1);
  at::Tensor px = ptr_x.to(at::kLong).contiguous();
  at::Tensor py = ptr_y.to(at::kLong).contiguous();
  const int64_t segments = px.numel() - 1;
  const int dtype = dtype_code(x);
  TORCH_CHECK(dtype != PCA_BF16,
              "nearest is not implemented for 'BFloat16'");
  // (the searched rows, y, are the ones a binned search orders)
  const bool binned =
      bins_wanted(m, n, segments, kNearestCost) &&
      dtype == PCA_F32 && d <= 3 && m > 0 &&
      !being_captured(
          c10::hip::getCurrentHIPStream(x.get_device()).stream());
  const size_t ws_bytes =
      binned ? pca_nearest_binned_workspace_bytes(n, m, d, segments)
             : pca_nearest_workspace_bytes(n, m, d, segments, dtype);
  TORCH_CHECK(ws_bytes > 0, "problem size not supported");
  auto workspace =
      at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
  hipStream_t stream = c10::hip::getCurrentHIPStream(x.get_device()).stream();
  if (binned) {
    check_status(pca_nearest_binned(
        x.data_ptr(), y.data_ptr(), px.data_ptr<int64_t>(),
        py.data_ptr<int64_t>(), n, m, d, segments, out.data_ptr<int64_t>(),
        workspace.data_ptr(), ws_bytes, stream));
    return out;
  }
  check_status(pca_nearest(x.data_ptr(), m > 0 ? y.data_ptr() : nullptr,
                           px.data_ptr<int64_t>(), py.data_ptr<int64_t>(), n,
                           m, d, segments, dtype, out.data_ptr<int64_t>(),
                           workspace.data_ptr(), ws_bytes, stream));
  return out;
}

// csrc/fps.cpp:22-36 -> fps_cuda (csrc/cuda/fps_cuda.cu:68-109): samples per
// example = ceil(deg * ratio) in the ratio's element type, random start rows
// from the device generator, one host read for the output size (here the
// largest example comes with it and selects the kernel).
// csrc/fps.cpp:31-33 -> fps_cpu (csrc/cpu/fps_cpu.cpp:11-64): the same
// arithmetic for the numbers of samples (in float, as there: :25-27), a random
// first row from the host generator, the sampling itself by the package's
// host code.
at::Tensor fps_host(at::Tensor src, at::Tensor ptr, at::Tensor ratio,
                    bool random_start) {
  PCA_CHECK_CPU(src);
  PCA_CHECK_CPU(ptr);
  PCA_CHECK_CPU(ratio);
  PCA_CHECK_INPUT(ptr.dim() == 1);
  PCA_CHECK_INPUT(ptr.numel() >= 2);
  PCA_CHECK_INPUT(src.dim() >= 1);
  src = src.view({src.size(0), -1});
  const auto type =
      src.scalar_type() == at::kDouble || !src.is_floating_point()
          ? at::kDouble
          : at::kFloat;
  src = src.to(type).contiguous();
  ptr = ptr.to(at::kLong).contiguous();
  const int64_t batch_size = ptr.numel() - 1;
  auto deg = ptr.narrow(0, 1, batch_size) - ptr.narrow(0, 0, batch_size);
  auto out_ptr = deg.toType(at::kFloat) * ratio;
  out_ptr = out_ptr.ceil().toType(at::kLong).cumsum(0);
  out_ptr = at::cat({at::zeros({1}, ptr.options()), out_ptr}, 0).contiguous();
  at::Tensor start;
  if (random_start) {
    start = (at::rand({batch_size}, at::kDouble) * deg.toType(at::kDouble))
                .toType(at::kLong)
                .contiguous();
  }
  auto out = at::empty({out_ptr[-1].item<int64_t>()}, ptr.options());
  const int rc = pca_fps_host(
      src.size(0) > 0 ? src.data_ptr() : nullptr, ptr.data_ptr<int64_t>(),
      out_ptr.data_ptr<int64_t>(),
      random_start ? start.data_ptr<int64_t>() : nullptr, src.size(0),
      src.size(1), batch_size, type == at::kDouble ? PCA_F64 : PCA_F32,
      at::get_num_threads(), out.data_ptr<int64_t>());
  TORCH_CHECK(rc == PCA_OK, pca_host_last_error());
  return out;
}

at::Tensor fps(at::Tensor src, at::Tensor ptr, at::Tensor ratio,
               bool random_start) {
  if (!src.device().is_cuda())
    return fps_host(src, ptr, ratio, random_start);
  PCA_CHECK_GPU(src);
  PCA_CHECK_GPU(ptr);
  PCA_CHECK_GPU(ratio);
  PCA_CHECK_INPUT(ptr.dim() == 1);
  PCA_CHECK_INPUT(ptr.numel() >= 2);
  PCA_CHECK_INPUT(src.dim() >= 1);
  DeviceScope scope(src.get_device());
  src = src.view({src.size(0), -1}).contiguous();
  ptr = ptr.to(at::kLong).contiguous();
  const int64_t batch_size = ptr.numel() - 1;

  auto deg = ptr.narrow(0, 1, batch_size) - ptr.narrow(0, 0, batch_size);
  auto out_ptr = deg.toType(ratio.scalar_type()) * ratio;
  out_ptr = out_ptr.ceil().toType(at::kLong).cumsum(0);
  out_ptr = at::cat({at::zeros({1}, ptr.options()), out_ptr}, 0).contiguous();

  at::Tensor start;
  if (random_start) {
    start = at::rand({batch_size}, src.options());
    start = (start * deg.toType(ratio.scalar_type())).toType(at::kLong);
    start = start.contiguous();
  }

  // [number of samples, largest example] in one read
  auto sizes = at::stack({out_ptr[-1], deg.max()}).cpu();
  const int64_t out_size = sizes[0].item<int64_t>();
  const int64_t max_rows = sizes[1].item<int64_t>();
  auto out = at::empty({out_size}, ptr.options());
  const int64_t n = src.size(0);
  if (n == 0 || out_size == 0)
    return out;
  const int64_t d = src.size(1);
  const int dtype = dtype_code(src);
  TORCH_CHECK(dtype != PCA_BF16, "fps is not implemented for 'BFloat16'");
  const size_t ws_bytes =
      pca_fps_workspace_bytes(n, d, batch_size, max_rows, dtype);
  TORCH_CHECK(ws_bytes > 0, "problem size not supported");
  auto workspace =
      at::empty({(int64_t)ws_bytes}, src.options().dtype(at::kByte));
  hipStream_t stream =
      c10::hip::getCurrentHIPStream(src.get_device()).stream();
  check_status(pca_fps(src.data_ptr(), ptr.data_ptr<int64_t>(),
                       out_ptr.data_ptr<int64_t>(),
                       random_start ? start.data_ptr<int64_t>() : nullptr, n,
                       d, batch_size, max_rows, dtype, out.data_ptr<int64_t>(),
                       workspace.data_ptr(), ws_bytes, stream));
  return out;
}

// The stock loader of the reference package calls this
// (torch_cluster/__init__.py:23, csrc/version.cpp:26-41).
int64_t cuda_version() { return HIP_VERSION; }

} // namespace

TORCH_LIBRARY(torch_cluster, m) {
  m.def("knn(Tensor x, Tensor y, Tensor? ptr_x, Tensor? ptr_y, int k, "
        "bool cosine, int num_workers) -> Tensor",
        &knn);
  m.def("radius(Tensor x, Tensor y, Tensor? ptr_x, Tensor? ptr_y, float r, "
        "int max_num_neighbors, int num_workers, bool ignore_same_index) "
        "-> Tensor",
        &radius);
  m.def("nearest(Tensor x, Tensor y, Tensor ptr_x, Tensor ptr_y) -> Tensor",
        &nearest);
  m.def("fps(Tensor src, Tensor ptr, Tensor ratio, bool random_start) -> "
        "Tensor",
        &fps);
  m.def("cuda_version() -> int", &cuda_version);
}

// Operators without a counterpart in the reference: the graph entry points of
// this package call them to get their edges in one pass.
TORCH_LIBRARY(pytorch_cluster_amd, m) {
  m.def("knn_edges(Tensor x, Tensor y, Tensor? ptr_x, Tensor? ptr_y, int k, "
        "bool cosine, bool drop_self, bool x_first) -> Tensor",
        &knn_edges);
  m.def("radius_edges(Tensor x, Tensor y, Tensor? ptr_x, Tensor? ptr_y, "
        "float r, int max_num_neighbors, bool ignore_same_index, "
        "bool x_first) -> Tensor",
        &radius_edges);
  m.def("knn_batched(Tensor x, Tensor y, Tensor batch_x, Tensor batch_y, "
        "int batch_size, int k, bool cosine, bool drop_self, bool x_first) "
        "-> Tensor",
        &knn_batched);
  m.def("radius_batched(Tensor x, Tensor y, Tensor batch_x, Tensor batch_y, "
        "int batch_size, float r, int max_num_neighbors, "
        "bool ignore_same_index, bool x_first) -> Tensor",
        &radius_batched);
  m.def("host_waits() -> int", &host_waits);
  m.def("set_search_strategy(str name) -> ()", &set_search_strategy);
  m.def("get_search_strategy() -> str", &get_search_strategy);
  m.def("strategy_for(str op, int searched, int searching, int num_segments) "
        "-> str",
        &strategy_for);
}
