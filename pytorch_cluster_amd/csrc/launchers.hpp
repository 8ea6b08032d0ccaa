// Host-side launch interface between the C ABI (capi.hip) and the kernel
// translation units.  Everything here is asynchronous on `stream`.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace pca {

// Per-query result slots every search kernel writes before compaction:
//   idx   [m, slots] int32  x rows (global numbers), valid in [0, count[q])
//   dist  [m, slots] fp32   their distances (kNN only; may be NULL)
//   count [m]        int32  number of valid slots of each query
struct DenseResult {
  int *idx;
  float *dist;
  int *count;
  int slots;
  // What the compaction otherwise finds out in a pass of its own, from a
  // search that leaves it behind (compact_hints; NULL: it does not): per
  // block of queries the number of slots the compaction will write (added up
  // with atomics; zeroed by the search's set-up launch), and for graph
  // results the slot of the query's own row (-1: none) and the count without
  // it.
  unsigned long long *edge_sums = nullptr;
  int *self_pos = nullptr;
  int *kept = nullptr;
};

struct SearchInput {
  const void *x;
  const void *y;
  const int64_t *ptr_x; // NULL = one segment
  const int64_t *ptr_y;
  int n, m, d;
  int num_segments; // >= 1 (1 when ptr_* are NULL)
};

// --- segments.hip ----------------------------------------------------------

// Segments given as sorted example ids (one int64 per row) instead of
// pointers: the kernel that plans the work derives the pointers first,
// ptr[b] = first row whose id is >= b, as the reference's wrappers do with two
// bucketize calls (torch_cluster/knn.py:75-79).
struct SegmentSource {
  const int64_t *ids_x = nullptr; // [n]; NULL: the caller passed pointers
  const int64_t *ids_y = nullptr; // [m]
  int n = 0, m = 0;
  int64_t *ptr_x = nullptr;       // [num_segments + 1], written
  int64_t *ptr_y = nullptr;
  // where the largest id met + 1 goes (device-accessible memory), or NULL
  int64_t *examples_out = nullptr;
};

// work_start[b] = sum over b' < b of ceil(m_b' / per_item): the first work item
// (query tile / wave task) of each segment; work_start has num_segments + 1
// entries.  src: derive the pointers of both sides first (ptr_y must then be
// src->ptr_y).
hipError_t launch_plan(const int64_t *ptr_y, int m, int num_segments,
                       int per_item, int *work_start, hipStream_t stream,
                       const SegmentSource *src = nullptr);
// The pointers alone (for the paths that plan their work elsewhere).
hipError_t launch_segment_pointers(const SegmentSource &src, int num_segments,
                                   hipStream_t stream);

// Upper bound of work_start[num_segments] that needs no device data.
inline int plan_upper_bound(int m, int num_segments, int per_item) {
  return m / per_item + num_segments;
}

size_t compact_workspace_bytes(int m);

// count -> exclusive offsets -> edges [2, E] (+ optional distances) and E.
// drop_self: the slot holding the query's own row number is left out;
// x_first: x rows in the first half of `edges`, query rows in the second.
hipError_t launch_compact(const DenseResult &dense, int m, int64_t *edges,
                          int64_t *num_edges, float *dist_out, void *workspace,
                          hipStream_t stream, bool drop_self = false,
                          bool x_first = false);
// Points dense.edge_sums (and, with drop_self, self_pos / kept) into the
// compaction's workspace when the call is small enough for the compaction
// that adds up the block sums on its own; launch_compact then skips its
// counting pass.  Only for searches that fill them (the low-dimensional
// matrix-core kernels, the one-kernel feature-space search).
void compact_hints(DenseResult &dense, int m, void *workspace, bool drop_self);
// Queries per block sum.
constexpr int kCompactBlockQueries = 256;

// --- knn_lowd_*.hip --------------------------------------------------------

// Shape of a low-dimensional kNN launch for a problem.
struct KnnLowdConfig {
  int kbucket;          // compiled list width (>= k)
  int queries_per_lane; // 1 or 2
  int tile_queries;     // queries per work item
  bool matrix_cores;    // pre-filter on the matrix cores (knn_lowd_mc_impl)
  int num_chunks;       // slices of every segment's x rows (>= 1)
  bool nearest;         // the `nearest` search (kbucket 1, matrix cores)
};
bool knn_lowd_supported(int d, int k, bool cosine);
KnnLowdConfig knn_lowd_config(int d, int k, int n, int m, int num_segments,
                              bool cosine);
// The `nearest` search over fp32 points of up to 8 dimensions: in.x are the
// candidates, in.y the rows that look for their nearest candidate.
KnnLowdConfig nearest_lowd_config(int d, int n, int m, int num_segments);
// Scratch the launch needs beyond the dense result (shared bounds + partial
// key lists of sliced segments).
size_t knn_lowd_scratch_bytes(const KnnLowdConfig &cfg, int n, int m, int d,
                              int num_segments, int k);
// Plans the work itself (work_start: num_segments + 1 entries, written; with
// src the segment pointers in.ptr_x / in.ptr_y = src->ptr_x / ptr_y are
// derived first) -- for the matrix-core kernel in the same launch that packs
// the rows.  cfg.nearest: `out` is unused and nearest_out [m] receives the
// rows.
hipError_t launch_knn_lowd(const SearchInput &in, int k, bool cosine,
                           const KnnLowdConfig &cfg, int *work_start,
                           void *scratch, const DenseResult &out,
                           hipEvent_t time_start, hipEvent_t time_stop,
                           hipStream_t stream, int64_t *nearest_out = nullptr,
                           const SegmentSource *src = nullptr);

// --- knn_binned.hip --------------------------------------------------------

// Exact Euclidean kNN for fp32 points of up to 3 dimensions, k <= 32, over
// rows binned along a space-filling curve (same results as the scans).
bool knn_binned_supported(int d, int k, bool cosine);
size_t knn_binned_scratch_bytes(int n, int m, int num_segments);
// The events bracket everything from binning to the search kernel.
hipError_t launch_knn_binned(const SearchInput &in, int k, void *scratch,
                             const DenseResult &out, hipEvent_t time_start,
                             hipEvent_t time_stop, hipStream_t stream);

// The `nearest` search over the same bins (fp32, up to 3 dimensions): in.x
// are the candidates, in.y the rows that look for their nearest candidate;
// out [in.m] receives the rows.  The events bracket binning and search.
hipError_t launch_nearest_binned(const SearchInput &in, void *scratch,
                                 int64_t *out, hipEvent_t time_start,
                                 hipEvent_t time_stop, hipStream_t stream);

// The radius search over the same bins: fp32 points of up to 3 dimensions,
// up to 32 slots per query (out.slots; out.dist unused).
bool radius_binned_supported(int d, int slots);
hipError_t launch_radius_binned(const SearchInput &in, float r2,
                                bool ignore_same_index, void *scratch,
                                const DenseResult &out, hipStream_t stream);

// --- knn_mfma*.hip ---------------------------------------------------------

constexpr int kMfmaTileQueries = 128;
bool knn_mfma_supported(int d, int k, bool cosine);
// forced_chunks > 0: for that number of slices instead of the call's own choice
size_t knn_mfma_scratch_bytes(int n, int m, int d, int num_segments, int k,
                              int forced_chunks = 0);
// The search as a second pass behind another one, for the queries that one
// flagged: nothing runs while *gate is 0; only tiles with a flagged query
// (redo_q [m], non-zero) are searched and only flagged queries written; the
// norms come from the first pass (x_norm: squared norms, for the cosine
// distance norms; y_norm: cosine only).
struct MfmaSecondPass {
  const int *gate;
  const int *redo_q;
  const float *x_norm;
  const float *y_norm;
  int chunks; // slices of every segment's x rows
};
// work_start: tiles of kMfmaTileQueries queries.  nearest_out: the `nearest`
// search (k = 1, Euclidean; `out` unused, [m] rows written there).
hipError_t launch_knn_mfma(const SearchInput &in, int k, bool cosine,
                           const int *work_start, void *scratch,
                           const DenseResult &out, hipEvent_t time_start,
                           hipEvent_t time_stop, hipStream_t stream,
                           int64_t *nearest_out = nullptr,
                           const MfmaSecondPass *second = nullptr);

// --- knn_feat*.hip ---------------------------------------------------------

// Feature-space kNN with the fp16 matrix-core filter and the exact second
// kernel (knn_feat_impl.hpp): fp32, 8 < d <= 512, k <= 100.
bool knn_feat_supported(int d, int k, bool cosine);
size_t knn_feat_scratch_bytes(int n, int m, int d, int num_segments, int k);
// work_start: tiles of kMfmaTileQueries queries (planned by the caller).
// r16 = 1 / 2: x and y hold fp16 / bf16 rows (knn_feat16_supported shapes
// only; scratch: knn_feat16_scratch_bytes); the results are those of the
// reference's kernel for that element type.
// radius: the radius search instead (radius_feat_supported shapes;
// k = max_num_neighbors, out.dist NULL; scratch as for kNN with that k; r2
// narrowed to the element type by the caller).
struct FeatRadius {
  float r2;
  bool ignore_same;
};
hipError_t launch_knn_feat(const SearchInput &in, int k, bool cosine,
                           const int *work_start, void *scratch,
                           const DenseResult &out, hipEvent_t time_start,
                           hipEvent_t time_stop, hipStream_t stream,
                           int r16 = 0, const FeatRadius *radius = nullptr);
// Feature-space radius search through the matrix-core filter
// (knn_feat_small_impl.hpp): fp32 rows of 8 < d <= 128 components, fp16 and
// bf16 rows of up to 128, at most 32 neighbours per query, and enough pairs to
// pay for the preparation; PCA_RADIUS_FEAT=0: never, 1: whenever the shape
// fits.  r16: 0 fp32, 1 fp16, 2 bf16.
bool radius_feat_supported(int n, int m, int d, int num_segments, int slots,
                           int r16 = 0);
// Whether launch_knn_feat serves such a call (fp32 rows) with its one-kernel
// search, which counts the edges itself (compact_hints applies).
bool knn_feat_one_kernel(int n, int m, int d, int num_segments, int k,
                         bool cosine);
// fp16 / bf16 rows through the matrix-core filter (knn_feat_small_impl.hpp):
// Euclidean, d <= 128, k <= 48; PCA_KNN_FEAT_16BIT=0: never.
bool knn_feat16_supported(int n, int d, int num_segments, int k, bool cosine,
                          bool bf16);
size_t knn_feat16_scratch_bytes(int n, int m, int d, int num_segments, int k);

// --- knn_generic_*.hip -----------------------------------------------------

// |x_i| for the cosine distance of the any-dimension kernel.
hipError_t launch_row_norms(const float *x, int n, int d, float *norm,
                            hipStream_t stream);
// Slices of every segment's x rows the any-dimension kernel works in, and
// the bytes of their partial lists (0: one slice, no scratch needed).
int knn_generic_slices(int n, int m, int num_segments);
size_t knn_generic_scratch_bytes(int n, int m, int num_segments, int k);
// x_norm: [n] row norms of x (cosine only, else NULL).  One query per lane:
// work items are tiles of kBlock queries times the slices.  scratch:
// knn_generic_scratch_bytes bytes, or NULL to search every segment in one
// slice.  As a second pass behind another search: gate (device flag, nothing
// runs while it is 0) and redo_q ([m], only queries with a non-zero entry are
// searched and written).
hipError_t launch_knn_generic(const SearchInput &in, int k, bool cosine,
                              const float *x_norm, const int *work_start,
                              int grid_bound, const DenseResult &out,
                              hipStream_t stream, void *scratch,
                              const int *gate = nullptr,
                              const int *redo_q = nullptr);

// --- anytype.hip (fp64 / fp16 / bf16; dtype codes of enum pca_dtype) -------

size_t anytype_norm_bytes(int n);
// work_start: tiles of kBlock queries (kNN), wave tasks of
// kRadiusQueriesPerWave queries (radius).
// scratch: knn_anytype_scratch_bytes bytes for the slices' lists, or NULL to
// search every segment in one slice.
int knn_anytype_slices(int n, int m, int num_segments);
size_t knn_anytype_scratch_bytes(int n, int m, int num_segments, int k);
hipError_t launch_knn_anytype(int dtype, const SearchInput &in, int k,
                              bool cosine, void *x_norm,
                              const int *work_start, int grid_bound,
                              const DenseResult &out, hipStream_t stream,
                              void *scratch);
// (scalar_t)(r * r) of the reference for fp16 / bf16 points
// (csrc/cuda/radius_cuda.cu:90), as a float.
float narrow_r2_16bit(double r2, bool bf16);
hipError_t launch_radius_anytype(int dtype, const SearchInput &in, double r,
                                 bool ignore_same_index,
                                 const int *work_start, int task_bound,
                                 const DenseResult &out, hipStream_t stream);

// --- anytype.hip: the `nearest` search, any element type and dimension ------

// work_start: tiles of kBlock rows of in.y (the rows that search); in.x are
// the candidates.  dtype: PCA_F32, PCA_F64 or PCA_F16.
hipError_t launch_nearest_any(int dtype, const SearchInput &in,
                              const int *work_start, int grid_bound,
                              int64_t *out, hipStream_t stream);

// --- fps.hip ---------------------------------------------------------------

// fp32 rows of up to 4 dimensions in examples of up to 16,384 rows are sampled
// from registers; everything else streams `dist` ([n], fps_dist_bytes) and
// the rows from memory.
bool fps_in_registers(int dtype, int d, int64_t max_rows);
size_t fps_dist_bytes(int64_t n);
// One workgroup per example.  start: NULL = first row of every example.
hipError_t launch_fps(int dtype, const void *src, const int64_t *ptr,
                      const int64_t *out_ptr, const int64_t *start, int d,
                      int num_segments, int64_t max_rows, void *dist,
                      int64_t *out, hipStream_t stream);

// --- radius_mc.hip ---------------------------------------------------------

constexpr int kRadiusMcTileQueries = 128;
bool radius_mc_supported(int d, int n, int m, int num_segments);
// packed rows of x
size_t radius_mc_scratch_bytes(int n, int d);
// Plans the work itself, in the launch that packs the rows (work_start:
// num_segments + 1 entries, written: tiles of kRadiusMcTileQueries queries;
// src as for launch_knn_lowd).  time_start: recorded right before the search
// kernel.
hipError_t launch_radius_mc(const SearchInput &in, float r2,
                            bool ignore_same_index, int *work_start,
                            int tiles_bound, void *scratch,
                            const DenseResult &out, hipEvent_t time_start,
                            hipStream_t stream,
                            const SegmentSource *src = nullptr);

// --- radius.hip ------------------------------------------------------------

constexpr int kRadiusQueriesPerWave = 8;
hipError_t launch_radius(const SearchInput &in, float r2,
                         bool ignore_same_index, const int *work_start,
                         int task_bound, const DenseResult &out,
                         hipStream_t stream);

} // namespace pca
