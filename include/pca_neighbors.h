/*
 * pca_neighbors.h -- C ABI of the MI355X (gfx950) neighbour-search library.
 *
 * Plain pointers and sizes only.  In the device entry points every pointer is
 * DEVICE memory of the GPU that is current on the calling thread unless a
 * parameter says otherwise; they are asynchronous on `stream` (a hipStream_t
 * passed as void*; NULL = the default stream), return a status code, and
 * never allocate or free device memory or synchronise with the host.  The
 * *_host entry points at the end take HOST memory and return when done.
 *
 * What the library keeps between calls:
 *   - per calling thread: pca_last_error's text, the one-shot
 *     pca_time_next_search request, the last size query of the binned
 *     searches' sort;
 *   - per device, from the first call that needs them until the process ends:
 *     the address of the fixed scratch of pca_knn_fixed_scratch, and -- for
 *     the *_binned entry points with 131,072 queries or more -- one extra
 *     stream and two events: the queries are ordered on that stream beside
 *     the rows on the caller's (forked and joined with events inside the
 *     call).  Calls on one device queue that part of their work under a mutex,
 *     one after the other; PCA_BINNED_SIDE_STREAM=0 in the environment keeps
 *     everything on the caller's stream.
 * Stream capture: the *_binned entry points refuse a stream that is being
 * captured into a graph (PCA_ERR_UNSUPPORTED: their sorts clear buffers with
 * memset nodes); all other device entry points record kernels only.
 *
 * The reference (rusty1s/pytorch_cluster 1.6.3) has no C ABI: its boundary is
 * the TorchScript operator registry.  Each entry point below names the
 * reference interface it stands under, so that a binding of that interface
 * (the C++ operator shim of this repository, or a maintainer's own) is a few
 * lines of validation, allocation and one call.
 *
 * Conventions shared by all entry points
 *   x          [n, d] row-major points that are searched
 *   y          [m, d] row-major query points
 *   ptr_x/y    [num_segments + 1] int64 CSR pointers (non-decreasing,
 *              ptr[0] = 0, ptr_x[last] = n, ptr_y[last] = m); segment b of y
 *              searches segment b of x only.  Both NULL = one segment
 *              ([0, n] / [0, m]); then num_segments is ignored.
 *   edges      int64 buffer of capacity 2 * m * slots (slots = k, or the
 *              effective max_num_neighbors).  On completion it holds a
 *              contiguous [2, E] matrix at its start: edges[0 .. E) are the
 *              query (y) rows, edges[E .. 2E) the matching x rows, global row
 *              numbers, grouped by ascending query row.
 *   num_edges  one int64 that receives E: device memory, or pinned host
 *              memory (the library only ever writes it, from a kernel; a
 *              caller that waits for the stream then reads E without a copy).
 *   workspace  scratch of at least the size the matching *_workspace_bytes()
 *              call returns, 256-byte aligned.
 *   n, m < 2^31 - 1.
 */
#ifndef PCA_NEIGHBORS_H
#define PCA_NEIGHBORS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PCA_ABI_VERSION 5

enum pca_status {
  PCA_OK = 0,
  PCA_ERR_INVALID_ARGUMENT = -1, /* NULL pointer, negative size, d mismatch   */
  PCA_ERR_K_TOO_LARGE = -2,      /* k > PCA_KNN_MAX_K                         */
  PCA_ERR_WORKSPACE = -3,        /* workspace too small or misaligned         */
  PCA_ERR_LAUNCH = -4,           /* the HIP runtime refused a launch          */
  PCA_ERR_UNSUPPORTED = -5,      /* combination not built (see message)       */
  PCA_ERR_NO_DEVICE = -6         /* no usable gfx950 device is current        */
};

/* Same limit as the reference GPU operator (csrc/cuda/knn_cuda.cu:98). */
#define PCA_KNN_MAX_K 100

/* Element types of x / y. */
enum pca_dtype {
  PCA_F32 = 0,
  PCA_F64 = 1,
  PCA_F16 = 2,
  PCA_BF16 = 3
};

/*
 * Edge options of pca_knn / pca_radius (`edge_flags`, 0 = the operators'
 * output as described above).  They fold the epilogue of the reference's
 * graph entry points (torch_cluster/knn.py:135-144,
 * torch_cluster/radius.py:143-148) into the pass that writes `edges`:
 *   PCA_EDGES_DROP_SELF  leave out the pairs whose x row number equals the
 *                        query's (the `row != col` mask of knn_graph when x
 *                        and y are the same rows; for pca_radius the same as
 *                        ignore_same_index)
 *   PCA_EDGES_X_FIRST    edges[0 .. E) are the x rows, edges[E .. 2E) the
 *                        query rows (flow "source_to_target")
 * and the prologue of all four entry points (torch_cluster/knn.py:62-79,
 * torch_cluster/radius.py:66-84) into the launch that prepares the search:
 *   PCA_SEGMENTS_BY_ID   ptr_x / ptr_y are not pointers but the SORTED example
 *                        ids of the rows ([n] and [m] int64, values in
 *                        [0, num_segments)); the pointers -- ptr[b] = number
 *                        of rows with an id below b, what the reference's
 *                        wrappers get from two bucketize calls -- are derived
 *                        on the device.  pca_knn, pca_knn_fixed_scratch and
 *                        pca_radius take it; for the other entry points call
 *                        pca_segment_pointers first.
 */
#define PCA_EDGES_DROP_SELF 1
#define PCA_EDGES_X_FIRST 2
#define PCA_SEGMENTS_BY_ID 4

/* ABI version of the loaded library (== PCA_ABI_VERSION it was built with). */
int pca_abi_version(void);

/* Static, human-readable text for a status code. */
const char *pca_status_string(int status);

/* Text describing the last failure on the calling thread ("" if none). */
const char *pca_last_error(void);

/*
 * Measurement hook: the next pca_knn / pca_radius / pca_nearest call of the
 * calling thread
 * records `start_event` immediately before and `stop_event` immediately after
 * its search kernel (the dominant kernel; planning and compaction kernels stay
 * outside) on that call's stream.  Both are hipEvent_t created by the caller
 * with timing enabled.  The request is consumed by that one call; pass NULLs
 * to cancel it.  No counterpart in the reference.
 */
int pca_time_next_search(void *start_event, void *stop_event);

/*
 * ptr_x[b] / ptr_y[b] = number of rows of x / y whose example id is below b,
 * b = 0 .. num_segments: the segment pointers of sorted example-id vectors
 * (torch_cluster/knn.py:75-79: two torch.bucketize calls).  One small launch;
 * ptr_x and ptr_y: num_segments + 1 entries each, device memory.
 */
int pca_segment_pointers(const int64_t *ids_x, int64_t n, const int64_t *ids_y,
                         int64_t m, int64_t num_segments, int64_t *ptr_x,
                         int64_t *ptr_y, void *stream);

/*
 * For a caller that does not know the number of examples (the reference's
 * wrappers read it from the device, torch_cluster/knn.py:62-72: two
 * batch.max() reductions with a host wait each): the next call of the calling
 * thread that derives pointers from example ids -- pca_knn / pca_radius /
 * pca_knn_fixed_scratch with PCA_SEGMENTS_BY_ID, or pca_segment_pointers --
 * stores the largest id it was given + 1 to *examples_in_use (memory the
 * device can write: device memory or pinned host memory) from the launch
 * that derives the pointers.  Such a caller passes its best guess as
 * num_segments, reads the number together with the edge count after the one
 * wait it needs anyway, and calls again only if the guess was too small.  (A
 * guess that is too large gives the same edges: examples without rows.  One
 * that is too small is harmless -- queries of the examples beyond it are
 * searched in the last example, their rows of x not at all, as the
 * reference's lookup does, csrc/cuda/utils.cuh:11-19 -- but not what the
 * caller wants.)  NULL cancels the request.
 */
int pca_report_examples(int64_t *examples_in_use);

/* ------------------------------------------------------------------ kNN -- */

/*
 * Workspace size of pca_knn for these sizes (bytes; 0 on invalid arguments).
 */
size_t pca_knn_workspace_bytes(int64_t n, int64_t m, int64_t d,
                               int64_t num_segments, int64_t k, int dtype);

/*
 * For every row of y the k nearest rows of x of the same segment.
 *
 * Stands under the reference operator
 *   torch_cluster::knn(x, y, ptr_x, ptr_y, k, cosine, num_workers)
 *   csrc/knn.cpp:22-40 -> knn_cuda, csrc/cuda/knn_cuda.cu:86-135
 * and reproduces knn_kernel (csrc/cuda/knn_cuda.cu:30-84): squared Euclidean
 * distance accumulated over the dimensions in ascending order (or
 * 1 - x.y / (|x| |y|) when cosine != 0), neighbours of a query ordered by
 * ascending distance with ties by ascending x row, min(k, segment size)
 * neighbours per query, candidates whose distance is >= 1e10 or NaN are never
 * returned.  `dtype` selects the element type of x and y (enum pca_dtype).
 *
 * edges: capacity 2 * m * k.  Optional outputs (NULL to skip):
 *   dist   [capacity m * k] element type of x: the distance of each returned
 *          edge, in edge order (the reference discards these).
 */
int pca_knn(const void *x, const void *y, const int64_t *ptr_x,
            const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
            int64_t num_segments, int64_t k, int cosine, int dtype,
            int edge_flags, int64_t *edges, int64_t *num_edges, void *dist,
            void *workspace, size_t workspace_bytes, void *stream);

/*
 * pca_knn without a workspace argument, for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid it).  No counterpart in the reference, whose operator allocates
 * its temporaries through PyTorch.  Same arguments, results and errors as
 * pca_knn; the scratch the kernels need lives in a buffer of
 * PCA_FIXED_SCRATCH_BYTES that is part of the library's device code (one copy
 * per GPU, held until the process ends), so the call itself allocates and
 * frees nothing.  A search whose pca_knn_workspace_bytes() exceeds
 * PCA_FIXED_SCRATCH_BYTES is refused with PCA_ERR_WORKSPACE before anything is
 * launched.  All calls on one GPU share that buffer: calls that may overlap
 * on the GPU (different streams, different host threads) race and must be
 * ordered by the caller.  The buffer's address is looked up at the first call
 * on a device; make that call outside of any stream capture.
 */
#define PCA_FIXED_SCRATCH_BYTES (32u << 20)

int pca_knn_fixed_scratch(const void *x, const void *y, const int64_t *ptr_x,
                          const int64_t *ptr_y, int64_t n, int64_t m,
                          int64_t d, int64_t num_segments, int64_t k,
                          int cosine, int dtype, int edge_flags,
                          int64_t *edges, int64_t *num_edges, void *dist,
                          void *stream);

/*
 * pca_knn for fp32 points of up to 3 dimensions, Euclidean distance and
 * k <= 64 (PCA_ERR_UNSUPPORTED otherwise) over spatially binned rows: the x
 * rows of every segment are ordered along a space-filling curve (the voxel
 * numbers of the reference's grid clustering, csrc/cuda/grid_cuda.cu:10-25,
 * bit-interleaved), cut into tiles with bounding boxes, and a query scans only
 * the tiles whose box is within its current k-th distance.  Stands under the
 * same operator as pca_knn (csrc/knn.cpp:22-40 -> csrc/cuda/knn_cuda.cu:86-135)
 * and returns the same edges, bit for bit, in the same order; only the work
 * differs (rows looked at per query: tens to hundreds instead of the whole
 * segment).  Arguments as for pca_knn.
 */
size_t pca_knn_binned_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                      int64_t num_segments, int64_t k);

int pca_knn_binned(const void *x, const void *y, const int64_t *ptr_x,
                   const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                   int64_t num_segments, int64_t k, int edge_flags,
                   int64_t *edges, int64_t *num_edges, void *dist,
                   void *workspace, size_t workspace_bytes, void *stream);

/* --------------------------------------------------------------- radius -- */

/*
 * Number of neighbour slots per query pca_radius uses for these sizes:
 * min(max_num_neighbors, n).  `edges` must hold 2 * m * slots int64.
 */
int64_t pca_radius_slots(int64_t n, int64_t max_num_neighbors);

size_t pca_radius_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                  int64_t num_segments,
                                  int64_t max_num_neighbors, int dtype);

/*
 * For every row of y the rows of x of the same segment with squared distance
 * strictly below r * r, at most max_num_neighbors of them: the first ones in
 * ascending x row order.
 *
 * Stands under the reference operator
 *   torch_cluster::radius(x, y, ptr_x, ptr_y, r, max_num_neighbors,
 *                         num_workers, ignore_same_index)
 *   csrc/radius.cpp:22-39 -> radius_cuda, csrc/cuda/radius_cuda.cu:44-96
 * and reproduces radius_kernel (csrc/cuda/radius_cuda.cu:9-42); r * r is
 * formed in double and narrowed to the element type as at
 * csrc/cuda/radius_cuda.cu:90.  With ignore_same_index != 0 the x row whose
 * global number equals the query's is skipped.  max_num_neighbors must be
 * >= 1 (the reference is undefined for 0).
 */
int pca_radius(const void *x, const void *y, const int64_t *ptr_x,
               const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
               int64_t num_segments, double r, int64_t max_num_neighbors,
               int ignore_same_index, int dtype, int edge_flags,
               int64_t *edges, int64_t *num_edges, void *workspace,
               size_t workspace_bytes, void *stream);

/*
 * pca_radius for fp32 points of up to 3 dimensions and at most 64 neighbours
 * per query (pca_radius_slots; PCA_ERR_UNSUPPORTED otherwise) over the
 * spatially binned rows of pca_knn_binned: a query scans only the tiles whose
 * box is closer than r, and of the rows found keeps the max_num_neighbors
 * with the smallest row numbers.  Stands under the same operator as
 * pca_radius (csrc/radius.cpp:22-39 -> csrc/cuda/radius_cuda.cu:44-96) and
 * returns the same edges in the same order.  Arguments as for pca_radius.
 */
size_t pca_radius_binned_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                         int64_t num_segments,
                                         int64_t max_num_neighbors);

int pca_radius_binned(const void *x, const void *y, const int64_t *ptr_x,
                      const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                      int64_t num_segments, double r,
                      int64_t max_num_neighbors, int ignore_same_index,
                      int edge_flags, int64_t *edges, int64_t *num_edges,
                      void *workspace, size_t workspace_bytes, void *stream);

/* -------------------------------------------------------------- nearest -- */

/*
 * NOTE the roles: as in the reference operator, here the rows of x SEARCH and
 * the rows of y ARE SEARCHED (the opposite of pca_knn / pca_radius).
 *   x      [n, d] rows that look for their nearest row of y
 *   y      [m, d] candidates
 *   ptr_x  [num_segments + 1] segments of x, ptr_y those of y (as above;
 *          every row of x must lie in a segment: ptr_x[last] = n)
 *   out    [n] int64: for every row of x the global number of the row of y
 *          of the same segment with the smallest squared distance.
 *
 * Stands under the reference operator
 *   torch_cluster::nearest(x, y, ptr_x, ptr_y)
 *   csrc/nearest.cpp:22-39 -> nearest_cuda, csrc/cuda/nearest_cuda.cu:68-94
 * and reproduces nearest_kernel (csrc/cuda/nearest_cuda.cu:10-66) including
 * its two corner rules: a candidate counts only if its distance is strictly
 * below 1e38 (narrowed to the element type: +inf for fp16), and a row with no
 * such candidate (empty segment of y, NaN, overflow) gets 0; among candidates
 * of equal distance the one with the smallest (row - segment start) % 1024
 * wins, then the smallest row (what that kernel's block of 1,024 threads and
 * its pairwise reduction return).
 * dtype: PCA_F32, PCA_F64 or PCA_F16 (the types the reference instantiates,
 * csrc/cuda/nearest_cuda.cu:85); PCA_BF16 returns PCA_ERR_UNSUPPORTED.
 */
size_t pca_nearest_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                   int64_t num_segments, int dtype);

int pca_nearest(const void *x, const void *y, const int64_t *ptr_x,
                const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                int64_t num_segments, int dtype, int64_t *out,
                void *workspace, size_t workspace_bytes, void *stream);

/*
 * pca_nearest for fp32 points of up to 3 dimensions (PCA_ERR_UNSUPPORTED
 * otherwise) over spatially binned rows of y, as pca_knn_binned bins the rows
 * of x: every row of x looks only at rows of y near it.  Stands under the same
 * operator as pca_nearest (csrc/nearest.cpp:22-36 ->
 * csrc/cuda/nearest_cuda.cu:68-94) and returns the same rows, the reference's
 * order among equal distances included.  Arguments as for pca_nearest, without
 * dtype.
 */
size_t pca_nearest_binned_workspace_bytes(int64_t n, int64_t m, int64_t d,
                                          int64_t num_segments);

int pca_nearest_binned(const void *x, const void *y, const int64_t *ptr_x,
                       const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                       int64_t num_segments, int64_t *out, void *workspace,
                       size_t workspace_bytes, void *stream);

/* ----------------------------------------------------- host (CPU) path -- */

/*
 * The two searches on the host, for points that are not on a GPU.  Every
 * pointer is HOST memory here; the calls run on `num_threads` threads of their
 * own (at least one), allocate their temporaries with the C++ allocator and
 * return when the result is complete.  Same arguments and the same result as
 * pca_knn / pca_radius (bit for bit, order included), no cosine distance; k
 * may exceed PCA_KNN_MAX_K.  edges: capacity 2 * m * min(k, n) resp.
 * 2 * m * pca_radius_slots(n, max_num_neighbors); *num_edges (host) receives E.
 * dist (optional, fp32 / fp64 points only): capacity m * min(k, n).
 *
 * Stand under the CPU branch of the reference operators
 *   csrc/knn.cpp:32-35 -> knn_cpu, csrc/cpu/knn_cpu.cpp:7-105
 *   csrc/radius.cpp:31-34 -> radius_cpu, csrc/cpu/radius_cpu.cpp:7-117
 * (nanoflann k-d trees), with the result contract of the GPU kernels instead
 * of nanoflann's: neighbours by ascending (distance, row), for the radius
 * search the first max_num_neighbors rows in row order where the reference's
 * CPU code keeps those its tree meets first.
 * Errors: status codes as above, text from pca_host_last_error().
 */
const char *pca_host_last_error(void);

int pca_knn_host(const void *x, const void *y, const int64_t *ptr_x,
                 const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                 int64_t num_segments, int64_t k, int dtype, int edge_flags,
                 int num_threads, int64_t *edges, int64_t *num_edges,
                 void *dist);

int pca_radius_host(const void *x, const void *y, const int64_t *ptr_x,
                    const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                    int64_t num_segments, double r, int64_t max_num_neighbors,
                    int ignore_same_index, int dtype, int edge_flags,
                    int num_threads, int64_t *edges, int64_t *num_edges);

/*
 * `fps` and `nearest` on the host (fp32 / fp64 points; all pointers HOST
 * memory, `num_threads` threads over the examples resp. over blocks of rows).
 * Arguments as for pca_fps / pca_nearest, and the same rows as those return:
 * the tie rules and limits of the reference's CUDA kernels
 * (csrc/cuda/fps_cuda.cu:10-66, csrc/cuda/nearest_cuda.cu:10-66), distances
 * by one fused multiply-add per component.  They stand under
 *   csrc/fps.cpp:31-33 -> fps_cpu, csrc/cpu/fps_cpu.cpp:11-64 (no 5e4 cap, the
 *   first row among equal values: the same samples wherever distances stay
 *   below 5e4 and do not tie)
 *   torch_cluster/nearest.py:93-124 (scipy.cluster.vq.vq per example: the
 *   lowest row among equal distances)
 * Errors: status codes as above, text from pca_host_last_error().
 */
int pca_fps_host(const void *src, const int64_t *ptr, const int64_t *out_ptr,
                 const int64_t *start, int64_t n, int64_t d,
                 int64_t num_segments, int dtype, int num_threads,
                 int64_t *out);

int pca_nearest_host(const void *x, const void *y, const int64_t *ptr_x,
                     const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                     int64_t num_segments, int dtype, int num_threads,
                     int64_t *out);

/* ------------------------------------------------------------------ fps -- */

/*
 * Farthest point sampling per segment.
 *   src      [n, d] row-major points
 *   ptr      [num_segments + 1] segments of src (required)
 *   out_ptr  [num_segments + 1] first output position of every segment
 *            (out_ptr[0] = 0); segment b receives out_ptr[b+1] - out_ptr[b]
 *            samples.  The reference computes it as the running sum of
 *            ceil(segment size * ratio) (csrc/cuda/fps_cuda.cu:80-83).
 *   start    [num_segments] offset of every segment's first sample within
 *            the segment, or NULL = its first row (random_start = false)
 *   out      [out_ptr[num_segments]] int64 row numbers of src, per segment in
 *            sampling order
 *   max_segment_rows  an upper bound of the segment sizes known to the caller
 *            (it selects the kernel: fp32 points of up to 4 dimensions in
 *            segments of up to 16,384 rows are sampled from registers), or 0
 *            = unknown.
 *
 * Stands under the reference operator
 *   torch_cluster::fps(src, ptr, ratio, random_start)
 *   csrc/fps.cpp:22-38 -> fps_cuda, csrc/cuda/fps_cuda.cu:68-109
 * and reproduces fps_kernel (csrc/cuda/fps_cuda.cu:10-66): running minimum
 * squared distances that start at 5e4 (larger distances count as 5e4), the
 * next sample = the row with the largest running minimum, among equal ones
 * the smallest (row - segment start) % 256, then the smallest row (what that
 * kernel's block of 256 threads returns); row 0 when every value is NaN.
 * dtype: PCA_F32, PCA_F64 or PCA_F16 (csrc/cuda/fps_cuda.cu:100).
 */
size_t pca_fps_workspace_bytes(int64_t n, int64_t d, int64_t num_segments,
                               int64_t max_segment_rows, int dtype);

int pca_fps(const void *src, const int64_t *ptr, const int64_t *out_ptr,
            const int64_t *start, int64_t n, int64_t d, int64_t num_segments,
            int64_t max_segment_rows, int dtype, int64_t *out, void *workspace,
            size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* PCA_NEIGHBORS_H */
