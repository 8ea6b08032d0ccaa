// Segment planning and output compaction kernels.
//
// Replaces, on the device and without host synchronisation:
//   * get_example_idx (csrc/cuda/utils.cuh:11-19 in the reference): instead of
//     every thread scanning ptr linearly, one tiny kernel turns ptr_y into a
//     table "first work item of each segment" that workgroups binary-search;
//   * the reference's post-kernel epilogue `mask = col != -1`,
//     2x masked_select, stack (csrc/cuda/knn_cuda.cu:133-134,
//     csrc/cuda/radius_cuda.cu:94-95): per-query counts -> exclusive scan ->
//     scatter into a contiguous [2, E] matrix, E left in device memory;
//   * on request the epilogue of the graph entry points as well
//     (torch_cluster/knn.py:135-144, torch_cluster/radius.py:143-148): pairs
//     of a row with itself are left out and the x row is written first, in
//     the same pass.
#include "device_utils.hpp"
#include "launchers.hpp"

namespace pca {

namespace {

// Single workgroup: exclusive scan of ceil(m_b / per_item) over segments;
// before that, when the caller passed sorted example ids instead of pointers,
// the pointers of both sides (ptr_y is then src.ptr_y).
__global__ __launch_bounds__(kPlanThreads) void plan_kernel(
    const int64_t *__restrict__ ptr_y, int m, int num_segments, int per_item,
    int *__restrict__ work_start, SegmentSource src) {
  __shared__ int partial[kPlanThreads];
  if (src.ids_x != nullptr) {
    pointers_from_ids(src, num_segments);
    __syncthreads();
  }
  plan_segments(ptr_y, m, num_segments, per_item, work_start, partial);
}

__global__ __launch_bounds__(kPlanThreads) void segment_pointers_kernel(
    SegmentSource src, int num_segments) {
  pointers_from_ids(src, num_segments);
}

// ---- compaction -----------------------------------------------------------

constexpr int kCompactQueries = kBlock; // queries per workgroup

// Block-wide exclusive scan of one int per thread; returns the exclusive
// prefix, *total receives the block sum.
__device__ __forceinline__ int block_exclusive_scan(int v, int *lds,
                                                    int *total) {
  const int tid = threadIdx.x;
  lds[tid] = v;
  __syncthreads();
  for (int off = 1; off < kBlock; off <<= 1) {
    int t = tid >= off ? lds[tid - off] : 0;
    __syncthreads();
    lds[tid] += t;
    __syncthreads();
  }
  *total = lds[kBlock - 1];
  return lds[tid] - v;
}

__global__ __launch_bounds__(kBlock) void block_sum_kernel(
    const int *__restrict__ count, int m, int64_t *__restrict__ block_sums) {
  __shared__ int lds[kBlock];
  const int q = blockIdx.x * kCompactQueries + threadIdx.x;
  int total;
  block_exclusive_scan(q < m ? count[q] : 0, lds, &total);
  if (threadIdx.x == 0)
    block_sums[blockIdx.x] = total;
}

// Single workgroup: in-place exclusive scan of the block sums, total -> E.
__global__ __launch_bounds__(kPlanThreads) void scan_block_sums_kernel(
    int64_t *__restrict__ block_sums, int num_blocks,
    int64_t *__restrict__ num_edges) {
  __shared__ int64_t partial[kPlanThreads];
  const int tid = threadIdx.x;
  const int per_thread = (num_blocks + kPlanThreads - 1) / kPlanThreads;
  const int i0 = min(tid * per_thread, num_blocks);
  const int i1 = min(i0 + per_thread, num_blocks);
  int64_t sum = 0;
  for (int i = i0; i < i1; ++i)
    sum += block_sums[i];
  partial[tid] = sum;
  __syncthreads();
  for (int off = 1; off < kPlanThreads; off <<= 1) {
    int64_t v = tid >= off ? partial[tid - off] : 0;
    __syncthreads();
    partial[tid] += v;
    __syncthreads();
  }
  int64_t run = partial[tid] - sum;
  for (int i = i0; i < i1; ++i) {
    int64_t v = block_sums[i];
    block_sums[i] = run;
    run += v;
  }
  // (the total also behind the offsets: the scatter reads it from there, so
  // that num_edges is only ever written -- it may be host memory)
  if (tid == kPlanThreads - 1) {
    *num_edges = partial[tid];
    block_sums[num_blocks] = partial[tid];
  }
}

// e / slots without a division, for the entries e < kCompactQueries * slots
// of a block: with magic = ceil(2^32 / slots) the product's high word is the
// quotient as long as e (slots - 1) < 2^32, which holds up to 4,000 slots; 0
// (one slot, or more than that) stands for "divide".
inline uint32_t slots_magic(int slots) {
  if (slots < 2 || slots > 4000)
    return 0;
  return (uint32_t)((((uint64_t)1 << 32) + (uint64_t)slots - 1) /
                    (uint64_t)slots);
}
__device__ __forceinline__ int quotient_by_slots(int e, int slots,
                                                 uint32_t magic) {
  return magic != 0 ? (int)__umulhi((uint32_t)e, magic) : e / slots;
}

// Both kernels below walk the slot rows of a block of queries as ONE flat
// range (element e = slot e % slots of query e / slots): reads are contiguous
// and independent of each other, so many are in flight per thread.
//
// find_self_kernel: position of the slot that holds the query's own row
// number (at most one: the rows of a query are distinct), or -1, and the
// number of slots without it.
__global__ __launch_bounds__(kBlock) void find_self_kernel(
    const int *__restrict__ idx, const int *__restrict__ count, int m,
    int slots, uint32_t magic, int *__restrict__ self_pos,
    int *__restrict__ kept) {
  __shared__ int s_self[kCompactQueries];
  __shared__ int s_count[kCompactQueries];
  const int tid = threadIdx.x;
  const int q0 = blockIdx.x * kCompactQueries;
  const int nq = min(kCompactQueries, m - q0);
  s_self[tid] = -1;
  s_count[tid] = tid < nq ? count[q0 + tid] : 0;
  __syncthreads();
  const int *rows = idx + (size_t)q0 * slots;
  const int total = nq * slots;
#pragma unroll 4
  for (int e = tid; e < total; e += kBlock) {
    const int ql = quotient_by_slots(e, slots, magic);
    const int sl = e - ql * slots;
    const int v = rows[e];
    if (sl < s_count[ql] && v == q0 + ql)
      s_self[ql] = sl;
  }
  __syncthreads();
  if (tid < nq) {
    self_pos[q0 + tid] = s_self[tid];
    kept[q0 + tid] = s_count[tid] - (s_self[tid] >= 0 ? 1 : 0);
  }
}

// The two kernels of the short path (up to kInlineScanBlocks blocks of
// queries): count_block_kernel = find_self_kernel + block_sum_kernel in one
// pass (self_pos == nullptr: nothing is left out, only the sums), and a
// scatter that adds up the sums of the blocks before it on its own.
constexpr int kInlineScanBlocks = 2048;

__global__ __launch_bounds__(kBlock) void count_block_kernel(
    const int *__restrict__ idx, const int *__restrict__ count, int m,
    int slots, uint32_t magic, int *__restrict__ self_pos,
    int *__restrict__ kept, int64_t *__restrict__ block_sums) {
  __shared__ int s_self[kCompactQueries];
  __shared__ int s_count[kCompactQueries];
  __shared__ int lds[kBlock];
  const int tid = threadIdx.x;
  const int q0 = blockIdx.x * kCompactQueries;
  const int nq = min(kCompactQueries, m - q0);
  int c = tid < nq ? count[q0 + tid] : 0;
  if (self_pos != nullptr) {
    s_self[tid] = -1;
    s_count[tid] = c;
    __syncthreads();
    const int *rows = idx + (size_t)q0 * slots;
    const int total = nq * slots;
#pragma unroll 4
    for (int e = tid; e < total; e += kBlock) {
      const int ql = quotient_by_slots(e, slots, magic);
      const int sl = e - ql * slots;
      const int v = rows[e];
      if (sl < s_count[ql] && v == q0 + ql)
        s_self[ql] = sl;
    }
    __syncthreads();
    if (tid < nq) {
      c -= s_self[tid] >= 0 ? 1 : 0;
      self_pos[q0 + tid] = s_self[tid];
      kept[q0 + tid] = c;
    }
  }
  int total;
  block_exclusive_scan(c, lds, &total);
  if (tid == 0)
    block_sums[blockIdx.x] = total;
}

// count: slots to write per query (without the self slot when self_pos is
// given).  x_first: the x row goes to the first half of `edges`.
// inline_scan: block_offsets holds the blocks' SUMS; this block adds up the
// ones before it and all of them (block 0 also stores the total).
__global__ __launch_bounds__(kBlock) void scatter_kernel(
    const int *__restrict__ idx, const float *__restrict__ dist,
    const int *__restrict__ count, const int *__restrict__ self_pos, int m,
    int slots, uint32_t magic, int x_first,
    const int64_t *__restrict__ block_offsets,
    int64_t *__restrict__ num_edges, int64_t *__restrict__ edges,
    float *__restrict__ dist_out, int inline_scan) {
  __shared__ int lds[kBlock];
  __shared__ int64_t s_before[kBlock], s_all[kBlock];
  __shared__ int s_count[kCompactQueries];
  __shared__ int s_offset[kCompactQueries];
  __shared__ int s_self[kCompactQueries];
  const int tid = threadIdx.x;
  const int q0 = blockIdx.x * kCompactQueries;
  const int q = q0 + tid;
  const int c = q < m ? count[q] : 0;
  int total;
  const int off = block_exclusive_scan(c, lds, &total);
  s_count[tid] = c;
  s_offset[tid] = off;
  // (a position no slot has when nothing is left out)
  s_self[tid] = (self_pos && q < m && self_pos[q] >= 0) ? self_pos[q] : slots;
  __syncthreads();
  int64_t E, base;
  if (inline_scan) {
    int64_t before = 0, all = 0;
    for (int b = tid; b < (int)gridDim.x; b += kBlock) {
      const int64_t v = block_offsets[b];
      all += v;
      before += b < (int)blockIdx.x ? v : 0;
    }
    s_before[tid] = before;
    s_all[tid] = all;
    __syncthreads();
    for (int off = kBlock / 2; off >= 1; off >>= 1) {
      if (tid < off) {
        s_before[tid] += s_before[tid + off];
        s_all[tid] += s_all[tid + off];
      }
      __syncthreads();
    }
    E = s_all[0];
    base = s_before[0];
    if (blockIdx.x == 0 && tid == 0)
      *num_edges = E;
  } else {
    E = block_offsets[gridDim.x];
    base = block_offsets[blockIdx.x];
  }
  if (total == 0)
    return;

  const int nq = min(kCompactQueries, m - q0);
  int64_t *first = x_first ? edges + E : edges;  // receives the query rows
  int64_t *second = x_first ? edges : edges + E; // receives the x rows
  const int *rows = idx + (size_t)q0 * slots;
  const float *row_dist = dist ? dist + (size_t)q0 * slots : nullptr;
  const int span = nq * slots;
#pragma unroll 4
  for (int e = tid; e < span; e += kBlock) {
    const int ql = quotient_by_slots(e, slots, magic);
    const int sl = e - ql * slots;
    const int skip = s_self[ql];
    // slot sl goes to position sl, or sl - 1 behind the left-out slot
    const int pos = sl - (sl > skip ? 1 : 0);
    if (sl != skip && pos < s_count[ql]) {
      const int64_t o = base + s_offset[ql] + pos;
      first[o] = q0 + ql;
      second[o] = rows[e];
      if (dist_out)
        dist_out[o] = row_dist[e];
    }
  }
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

} // namespace

hipError_t launch_plan(const int64_t *ptr_y, int m, int num_segments,
                       int per_item, int *work_start, hipStream_t stream,
                       const SegmentSource *src) {
  hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(kPlanThreads), 0, stream, ptr_y,
                     m, num_segments, per_item, work_start,
                     src ? *src : SegmentSource{});
  return hipGetLastError();
}

hipError_t launch_segment_pointers(const SegmentSource &src, int num_segments,
                                   hipStream_t stream) {
  hipLaunchKernelGGL(segment_pointers_kernel, dim3(1), dim3(kPlanThreads), 0,
                     stream, src, num_segments);
  return hipGetLastError();
}

size_t compact_workspace_bytes(int m) {
  const int blocks = (m + kCompactQueries - 1) / kCompactQueries;
  // block sums, then the two per-query arrays of find_self_kernel
  return align256(sizeof(int64_t) * (size_t)(blocks + 1)) +
         2 * align256(sizeof(int) * (size_t)m);
}

void compact_hints(DenseResult &dense, int m, void *workspace, bool drop_self) {
  static_assert(kCompactBlockQueries == kCompactQueries, "one block, one sum");
  const int blocks = (m + kCompactQueries - 1) / kCompactQueries;
  if (blocks > kInlineScanBlocks)
    return;
  char *ws = static_cast<char *>(workspace);
  dense.edge_sums = reinterpret_cast<unsigned long long *>(ws);
  ws += align256(sizeof(int64_t) * (size_t)(blocks + 1));
  if (drop_self) {
    dense.self_pos = reinterpret_cast<int *>(ws);
    dense.kept = reinterpret_cast<int *>(ws + align256(sizeof(int) * (size_t)m));
  }
}

hipError_t launch_compact(const DenseResult &dense, int m, int64_t *edges,
                          int64_t *num_edges, float *dist_out, void *workspace,
                          hipStream_t stream, bool drop_self, bool x_first) {
  const int blocks = (m + kCompactQueries - 1) / kCompactQueries;
  char *ws = static_cast<char *>(workspace);
  int64_t *block_sums = reinterpret_cast<int64_t *>(ws);
  ws += align256(sizeof(int64_t) * (size_t)(blocks + 1));
  int *self_pos = reinterpret_cast<int *>(ws);
  int *kept = reinterpret_cast<int *>(ws + align256(sizeof(int) * (size_t)m));
  const int *count = dense.count;
  const uint32_t magic = slots_magic(dense.slots);
  if (dense.edge_sums != nullptr && blocks <= kInlineScanBlocks &&
      (!drop_self || dense.self_pos != nullptr)) {
    // the search left the block sums (and the self slots) behind
    hipLaunchKernelGGL(scatter_kernel, dim3(blocks), dim3(kBlock), 0, stream,
                       dense.idx, dense.dist, drop_self ? dense.kept : count,
                       drop_self ? dense.self_pos : (const int *)nullptr, m,
                       dense.slots, magic, x_first ? 1 : 0,
                       reinterpret_cast<const int64_t *>(dense.edge_sums),
                       num_edges, edges, dist_out, 1);
    return hipGetLastError();
  }
  if (blocks <= kInlineScanBlocks) {
    hipLaunchKernelGGL(count_block_kernel, dim3(blocks), dim3(kBlock), 0,
                       stream, dense.idx, dense.count, m, dense.slots, magic,
                       drop_self ? self_pos : (int *)nullptr, kept,
                       block_sums);
    hipLaunchKernelGGL(scatter_kernel, dim3(blocks), dim3(kBlock), 0, stream,
                       dense.idx, dense.dist, drop_self ? kept : count,
                       drop_self ? self_pos : (const int *)nullptr, m,
                       dense.slots, magic, x_first ? 1 : 0, block_sums,
                       num_edges, edges, dist_out, 1);
    return hipGetLastError();
  }
  if (drop_self) {
    hipLaunchKernelGGL(find_self_kernel, dim3(blocks), dim3(kBlock), 0, stream,
                       dense.idx, dense.count, m, dense.slots, magic, self_pos,
                       kept);
    count = kept;
  }
  hipLaunchKernelGGL(block_sum_kernel, dim3(blocks), dim3(kBlock), 0, stream,
                     count, m, block_sums);
  hipLaunchKernelGGL(scan_block_sums_kernel, dim3(1), dim3(kPlanThreads), 0,
                     stream, block_sums, blocks, num_edges);
  hipLaunchKernelGGL(scatter_kernel, dim3(blocks), dim3(kBlock), 0, stream,
                     dense.idx, dense.dist, count,
                     drop_self ? self_pos : (const int *)nullptr, m,
                     dense.slots, magic, x_first ? 1 : 0, block_sums, num_edges,
                     edges, dist_out, 0);
  return hipGetLastError();
}

} // namespace pca
