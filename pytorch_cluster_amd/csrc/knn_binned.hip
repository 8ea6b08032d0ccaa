// Exact Euclidean kNN over spatially binned rows: fp32 points of up to three
// dimensions, k <= 64 (more than 32 with the matrix-core scan of
// knn_binned_mc_impl.hpp only), and the radius and nearest searches over the
// same bins (further down).  This comment describes the vector-ALU kNN scan,
// the first of them, and the binning all share.  Same results, bit for bit, as the reference's scan of
// every row of the segment (csrc/cuda/knn_cuda.cu:52-78: distances as chains
// of direct differences and fused multiply-adds, neighbours by ascending
// distance, ties by ascending row, strictly below 1e10), but a query looks only
// at rows near it.
//
// Per call: every segment's x rows are ordered along a space-filling curve
// (30-bit Morton codes inside the segment's bounding box - the voxel number of
// the reference's grid clustering, csrc/cuda/grid_cuda.cu:10-25, with its bits
// interleaved - sorted by rocPRIM's radix sort), copied in that order together
// with their row numbers, and cut into tiles of 32 rows with a bounding box
// each.  The queries are ordered the same way, so the 64 queries of a wave
// (one per lane) are neighbours in space and share one bounding box.
//
// A wave first scans the tiles around its queries' position in the order of x
// (that fills the lists and gives every query a k-th distance), then goes
// through the segment's groups of 64 tiles outwards from that position: a
// group, and inside it a tile, is looked into only if for SOME lane the
// distance from its query to the box is not above that query's k-th distance.
// Boxes are tested 64 at a time first (one per lane, against the box around
// the wave's queries and the wave's largest k-th distance); the few that pass
// are broadcast lane by lane for the per-query test (a dozen vector
// instructions per box for all 64 queries).  That box distance is
// computed with the operations of the exact chain (one difference per axis,
// product, fused multiply-adds in the same order) applied to per-axis gaps
// that are not above any row's difference: rounding is monotone, so the value
// is never above the computed distance of any row of the box, and a skipped
// tile cannot hold a neighbour.  Testing per query, not per wave, bounds the
// work of a wave whose queries straddle a jump of the curve: it pays for the
// neighbourhoods of its queries, not for the space between them.
// Rows of a scanned tile are uniform over the wave as well; a lane whose
// distance passes its own bound parks (distance, row) in a queue in LDS, and
// the queues are emptied into the sorted lists by all lanes together when one
// fills up, as in the scanning kernels.  Rows arrive out of row order here, so
// a row of EQUAL distance may still displace a neighbour with a larger row
// number: a full list admits d <= its k-th distance and the 64-bit
// (distance, row) keys decide.
#include "device_utils.hpp"
#include "knn_binned_mc_impl.hpp"
#include "knn_lowd_impl.hpp"
#include "launchers.hpp"

#include <climits>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>

#include <rocprim/device/device_radix_sort.hpp>

namespace pca {

namespace {

constexpr int kBinQueueCap = 16;  // parked rows per lane

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// floats as integers of the same order (for atomic min / max)
__device__ __forceinline__ int ordered_int(float f) {
  const int i = __float_as_int(f);
  return i >= 0 ? i : i ^ 0x7fffffff;
}
__device__ __forceinline__ float from_ordered_int(int i) {
  return __int_as_float(i >= 0 ? i : i ^ 0x7fffffff);
}

__device__ __forceinline__ int find_segment64(const int64_t *__restrict__ ptr,
                                              int num_segments, int64_t v) {
  if (ptr == nullptr)
    return 0;
  int lo = 0, hi = num_segments;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (ptr[mid] <= v)
      lo = mid;
    else
      hi = mid;
  }
  return lo;
}

// The first launch of a binned search (a call starts with kernels so short
// that the host's launch rate sets the pace: one launch instead of five):
// workgroups 0-3 count the work items of the segments - tiles and groups of
// tiles of x, tasks of 64 and of 32 queries of y -, the others empty the
// segment boxes and the extra task slots.  seg_box: [num_segments][6] = lower
// corner, upper corner (ordered integers).
struct BinsSetup {
  const int64_t *ptr_x, *ptr_y;
  int n, m, num_segments;
  int *tile_start, *group_start, *wave_start, *half_start;
  int *seg_box;
  // task slots (task_span_kernel's; task_extra == 0: no tasks wanted)
  int task_blocks, task_extra;
  int *extra_used;
  int2 *task_desc;
};
__global__ __launch_bounds__(kPlanThreads) void bins_setup_kernel(BinsSetup s) {
  __shared__ int partial[kPlanThreads];
  const int job = blockIdx.x; // (uniform over the workgroup)
  if (job == 0) {
    plan_segments(s.ptr_x, s.n, s.num_segments, kBinTile, s.tile_start,
                  partial);
  } else if (job == 1) {
    plan_segments(s.ptr_x, s.n, s.num_segments, kBinTile * kBinGroup,
                  s.group_start, partial);
  } else if (job == 2) {
    plan_segments(s.ptr_y, s.m, s.num_segments, kWave, s.wave_start, partial);
  } else if (job == 3) {
    plan_segments(s.ptr_y, s.m, s.num_segments, kWave / 2, s.half_start,
                  partial);
  } else {
    const int i = (job - 4) * kPlanThreads + (int)threadIdx.x;
    if (i < 6 * s.num_segments)
      s.seg_box[i] = (i % 6) < 3 ? INT_MAX : INT_MIN;
    // the extra task slots start out unused
    if (i == 0 && s.extra_used != nullptr)
      *s.extra_used = 0;
    if (i < s.task_extra)
      s.task_desc[s.task_blocks + i] = make_int2(0, 0);
  }
}

// Bounding box of the finite coordinates of every segment; grid (parts,
// up to 65,535 segments at a time).
__global__ __launch_bounds__(kBlock) void seg_box_kernel(
    const float *__restrict__ x, const int64_t *__restrict__ ptr_x, int n,
    int d, int seg_count, int *__restrict__ seg_box) {
  __shared__ float part[kBlock / kWave][6];
  for (int seg = blockIdx.y; seg < seg_count; seg += gridDim.y) {
    const int64_t begin = ptr_x ? ptr_x[seg] : 0;
    const int64_t end = ptr_x ? ptr_x[seg + 1] : n;
    float lo[3], hi[3];
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      lo[c] = __builtin_inff();
      hi[c] = -__builtin_inff();
    }
    for (int64_t i = begin + (int64_t)blockIdx.x * kBlock + threadIdx.x;
         i < end; i += (int64_t)gridDim.x * kBlock) {
#pragma unroll
      for (int c = 0; c < 3; ++c)
        if (c < d) {
          const float v = x[(size_t)i * d + c];
          if (__builtin_fabsf(v) < __builtin_inff()) {
            lo[c] = __builtin_fminf(lo[c], v);
            hi[c] = __builtin_fmaxf(hi[c], v);
          }
        }
    }
#pragma unroll
    for (int c = 0; c < 3; ++c) {
#pragma unroll
      for (int sh = 1; sh < kWave; sh <<= 1) {
        lo[c] = __builtin_fminf(lo[c], __shfl_xor(lo[c], sh));
        hi[c] = __builtin_fmaxf(hi[c], __shfl_xor(hi[c], sh));
      }
    }
    // one set of atomic updates per workgroup
    __syncthreads(); // (the previous segment's values have been read)
    if ((threadIdx.x & (kWave - 1)) == 0) {
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        part[threadIdx.x / kWave][c] = lo[c];
        part[threadIdx.x / kWave][3 + c] = hi[c];
      }
    }
    __syncthreads();
    if (threadIdx.x < 6) {
      float v = part[0][threadIdx.x];
      for (int w = 1; w < kBlock / kWave; ++w)
        v = threadIdx.x < 3 ? __builtin_fminf(v, part[w][threadIdx.x])
                            : __builtin_fmaxf(v, part[w][threadIdx.x]);
      if (threadIdx.x < 3)
        atomicMin(&seg_box[seg * 6 + threadIdx.x], ordered_int(v));
      else
        atomicMax(&seg_box[seg * 6 + threadIdx.x], ordered_int(v));
    }
  }
}

// 10 bits spread to every third position
__device__ __forceinline__ uint32_t spread3(uint32_t v) {
  v &= 0x3ffu;
  v = (v | (v << 16)) & 0x030000ffu;
  v = (v | (v << 8)) & 0x0300f00fu;
  v = (v | (v << 4)) & 0x030c30c3u;
  v = (v | (v << 2)) & 0x09249249u;
  return v;
}

// keys[i] = (segment << 3 axis_bits) | Morton code of row i inside its
// segment's box of x rows, axis_bits bits per axis (coordinates outside the
// box, NaN and missing axes go to its border); vals[i] = i.
__global__ __launch_bounds__(kBlock) void morton_keys_kernel(
    const float *__restrict__ pts, const int64_t *__restrict__ ptr, int count,
    int d, int num_segments, const int *__restrict__ seg_box,
    int axis_bits, uint32_t *__restrict__ keys,
    uint32_t *__restrict__ vals, bool searched_side) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= count)
    return;
  // rows of x behind the last pointer belong to no segment (a caller's
  // batch_size below the ids in use: the reference never searches them,
  // csrc/cuda/utils.cuh:11-19): they sort behind every segment's rows
  if (searched_side && ptr != nullptr && (int64_t)i >= ptr[num_segments]) {
    keys[i] = 0xffffffffu;
    vals[i] = (uint32_t)i;
    return;
  }
  const int seg = find_segment64(ptr, num_segments, i);
  uint32_t code = 0;
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    uint32_t cell = 0;
    if (c < d) {
      const float lo = from_ordered_int(seg_box[seg * 6 + c]);
      const float hi = from_ordered_int(seg_box[seg * 6 + 3 + c]);
      const float v = pts[(size_t)i * d + c];
      const float cells = (float)(1 << axis_bits);
      const float t = (v - lo) / (hi - lo) * cells;
      // (NaN, also from an empty or flat box, fails the first comparison)
      cell = t >= 0.0f ? (uint32_t)__builtin_fminf(t, cells - 1.0f) : 0u;
    }
    code |= spread3(cell) << c;
  }
  keys[i] = ((uint32_t)seg << (3 * axis_bits)) | code;
  vals[i] = (uint32_t)i;
}

// Rows in curve order with their row numbers (plain and as the matrix-core
// filter takes them), and the box of every tile of 32: half a wave per tile.
__global__ __launch_bounds__(kBlock) void gather_tiles_kernel(
    const float *__restrict__ x, const int64_t *__restrict__ ptr_x, int n,
    int d, int num_segments, const int *__restrict__ tile_start,
    const uint32_t *__restrict__ perm, float4 *__restrict__ rows,
    uint4 *__restrict__ packed, Box *__restrict__ box) {
  const int gt = (blockIdx.x * kBlock + threadIdx.x) / kBinTile;
  const int r = threadIdx.x & (kBinTile - 1);
  // behind the last row a tile of rows that never pass the filter (operand
  // w = NaN), so that a fetch of a whole tile stays inside the copy
  if (blockIdx.x == 0 && threadIdx.x < kBinTile) {
    packed[(size_t)(n + r) * 2] = make_uint4(0u, 0x7fc00000u, 0u, 0u);
    packed[(size_t)(n + r) * 2 + 1] = make_uint4(0u, 0u, 0u, 0u);
  }
  if (gt >= tile_start[num_segments])
    return;
  const int seg = find_segment(tile_start, num_segments, gt);
  const int x_begin = ptr_x ? (int)ptr_x[seg] : 0;
  const int x_end = ptr_x ? (int)ptr_x[seg + 1] : n;
  const int j = x_begin + (gt - tile_start[seg]) * kBinTile + r;
  const bool ok = j < x_end;
  const uint32_t id = ok ? perm[j] : 0u;
  float v[3];
#pragma unroll
  for (int c = 0; c < 3; ++c)
    v[c] = (ok && c < d) ? x[(size_t)id * d + c] : 0.0f;
  if (ok) {
    // (the plain copy is read by the vector-ALU scans only)
    if (rows != nullptr)
      rows[j] = make_float4(v[0], v[1], v[2], __uint_as_float(id));
    // the operand of the matrix-core filter, then coordinates and row number
    uint4 rec[McShape<3>::REC];
    mc_pack_row<3>(v, rec);
    rec[1].w = id;
    packed[(size_t)j * 2] = rec[0];
    packed[(size_t)j * 2 + 1] = rec[1];
  }
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    // (fminf / fmaxf drop a NaN operand: a NaN coordinate is in no box, and
    // such a row has no distance below the limit either)
    float lo = ok ? v[c] : __builtin_inff();
    float hi = ok ? v[c] : -__builtin_inff();
#pragma unroll
    for (int sh = 1; sh < kBinTile; sh <<= 1) {
      lo = __builtin_fminf(lo, __shfl_xor(lo, sh));
      hi = __builtin_fmaxf(hi, __shfl_xor(hi, sh));
    }
    if (r == 0) {
      box[gt].lo[c] = lo;
      box[gt].hi[c] = hi;
    }
  }
  uint32_t min_row = ok ? id : 0xffffffffu;
#pragma unroll
  for (int sh = 1; sh < kBinTile; sh <<= 1)
    min_row = min(min_row, (uint32_t)__shfl_xor((int)min_row, sh));
  if (r == 0) {
    box[gt].min_row = min_row;
    box[gt].pad = 0u;
  }
}

// Boxes of the groups of kBinGroup consecutive tiles of a segment: one wave
// per group.
__global__ __launch_bounds__(kBlock) void group_boxes_kernel(
    int num_segments, const int *__restrict__ tile_start,
    const int *__restrict__ group_start, const Box *__restrict__ box,
    Box *__restrict__ group_box) {
  const int gg = (blockIdx.x * kBlock + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (gg >= group_start[num_segments])
    return;
  const int seg = find_segment(group_start, num_segments, gg);
  const int t = (gg - group_start[seg]) * kBinGroup + lane;
  const int tiles = tile_start[seg + 1] - tile_start[seg];
  const bool ok = t < tiles;
  static_assert(kBinGroup == kWave, "one tile per lane");
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    float lo = ok ? box[tile_start[seg] + t].lo[c] : __builtin_inff();
    float hi = ok ? box[tile_start[seg] + t].hi[c] : -__builtin_inff();
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1) {
      lo = __builtin_fminf(lo, __shfl_xor(lo, sh));
      hi = __builtin_fmaxf(hi, __shfl_xor(hi, sh));
    }
    if (lane == 0) {
      group_box[gg].lo[c] = lo;
      group_box[gg].hi[c] = hi;
    }
  }
  uint32_t min_row = ok ? box[tile_start[seg] + t].min_row : 0xffffffffu;
#pragma unroll
  for (int sh = 1; sh < kWave; sh <<= 1)
    min_row = min(min_row, (uint32_t)__shfl_xor((int)min_row, sh));
  if (lane == 0) {
    group_box[gg].min_row = min_row;
    group_box[gg].pad = 0u;
  }
}

template <int K>
__global__ __launch_bounds__(kBlock) void knn_binned_kernel(BinnedParams p) {
  // parked rows: distance and row number, [slot][thread]
  __shared__ float queue_d[2 * kBinQueueCap][kBlock];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int task = blockIdx.x * (kBlock / kWave) +
                   __builtin_amdgcn_readfirstlane(tid / kWave);
  if (task >= p.wave_start[p.num_segments])
    return; // (whole waves leave; no barrier below)
  const int seg = find_segment(p.wave_start, p.num_segments, task);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int jq = y_begin + (task - p.wave_start[seg]) * kWave + lane;
  const bool valid = jq < y_end;
  const int q = valid ? (int)p.perm_y[jq] : 0;
  const int k = p.k;
  const int d_in = p.d;

  float yq[3];
#pragma unroll
  for (int c = 0; c < 3; ++c)
    yq[c] = (valid && c < d_in) ? p.y[(size_t)q * d_in + c] : 0.0f;
  // a query with a coordinate that is not finite has no distance below the
  // limit: it looks at nothing and returns nothing
  const bool searching = valid && __builtin_fabsf(yq[0]) < __builtin_inff() &&
                         __builtin_fabsf(yq[1]) < __builtin_inff() &&
                         __builtin_fabsf(yq[2]) < __builtin_inff();

  // the wave's box (lanes that do not search stay out)
  float q_lo[3], q_hi[3];
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    float lo = searching ? yq[c] : __builtin_inff();
    float hi = searching ? yq[c] : -__builtin_inff();
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1) {
      lo = __builtin_fminf(lo, __shfl_xor(lo, sh));
      hi = __builtin_fmaxf(hi, __shfl_xor(hi, sh));
    }
    q_lo[c] = lo;
    q_hi[c] = hi;
  }

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - k) ? lowest_key() : empty_key();
  // a row is parked when its distance is strictly below `admit`: the limit
  // while the list has room, just above the k-th distance afterwards (a row of
  // equal distance and smaller number still gets in); nothing for a lane
  // that does not search.  `kth`: the k-th distance (the limit while the list
  // has room; below every distance for a lane that does not search): a box
  // farther away than that holds no neighbour of this lane's query.
  float admit = searching ? kKnnSentinel : -__builtin_inff();
  float kth = searching ? kKnnSentinel : -1.0f;
  // byte offset in the queue at which the lane's next row goes
  const int park_first = tid * (int)sizeof(float);
  int park_at = park_first;

  auto drain = [&]() {
    for (;;) {
      const bool has = park_at > park_first;
      if (!__any(has))
        break;
      park_at -= has ? kBlock * (int)sizeof(float) : 0;
      const float *slot = reinterpret_cast<const float *>(
          reinterpret_cast<const char *>(&queue_d[0][0]) + park_at);
      const float d = slot[0];
      const uint32_t id = __float_as_uint(slot[kBinQueueCap * kBlock]);
      // (parked under an older bound: the keys sort it out)
      const double key = (has && d < admit) ? make_key(d, id) : empty_key();
      sorted_insert<K>(best, key);
      const float now = key_dist(best[K - 1]);
      if (searching && now < kKnnSentinel) {
        kth = now;
        admit = next_up_positive(now);
      }
    }
  };

  // rows of one tile against every lane's query, four rows per step (the
  // copy of the rows is padded, so a step may read past the tile's rows;
  // FULL: the tile has all its 32 rows, no step needs a bound)
  auto scan_rows = [&](const float4 *__restrict__ src, int rows,
                       auto full) {
    constexpr bool FULL = decltype(full)::value;
    for (int r = 0; r < (FULL ? kBinTile : rows); r += 4) {
      float4 row[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        row[u] = src[r + u]; // (uniform addresses)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float d0 = row[u].x - yq[0];
        float dd = d0 * d0;
        const float d1 = row[u].y - yq[1];
        dd = __builtin_fmaf(d1, d1, dd);
        const float d2 = row[u].z - yq[2];
        dd = __builtin_fmaf(d2, d2, dd);
        const bool hit = dd < admit && (FULL || r + u < rows);
        if (hit) {
          // (one address for both queues: the row numbers sit a fixed
          // distance behind the distances)
          float *slot = reinterpret_cast<float *>(
              reinterpret_cast<char *>(&queue_d[0][0]) + park_at);
          slot[0] = dd;
          slot[kBinQueueCap * kBlock] = row[u].w;
          park_at += kBlock * (int)sizeof(float);
        }
      }
      if (__any(park_at > park_first + (kBinQueueCap - 4) * kBlock *
                                          (int)sizeof(float)))
        drain();
    }
  };
  auto scan_tile = [&](int tile) {
    const int j0 = x_begin + tile * kBinTile;
    const int rows = min(kBinTile, x_end - j0);
    if (rows == kBinTile)
      scan_rows(p.rows + j0, rows, std::true_type{});
    else
      scan_rows(p.rows + j0, rows, std::false_type{});
  };

  // largest k-th distance among the wave's queries
  auto wave_reach = [&]() {
    float r = kth;
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1)
      r = __builtin_fmaxf(r, __shfl_xor(r, sh));
    return r;
  };
  // Of the 64 boxes the lanes hold (lane l: box l, `mine` = it exists), is
  // the box of lane `src` within reach of some lane's query?  (A NaN - from an
  // infinite or empty box - never rules a box out.)
  auto reachable = [&](const Box &held, int src) {
    float lo[3], hi[3];
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      lo[c] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
          (int)__float_as_uint(held.lo[c]), src));
      hi[c] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
          (int)__float_as_uint(held.hi[c]), src));
    }
    return __any(!(box_gap2(lo, hi, yq, yq) > kth));
  };
  const int tile0 = p.tile_start[seg];
  const int num_tiles = p.tile_start[seg + 1] - tile0;
  if (num_tiles > 0) {
    // where the wave's first and last query fall in the order of x
    const int last_lane = min(kWave, y_end - (jq - lane)) - 1;
    const uint32_t key_first =
        p.keys_y[__builtin_amdgcn_readfirstlane(jq - lane)];
    const uint32_t key_last =
        p.keys_y[__builtin_amdgcn_readfirstlane(jq - lane + last_lane)];
    const int pos_first =
        wave_lower_bound(p.keys_x, x_begin, x_end, key_first, lane);
    const int pos_last =
        wave_lower_bound(p.keys_x, x_begin, x_end, key_last, lane);
    const int t_first = min(num_tiles - 1, (pos_first - x_begin) / kBinTile);
    const int t_last = min(num_tiles - 1, (pos_last - x_begin) / kBinTile);
    // tiles seed_lo .. seed_hi are scanned up front
    int seed_lo = max(0, t_first - 1);
    int seed_hi = min(num_tiles - 1, max(t_last, t_first) + 1);
    if (seed_hi - seed_lo + 1 > kBinSeedTiles) {
      // queries far apart in the order of x: the middle of their range
      const int mid = (seed_lo + seed_hi) / 2;
      seed_lo = max(0, mid - kBinSeedTiles / 2);
      seed_hi = min(num_tiles - 1, seed_lo + kBinSeedTiles - 1);
    }
    for (int t = seed_lo; t <= seed_hi; ++t)
      scan_tile(t);
    drain();
    float reach = wave_reach();

    // Groups of tiles, 64 at a time (one box per lane), nearest to the seed
    // tiles first.  A group, then a tile, is looked into if its box is within
    // the wave's largest k-th distance of the box around the wave's queries
    // (all 64 boxes at once), and then within some query's own k-th distance
    // of that query (a dozen instructions per box).
    const int group0 = p.group_start[seg];
    const int num_groups = (num_tiles + kBinGroup - 1) / kBinGroup;
    const int centre = ((seed_lo + seed_hi) / 2) / kBinGroup;
    const int num_rounds = (num_groups + kWave - 1) / kWave;
    const int centre_round = centre / kWave;
    for (int i = 0; i < 2 * num_rounds; ++i) {
      const int round = centre_round + ((i & 1) ? -((i + 1) >> 1) : (i >> 1));
      if (round < 0 || round >= num_rounds)
        continue;
      const int g_mine = round * kWave + lane;
      Box g_box = {};
      if (g_mine < num_groups)
        g_box = p.group_box[group0 + g_mine];
      uint64_t g_todo =
          __ballot(g_mine < num_groups &&
                   !(box_gap2(g_box.lo, g_box.hi, q_lo, q_hi) > reach));
      const int g_at = min(max(centre - round * kWave, 0), kWave - 1);
      while (g_todo != 0) {
        const int g_lane = nearest_bit(g_todo, g_at);
        g_todo &= ~((uint64_t)1 << g_lane);
        if (!reachable(g_box, g_lane))
          continue;
        const int group = round * kWave + g_lane;
        const int t_mine = group * kBinGroup + lane;
        const bool t_ok =
            t_mine < num_tiles && !(t_mine >= seed_lo && t_mine <= seed_hi);
        Box t_box = {};
        if (t_ok)
          t_box = p.box[tile0 + t_mine];
        uint64_t t_todo = __ballot(
            t_ok && !(box_gap2(t_box.lo, t_box.hi, q_lo, q_hi) > reach));
        while (t_todo != 0) {
          const int t_lane = (int)__builtin_ctzll(t_todo);
          t_todo &= t_todo - 1;
          if (!reachable(t_box, t_lane))
            continue;
          scan_tile(group * kBinGroup + t_lane);
        }
        if (__any(park_at > park_first)) {
          drain();
          reach = wave_reach();
        }
      }
    }
    drain();
  }

  if (valid)
    write_dense<K>(best, k, q, p.out_idx, p.out_dist, p.out_count);
}

// The radius search over the same bins (reference: radius_kernel,
// csrc/cuda/radius_cuda.cu:9-42): every row with a squared distance strictly
// below r2, at most `slots` of them - the ones with the smallest row numbers,
// in ascending order.  The radius is known from the start, so there are no
// seed tiles: boxes at r2 or farther from every query are skipped, rows that
// qualify are parked by number, and the lists keep the `slots` smallest
// numbers (as doubles; a full list admits only smaller numbers).
template <int K>
__global__ __launch_bounds__(kBlock) void radius_binned_kernel(
    BinnedParams p, float r2, int ignore_same_index) {
  __shared__ uint32_t queue[kBinQueueCap][kBlock];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int task = blockIdx.x * (kBlock / kWave) +
                   __builtin_amdgcn_readfirstlane(tid / kWave);
  if (task >= p.wave_start[p.num_segments])
    return; // (whole waves leave; no barrier below)
  const int seg = find_segment(p.wave_start, p.num_segments, task);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int jq = y_begin + (task - p.wave_start[seg]) * kWave + lane;
  const bool valid = jq < y_end;
  const int q = valid ? (int)p.perm_y[jq] : 0;
  const int slots = p.k;
  const int d_in = p.d;

  float yq[3];
#pragma unroll
  for (int c = 0; c < 3; ++c)
    yq[c] = (valid && c < d_in) ? p.y[(size_t)q * d_in + c] : 0.0f;
  // (a coordinate that is not finite: no distance below r2)
  const bool searching = valid && __builtin_fabsf(yq[0]) < __builtin_inff() &&
                         __builtin_fabsf(yq[1]) < __builtin_inff() &&
                         __builtin_fabsf(yq[2]) < __builtin_inff();
  float q_lo[3], q_hi[3];
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    float lo = searching ? yq[c] : __builtin_inff();
    float hi = searching ? yq[c] : -__builtin_inff();
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1) {
      lo = __builtin_fminf(lo, __shfl_xor(lo, sh));
      hi = __builtin_fmaxf(hi, __shfl_xor(hi, sh));
    }
    q_lo[c] = lo;
    q_hi[c] = hi;
  }

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - slots) ? -__builtin_inf() : __builtin_inf();
  // rows with a number below `below` are parked: all while the list has
  // room, those under its largest number afterwards; none for a lane that
  // does not search
  uint32_t below = searching ? 0xffffffffu : 0u;
  const uint32_t self = ignore_same_index ? (uint32_t)q : 0xffffffffu;
  // a lane without a query never passes d < limit
  const float limit = searching ? r2 : -__builtin_inff();
  int parked = 0;

  auto drain = [&]() {
    for (;;) {
      const bool has = parked > 0;
      if (!__any(has))
        break;
      parked -= has ? 1 : 0;
      const uint32_t id = queue[has ? parked : 0][tid];
      const double key = (has && id < below) ? (double)id : __builtin_inf();
      sorted_insert<K>(best, key);
      if (searching && best[K - 1] < __builtin_inf())
        below = (uint32_t)best[K - 1];
    }
  };

  auto scan_tile = [&](int tile) {
    const int j0 = x_begin + tile * kBinTile;
    const int rows = min(kBinTile, x_end - j0);
    const float4 *__restrict__ src = p.rows + j0;
    for (int r = 0; r < rows; r += 4) {
      float4 row[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        row[u] = src[r + u]; // (uniform addresses; the copy is padded)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float d0 = row[u].x - yq[0];
        float dd = d0 * d0;
        const float d1 = row[u].y - yq[1];
        dd = __builtin_fmaf(d1, d1, dd);
        const float d2 = row[u].z - yq[2];
        dd = __builtin_fmaf(d2, d2, dd);
        const uint32_t id = __float_as_uint(row[u].w);
        const bool hit = dd < limit && id < below && id != self &&
                         r + u < rows;
        if (hit) {
          queue[parked][tid] = id;
          ++parked;
        }
      }
      if (__any(parked > kBinQueueCap - 4))
        drain();
    }
  };

  // is the box of lane `src` closer than the radius to some lane's query?
  // (A NaN - from an infinite or empty box - never rules a box out.)
  auto reachable = [&](const Box &held, int src) {
    float lo[3], hi[3];
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      lo[c] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
          (int)__float_as_uint(held.lo[c]), src));
      hi[c] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
          (int)__float_as_uint(held.hi[c]), src));
    }
    return __any(searching && !(box_gap2(lo, hi, yq, yq) >= r2));
  };

  const int tile0 = p.tile_start[seg];
  const int num_tiles = p.tile_start[seg + 1] - tile0;
  const int group0 = p.group_start[seg];
  const int num_groups = (num_tiles + kBinGroup - 1) / kBinGroup;
  if (__any(searching)) {
    for (int g_base = 0; g_base < num_groups; g_base += kWave) {
      const int g_mine = g_base + lane;
      Box g_box = {};
      if (g_mine < num_groups)
        g_box = p.group_box[group0 + g_mine];
      uint64_t g_todo =
          __ballot(g_mine < num_groups &&
                   !(box_gap2(g_box.lo, g_box.hi, q_lo, q_hi) >= r2));
      while (g_todo != 0) {
        const int g_lane = (int)__builtin_ctzll(g_todo);
        g_todo &= g_todo - 1;
        if (!reachable(g_box, g_lane))
          continue;
        const int group = g_base + g_lane;
        const int t_mine = group * kBinGroup + lane;
        Box t_box = {};
        if (t_mine < num_tiles)
          t_box = p.box[tile0 + t_mine];
        uint64_t t_todo =
            __ballot(t_mine < num_tiles &&
                     !(box_gap2(t_box.lo, t_box.hi, q_lo, q_hi) >= r2));
        while (t_todo != 0) {
          const int t_lane = (int)__builtin_ctzll(t_todo);
          t_todo &= t_todo - 1;
          if (reachable(t_box, t_lane))
            scan_tile(group * kBinGroup + t_lane);
        }
        if (__any(parked > 0))
          drain();
      }
    }
  }

  if (valid) {
    const size_t row = (size_t)q * slots;
    int found = 0;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int e = j - (K - slots);
      if (e >= 0 && best[j] < __builtin_inf()) {
        p.out_idx[row + e] = (int)best[j];
        ++found;
      }
    }
    p.out_count[q] = found;
  }
}

struct BinnedLayout {
  size_t seg_box, keys_a, keys_b, keys_x, keys_y, vals_a, vals_b, perm_x,
      perm_y, rows, packed, box, group_box, tile_start, group_start,
      wave_start, half_start, task_keys, sort_temp, side_temp;
  int tiles_bound, groups_bound;
  size_t total() const {
    return seg_box + keys_a + keys_b + keys_x + keys_y + vals_a + vals_b +
           perm_x + perm_y + rows + packed + box + group_box + tile_start +
           group_start + wave_start + half_start + task_keys + sort_temp +
           side_temp;
  }
};

// Keys are 32 bits: the segment above the Morton code, whose bits per axis
// (at most 10) shrink as the segments get more (and with that smaller).
int segment_bits(int num_segments) {
  int bits = 0;
  while (bits < 31 && ((int64_t)1 << bits) < num_segments)
    ++bits;
  return bits;
}
int axis_bits(int num_segments) {
  return std::min(10, (32 - segment_bits(num_segments)) / 3);
}

// rocPRIM's radix sort with this file's choices (measured on 1.03 M pairs
// with 30-bit keys: the library's default - merge sort up to 2^20 items, 19
// launches - 170 us; its one-sweep radix sort as configured by default
// 140 us; the same with workgroups of 1,024 threads x 8 items and the
// match-based ranking 109 us, and 98 us with 10 bits per pass, which saves
// the fourth pass).  Below 200,000 items the merge sort is quicker (54 us
// against 68 us at 131,072).
template <unsigned int RadixBits>
using SortConfig = rocprim::radix_sort_config<
    rocprim::default_config, rocprim::default_config,
    rocprim::radix_sort_onesweep_config<
        rocprim::kernel_config<256, 12>, rocprim::kernel_config<1024, 8>,
        RadixBits, rocprim::block_radix_rank_algorithm::match>,
    200000>;

hipError_t sort_pairs(void *temp, size_t &temp_bytes, const uint32_t *keys_in,
                      uint32_t *keys_out, const uint32_t *vals_in,
                      uint32_t *vals_out, int count, int num_segments,
                      hipStream_t stream) {
  const unsigned int bits = (unsigned int)std::max(
      segment_bits(num_segments) + 3 * axis_bits(num_segments), 1);
  // (10 bits per pass where that takes fewer passes than 8)
  if ((bits + 9) / 10 < (bits + 7) / 8)
    return rocprim::radix_sort_pairs<SortConfig<10>>(
        temp, temp_bytes, keys_in, keys_out, vals_in, vals_out,
        (unsigned int)count, 0u, bits, stream, false);
  return rocprim::radix_sort_pairs<SortConfig<8>>(
      temp, temp_bytes, keys_in, keys_out, vals_in, vals_out,
      (unsigned int)count, 0u, bits, stream, false);
}

// Tasks in a row that one XCD takes, as a power of two: long runs keep what a
// task fetches in the L2 its neighbours fill (256 in a row: 258 MB fetched by
// the search kernel of the 1 M-point workload, 8 in a row: 594 MB, at the
// same speed), but every XCD needs a few runs for its share of the long tasks
// at the front of the order.  PCA_BINNED_XCD_RUN_LOG2 overrides.
int xcd_run_log2(int tasks) {
  static const int fixed = [] {
    const char *text = std::getenv("PCA_BINNED_XCD_RUN_LOG2");
    if (!text)
      return -1;
    const int v = std::atoi(text);
    return v < 0 ? 0 : (v > 12 ? 12 : v);
  }();
  if (fixed >= 0)
    return fixed;
  int log2 = 3;
  while (log2 < 8 && (size_t)(8 << (log2 + 1)) * 3 <= (size_t)tasks)
    ++log2;
  return log2;
}

// Workgroups of a search on matrix cores: whole runs on each of the 8 XCDs.
int xcd_run_grid(int tasks) {
  const int unit = 8 << xcd_run_log2(tasks);
  return (tasks + unit - 1) / unit * unit;
}

// Task slots for `blocks` blocks of 32 queries: one each, and half as many
// again for the parts of split blocks - while the blocks are not many more
// than the waves the device holds at once (256 CUs x 4 SIMDs x 4 waves).  With
// several rounds of waves the long tasks, started first, are covered by the
// others, and splitting only adds work (measured: it gains 15-25 % up to
// ~4,000 blocks and loses 5 % at 8,000).
int task_slots(int blocks) {
  return blocks <= 6144 ? blocks + (blocks / 6) * 3 : blocks;
}

// Words of the task-slot buffer (see TaskBuffers).
size_t task_buffer_words(int m, int num_segments) {
  const int blocks = plan_upper_bound(m, num_segments, kWave / 2);
  const int groups = (blocks + kBlock - 1) / kBlock;
  return 64 + 4 * (size_t)task_slots(blocks) + (size_t)kTaskClasses * groups;
}

BinnedLayout binned_layout(int n, int m, int num_segments) {
  BinnedLayout w;
  w.seg_box = align256(sizeof(int) * 6 * (size_t)num_segments);
  // unsorted (key, row) of the rows (a) and of the queries (b): the two are
  // sorted at the same time
  w.keys_a = align256(sizeof(uint32_t) * (size_t)n);
  w.keys_b = align256(sizeof(uint32_t) * (size_t)m);
  w.keys_x = align256(sizeof(uint32_t) * (size_t)n);
  w.keys_y = align256(sizeof(uint32_t) * (size_t)m);
  w.vals_a = align256(sizeof(uint32_t) * (size_t)n);
  w.vals_b = align256(sizeof(uint32_t) * (size_t)m);
  w.perm_x = align256(sizeof(uint32_t) * (size_t)n);
  w.perm_y = align256(sizeof(uint32_t) * (size_t)m);
  // (padded: the search reads rows four at a time)
  w.rows = align256(sizeof(float4) * ((size_t)n + kBinTile));
  w.packed = align256(sizeof(uint4) * 2 * ((size_t)n + kBinTile));
  w.tiles_bound = plan_upper_bound(n, num_segments, kBinTile);
  w.groups_bound = plan_upper_bound(n, num_segments, kBinTile * kBinGroup);
  w.box = align256(sizeof(Box) * (size_t)w.tiles_bound);
  w.group_box = align256(sizeof(Box) * (size_t)w.groups_bound);
  w.tile_start = align256(sizeof(int) * (size_t)(num_segments + 1));
  w.group_start = align256(sizeof(int) * (size_t)(num_segments + 1));
  w.wave_start = align256(sizeof(int) * (size_t)(num_segments + 1));
  w.half_start = align256(sizeof(int) * (size_t)(num_segments + 1));
  // per task slot: descriptor (2 words), class, place in the starting order;
  // a histogram of the classes per kBlock blocks
  w.task_keys = align256(sizeof(uint32_t) * task_buffer_words(m, num_segments));
  // (the sort's size queries are kept per thread for the sizes asked last:
  // a call asks for the same layout three times -- workspace query, argument
  // check, carving)
  struct SortSizes {
    int n = -1, m = -1, num_segments = -1;
    size_t tx = 0, ty = 0;
    bool sized = false;
  };
  thread_local SortSizes last;
  if (last.n != n || last.m != m || last.num_segments != num_segments) {
    last.n = n;
    last.m = m;
    last.num_segments = num_segments;
    last.tx = last.ty = 0;
    const hipError_t ex =
        sort_pairs(nullptr, last.tx, nullptr, nullptr, nullptr, nullptr, n,
                   num_segments, nullptr);
    const hipError_t ey =
        sort_pairs(nullptr, last.ty, nullptr, nullptr, nullptr, nullptr, m,
                   num_segments, nullptr);
    last.sized = ex == hipSuccess && ey == hipSuccess;
  }
  const size_t tx = last.tx, ty = last.ty;
  // (a failed size query leaves a size no workspace can meet)
  const bool sized = last.sized;
  w.sort_temp = sized ? align256(tx) : ~(size_t)0 / 2;
  // (the queries are sorted beside the rows' stream)
  w.side_temp = sized ? align256(ty) : 0;
  return w;
}

// Everything a binned search reads, as prepare_bins leaves it in the scratch.
struct Bins {
  const int *tile_start, *group_start;
  const int *wave_start; // tasks of 64 queries
  const int *half_start; // tasks of 32 queries
  const uint32_t *keys_x, *keys_y, *perm_y;
  const float4 *rows;
  const uint4 *packed;
  const Box *box, *group_box;
  // the tasks of 32 queries in starting order (when asked for)
  const int2 *task_desc;
  const uint32_t *task_order;
  int task_slots; // slots of the order
  int task_grid;  // workgroups that cover them: whole runs of
                  // 2^xcd_run_log2(task_slots) tasks on each of 8 XCDs
  int code_bits;
};

// A second stream of the device: the queries are ordered there while the rows
// are ordered on the caller's stream (both chains are short kernels that
// leave most of the device idle).  The library keeps one such stream and two
// events per device, made at the first call that needs them and held until
// the process ends; fork / join are recorded and waited for within one call,
// under g_lane_mutex (held only while that call queues its work).
struct SideLane {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
};
constexpr int kMaxDevices = 64;
constexpr int kSideLaneQueries = 131072; // fewer queries stay on one stream
std::mutex g_lane_mutex;
SideLane g_lanes[kMaxDevices];

// The current device's lane, made at its first use (g_lane_mutex held).
// PCA_BINNED_SIDE_STREAM=0 (diagnostic switch) keeps everything on the
// caller's stream: `lane` stays null.
hipError_t side_lane(SideLane *&lane) {
  lane = nullptr;
  const char *env = getenv("PCA_BINNED_SIDE_STREAM");
  if (env != nullptr && env[0] == '0')
    return hipSuccess;
  int device = 0;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess)
    return err;
  if (device < 0 || device >= kMaxDevices)
    return hipSuccess;
  SideLane &mine = g_lanes[device];
  if (mine.stream == nullptr) {
    SideLane made;
    if ((err = hipStreamCreateWithFlags(&made.stream, hipStreamNonBlocking)) !=
        hipSuccess)
      return err;
    if ((err = hipEventCreateWithFlags(&made.fork, hipEventDisableTiming)) !=
            hipSuccess ||
        (err = hipEventCreateWithFlags(&made.join, hipEventDisableTiming)) !=
            hipSuccess) {
      // nothing half-made is kept
      if (made.fork != nullptr)
        (void)hipEventDestroy(made.fork);
      (void)hipStreamDestroy(made.stream);
      return err;
    }
    mine = made;
  }
  lane = &mine;
  return hipSuccess;
}

// The tasks (blocks of 32 queries, long spans split) and their starting
// order, from the sorted keys of the queries; results in `bins`.
// The pieces of the task-slot buffer.
struct TaskBuffers {
  int blocks, slots, groups; // groups: workgroups of kBlock blocks
  int *extra_used;
  int2 *desc;
  uint32_t *cls, *order;
  int *hist;
};
TaskBuffers task_buffers(uint32_t *task_keys, int m, int num_segments) {
  TaskBuffers t;
  t.blocks = plan_upper_bound(m, num_segments, kWave / 2);
  t.slots = task_slots(t.blocks);
  t.groups = (t.blocks + kBlock - 1) / kBlock;
  t.extra_used = reinterpret_cast<int *>(task_keys);
  t.desc = reinterpret_cast<int2 *>(task_keys + 64);
  t.cls = task_keys + 64 + 2 * (size_t)t.slots;
  t.order = t.cls + t.slots;
  t.hist = reinterpret_cast<int *>(t.order + t.slots);
  return t;
}

// The tasks (blocks of 32 queries, long spans split) and their starting
// order, from the sorted keys of the queries; results in `bins`.  (The extra
// slots were cleared by bins_setup_kernel.)
hipError_t order_tasks(const SearchInput &in, Bins &bins, uint32_t *task_keys,
                       hipStream_t stream) {
  const TaskBuffers t = task_buffers(task_keys, in.m, in.num_segments);
  const int extra = t.slots - t.blocks;
  // (what task_span_kernel reads)
  BinnedParams p;
  memset(&p, 0, sizeof(p));
  p.ptr_y = in.ptr_y;
  p.m = in.m;
  p.num_segments = in.num_segments;
  p.wave_start = bins.half_start;
  p.keys_y = bins.keys_y;
  p.code_bits = 3 * axis_bits(in.num_segments);
  hipLaunchKernelGGL(task_span_kernel, dim3(t.groups), dim3(kBlock), 0, stream,
                     p, t.blocks, extra, t.extra_used, t.desc, t.cls, t.hist);
  hipLaunchKernelGGL(task_order_kernel, dim3(t.groups), dim3(kBlock), 0,
                     stream, t.blocks, extra, t.extra_used, t.cls, t.hist,
                     t.order);
  bins.task_desc = t.desc;
  bins.task_order = t.order;
  bins.task_slots = t.slots;
  bins.task_grid = xcd_run_grid(t.slots);
  bins.code_bits = p.code_bits;
  return hipGetLastError();
}

// Orders rows and queries along the curve, copies the rows, builds the boxes;
// with `with_tasks` also the tasks of 32 queries and their starting order.
hipError_t prepare_bins(const SearchInput &in, void *scratch, bool with_tasks,
                        bool plain_rows, Bins &bins, hipStream_t stream) {
  const BinnedLayout lay = binned_layout(in.n, in.m, in.num_segments);
  char *cursor = static_cast<char *>(scratch);
  auto take = [&cursor](size_t bytes) {
    char *piece = cursor;
    cursor += bytes;
    return static_cast<void *>(piece);
  };
  int *seg_box = static_cast<int *>(take(lay.seg_box));
  uint32_t *keys_a = static_cast<uint32_t *>(take(lay.keys_a));
  uint32_t *keys_b = static_cast<uint32_t *>(take(lay.keys_b));
  uint32_t *keys_x = static_cast<uint32_t *>(take(lay.keys_x));
  uint32_t *keys_y = static_cast<uint32_t *>(take(lay.keys_y));
  uint32_t *vals_a = static_cast<uint32_t *>(take(lay.vals_a));
  uint32_t *vals_b = static_cast<uint32_t *>(take(lay.vals_b));
  uint32_t *perm_x = static_cast<uint32_t *>(take(lay.perm_x));
  uint32_t *perm_y = static_cast<uint32_t *>(take(lay.perm_y));
  float4 *rows = static_cast<float4 *>(take(lay.rows));
  uint4 *packed = static_cast<uint4 *>(take(lay.packed));
  Box *box = static_cast<Box *>(take(lay.box));
  Box *group_box = static_cast<Box *>(take(lay.group_box));
  int *tile_start = static_cast<int *>(take(lay.tile_start));
  int *group_start = static_cast<int *>(take(lay.group_start));
  int *wave_start = static_cast<int *>(take(lay.wave_start));
  int *half_start = static_cast<int *>(take(lay.half_start));
  uint32_t *task_keys = static_cast<uint32_t *>(take(lay.task_keys));
  void *sort_temp = take(lay.sort_temp);
  void *side_temp = take(lay.side_temp);

  const float *x = static_cast<const float *>(in.x);
  const float *y = static_cast<const float *>(in.y);
  const int nseg = in.num_segments;
  // the rows searching for themselves (the graph entry points): one order
  // serves both sides
  const bool self_search = in.y == in.x && in.m == in.n &&
                           (in.ptr_y == in.ptr_x || in.ptr_x == nullptr);
  if (self_search) {
    keys_y = keys_x;
    perm_y = perm_x;
  }
  bins.tile_start = tile_start;
  bins.group_start = group_start;
  bins.wave_start = wave_start;
  bins.half_start = half_start;
  bins.keys_x = keys_x;
  bins.keys_y = keys_y;
  bins.perm_y = perm_y;
  bins.rows = rows;
  bins.packed = packed;
  bins.box = box;
  bins.group_box = group_box;
  bins.task_desc = nullptr;
  bins.task_order = nullptr;
  bins.task_slots = 0;
  bins.task_grid = 0;
  bins.code_bits = 0;

  hipError_t err;
  {
    BinsSetup setup;
    setup.ptr_x = in.ptr_x;
    setup.ptr_y = in.ptr_y;
    setup.n = in.n;
    setup.m = in.m;
    setup.num_segments = nseg;
    setup.tile_start = tile_start;
    setup.group_start = group_start;
    setup.wave_start = wave_start;
    setup.half_start = half_start;
    setup.seg_box = seg_box;
    const TaskBuffers t = task_buffers(task_keys, in.m, nseg);
    setup.task_blocks = t.blocks;
    setup.task_extra = with_tasks ? t.slots - t.blocks : 0;
    setup.extra_used = with_tasks ? t.extra_used : nullptr;
    setup.task_desc = t.desc;
    const int resets = std::max(6 * nseg, setup.task_extra);
    hipLaunchKernelGGL(bins_setup_kernel,
                       dim3(4 + (resets + kPlanThreads - 1) / kPlanThreads),
                       dim3(kPlanThreads), 0, stream, setup);
  }
  {
    // enough workgroups per segment to fill the device when segments are few
    // (more of them were no quicker: their atomic updates of the same few
    // words take turns)
    const int parts = std::max(
        1, std::min((in.n / nseg + 16 * kBlock - 1) / (16 * kBlock),
                    std::max(1, 1024 / nseg)));
    hipLaunchKernelGGL(seg_box_kernel, dim3(parts, std::min(nseg, 65535)),
                       dim3(kBlock), 0, stream, x, in.ptr_x, in.n, in.d, nseg,
                       seg_box);
  }
  if ((err = hipGetLastError()) != hipSuccess)
    return err;

  // The queries' chain (keys, sort, tasks) runs beside the rows' chain: it
  // forks off the caller's stream here and joins it again below - when it is
  // long enough to pay for the two waits between streams (measured, with
  // rocPRIM's default sort configuration: 0.82 -> 0.77 ms for 1.03 M rows and
  // 258 k queries, 0.68 -> 0.59 ms for 500 k queries among 1 M rows; a loss
  // of 0.02 ms at 65 k queries).  When the
  // rows' order serves the queries too, only the tasks are left to order,
  // which follows the rows' sort on the caller's stream.
  const bool beside = !self_search && in.m >= kSideLaneQueries;
  std::unique_lock<std::mutex> lane_lock(g_lane_mutex, std::defer_lock);
  SideLane *lane = nullptr;
  hipStream_t side = stream;
  // Once the side stream has work of this call, the caller's stream waits for
  // it on EVERY way out of this function -- also the failing ones: the
  // workspace may be reused as soon as the caller's stream gets there.
  struct Rejoin {
    SideLane *&lane;
    hipStream_t stream;
    bool forked = false, joined = false;
    hipError_t join() {
      if (!forked || joined || lane == nullptr)
        return hipSuccess;
      joined = true;
      hipError_t e = hipEventRecord(lane->join, lane->stream);
      if (e == hipSuccess)
        e = hipStreamWaitEvent(stream, lane->join, 0);
      return e;
    }
    ~Rejoin() { (void)join(); }
  } rejoin{lane, stream};
  auto fork = [&]() -> hipError_t {
    lane_lock.lock();
    hipError_t e = side_lane(lane);
    if (e != hipSuccess || lane == nullptr)
      return e;
    side = lane->stream;
    e = hipEventRecord(lane->fork, stream);
    if (e == hipSuccess)
      e = hipStreamWaitEvent(side, lane->fork, 0);
    rejoin.forked = e == hipSuccess;
    return e;
  };
  auto queries_chain = [&]() -> hipError_t {
    hipError_t e = hipSuccess;
    if (!self_search) {
      hipLaunchKernelGGL(morton_keys_kernel,
                         dim3((in.m + kBlock - 1) / kBlock), dim3(kBlock), 0,
                         side, y, in.ptr_y, in.m, in.d, nseg, seg_box,
                         axis_bits(nseg), keys_b, vals_b, false);
      if ((e = hipGetLastError()) != hipSuccess)
        return e;
      size_t bytes = lay.side_temp;
      if ((e = sort_pairs(side_temp, bytes, keys_b, keys_y, vals_b, perm_y,
                          in.m, nseg, side)) != hipSuccess)
        return e;
    }
    if (with_tasks)
      e = order_tasks(in, bins, task_keys, side);
    return e;
  };
  // (the fork is where the segment boxes are done; the longer of the two
  // chains is handed to the device first)
  if (beside && (err = fork()) != hipSuccess)
    return err;
  const bool queries_first = beside && in.m > in.n;
  if (queries_first && (err = queries_chain()) != hipSuccess)
    return err;
  hipLaunchKernelGGL(morton_keys_kernel, dim3((in.n + kBlock - 1) / kBlock),
                     dim3(kBlock), 0, stream, x, in.ptr_x, in.n, in.d, nseg,
                     seg_box, axis_bits(nseg), keys_a, vals_a, true);
  if ((err = hipGetLastError()) != hipSuccess)
    return err;
  size_t sort_bytes = lay.sort_temp;
  if ((err = sort_pairs(sort_temp, sort_bytes, keys_a, keys_x, vals_a, perm_x,
                        in.n, nseg, stream)) != hipSuccess)
    return err;
  if (!queries_first && (!self_search || with_tasks) &&
      (err = queries_chain()) != hipSuccess)
    return err;
  {
    const int per_block = kBlock / kBinTile;
    hipLaunchKernelGGL(gather_tiles_kernel,
                       dim3((lay.tiles_bound + per_block - 1) / per_block),
                       dim3(kBlock), 0, stream, x, in.ptr_x, in.n, in.d, nseg,
                       tile_start, perm_x, plain_rows ? rows : nullptr, packed,
                       box);
    const int groups_per_block = kBlock / kWave;
    hipLaunchKernelGGL(
        group_boxes_kernel,
        dim3((lay.groups_bound + groups_per_block - 1) / groups_per_block),
        dim3(kBlock), 0, stream, nseg, tile_start, group_start, box,
        group_box);
  }
  if ((err = hipGetLastError()) != hipSuccess)
    return err;
  return rejoin.join();
}

void fill_params(BinnedParams &p, const SearchInput &in, const Bins &bins,
                 const DenseResult &out) {
  p.y = static_cast<const float *>(in.y);
  p.ptr_x = in.ptr_x;
  p.ptr_y = in.ptr_y;
  p.n = in.n;
  p.m = in.m;
  p.d = in.d;
  p.num_segments = in.num_segments;
  p.tile_start = bins.tile_start;
  p.wave_start = bins.wave_start;
  p.keys_x = bins.keys_x;
  p.keys_y = bins.keys_y;
  p.perm_y = bins.perm_y;
  p.rows = bins.rows;
  p.packed = bins.packed;
  p.box = bins.box;
  p.group_start = bins.group_start;
  p.group_box = bins.group_box;
  p.out_idx = out.idx;
  p.out_dist = out.dist;
  p.out_count = out.count;
  p.out_nearest = nullptr;
  p.task_order = bins.task_order;
  p.task_desc = bins.task_desc;
  p.task_slots = bins.task_slots;
  p.xcd_run_log2 = xcd_run_log2(bins.task_slots);
  p.code_bits = bins.code_bits;
}

} // namespace

bool knn_binned_supported(int d, int k, bool cosine) {
  return !cosine && d >= 1 && d <= 3 && k >= 1 && k <= 64;
}

size_t knn_binned_scratch_bytes(int n, int m, int num_segments) {
  return binned_layout(n, m, num_segments).total();
}

hipError_t launch_knn_binned(const SearchInput &in, int k, void *scratch,
                             const DenseResult &out, hipEvent_t time_start,
                             hipEvent_t time_stop, hipStream_t stream) {
  if (time_start)
    (void)hipEventRecord(time_start, stream);
  // (diagnostic switch: the vector-ALU scan instead of the matrix-core one)
  // (lists of more than 32 entries exist for the matrix-core scan only)
  const char *env = getenv("PCA_KNN_BINNED_MATRIX_CORES");
  const bool matrix_cores = k > 32 || !(env != nullptr && env[0] == '0');
  Bins bins;
  const hipError_t err =
      prepare_bins(in, scratch, matrix_cores, !matrix_cores, bins, stream);
  if (err != hipSuccess)
    return err;
  BinnedParams p;
  fill_params(p, in, bins, out);
  p.k = k;
  if (matrix_cores)
    p.wave_start = bins.half_start;
  const int waves = plan_upper_bound(in.m, in.num_segments, kWave);
  const int grid = (waves + kBlock / kWave - 1) / (kBlock / kWave);
  const int slots = bins.task_grid;
#define PCA_BINNED_LAUNCH(K_)                                                  \
  do {                                                                         \
    if (matrix_cores)                                                          \
      hipLaunchKernelGGL((knn_binned_mc_kernel<K_>), dim3(slots),              \
                         dim3(kBinMcBlock), 0, stream, p);                     \
    else                                                                       \
      hipLaunchKernelGGL((knn_binned_kernel<K_>), dim3(grid), dim3(kBlock), 0, \
                         stream, p);                                           \
  } while (0)
#define PCA_BINNED_LAUNCH_WIDE(K_)                                             \
  hipLaunchKernelGGL((knn_binned_mc_kernel<K_>), dim3(slots),                  \
                     dim3(kBinMcBlock), 0, stream, p)
  // (list widths in steps of 8: the bound shared by the two lanes of a query
  // reads one of the five middle entries of a list)
  if (k <= 8)
    PCA_BINNED_LAUNCH(8);
  else if (k <= 16)
    PCA_BINNED_LAUNCH(16);
  else if (k <= 24)
    PCA_BINNED_LAUNCH(24);
  else if (k <= 32)
    PCA_BINNED_LAUNCH(32);
  else if (k <= 40)
    PCA_BINNED_LAUNCH_WIDE(40);
  else if (k <= 48)
    PCA_BINNED_LAUNCH_WIDE(48);
  else if (k <= 56)
    PCA_BINNED_LAUNCH_WIDE(56);
  else
    PCA_BINNED_LAUNCH_WIDE(64);
#undef PCA_BINNED_LAUNCH_WIDE
#undef PCA_BINNED_LAUNCH
  if (time_stop)
    (void)hipEventRecord(time_stop, stream);
  return hipGetLastError();
}

hipError_t launch_nearest_binned(const SearchInput &in, void *scratch,
                                 int64_t *out, hipEvent_t time_start,
                                 hipEvent_t time_stop, hipStream_t stream) {
  if (time_start)
    (void)hipEventRecord(time_start, stream);
  Bins bins;
  const hipError_t err = prepare_bins(in, scratch, true, false, bins, stream);
  if (err != hipSuccess)
    return err;
  BinnedParams p;
  const DenseResult none{nullptr, nullptr, nullptr, 1};
  fill_params(p, in, bins, none);
  p.k = 1;
  p.out_nearest = out;
  p.wave_start = bins.half_start;
  hipLaunchKernelGGL((knn_binned_mc_kernel<1, true>), dim3(bins.task_grid),
                     dim3(kBinMcBlock), 0, stream, p);
  if (time_stop)
    (void)hipEventRecord(time_stop, stream);
  return hipGetLastError();
}

bool radius_binned_supported(int d, int slots) {
  return d >= 1 && d <= 3 && slots >= 1 && slots <= 64;
}

hipError_t launch_radius_binned(const SearchInput &in, float r2,
                                bool ignore_same_index, void *scratch,
                                const DenseResult &out, hipStream_t stream) {
  // (diagnostic switch: the vector-ALU scan instead of the matrix-core one)
  // (lists of more than 32 entries exist for the matrix-core scan only)
  const char *env = getenv("PCA_RADIUS_BINNED_MATRIX_CORES");
  const bool matrix_cores =
      out.slots > 32 || !(env != nullptr && env[0] == '0');
  Bins bins;
  const hipError_t err =
      prepare_bins(in, scratch, false, !matrix_cores, bins, stream);
  if (err != hipSuccess)
    return err;
  BinnedParams p;
  fill_params(p, in, bins, out);
  p.k = out.slots;
  const int same = ignore_same_index ? 1 : 0;
  const int per_task = matrix_cores ? kWave / 2 : kWave;
  if (matrix_cores)
    p.wave_start = bins.half_start;
  const int waves = plan_upper_bound(in.m, in.num_segments, per_task);
  const int grid = (waves + kBlock / kWave - 1) / (kBlock / kWave);
  p.xcd_run_log2 = xcd_run_log2(waves); // (tasks in curve order, no slots)
#define PCA_BINNED_LAUNCH(K_)                                                  \
  do {                                                                         \
    if (matrix_cores)                                                          \
      hipLaunchKernelGGL((radius_binned_mc_kernel<K_>),                        \
                         dim3(xcd_run_grid(waves)), dim3(kBinMcBlock), 0,   \
                         stream, p, r2, same);                                 \
    else                                                                       \
      hipLaunchKernelGGL((radius_binned_kernel<K_>), dim3(grid), dim3(kBlock), \
                         0, stream, p, r2, same);                              \
  } while (0)
#define PCA_BINNED_LAUNCH_WIDE(K_)                                             \
  hipLaunchKernelGGL((radius_binned_mc_kernel<K_>),                            \
                     dim3(xcd_run_grid(waves)), dim3(kBinMcBlock), 0,       \
                     stream, p, r2, same)
  if (out.slots <= 8)
    PCA_BINNED_LAUNCH(8);
  else if (out.slots <= 16)
    PCA_BINNED_LAUNCH(16);
  else if (out.slots <= 24)
    PCA_BINNED_LAUNCH(24);
  else if (out.slots <= 32)
    PCA_BINNED_LAUNCH(32);
  else if (out.slots <= 40)
    PCA_BINNED_LAUNCH_WIDE(40);
  else if (out.slots <= 48)
    PCA_BINNED_LAUNCH_WIDE(48);
  else if (out.slots <= 56)
    PCA_BINNED_LAUNCH_WIDE(56);
  else
    PCA_BINNED_LAUNCH_WIDE(64);
#undef PCA_BINNED_LAUNCH_WIDE
#undef PCA_BINNED_LAUNCH
  return hipGetLastError();
}

} // namespace pca
