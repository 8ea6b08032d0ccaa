// The binned kNN search (knn_binned.hip) with the scan of a tile done by the
// matrix-core pre-filter of knn_lowd_mc_impl.hpp: one
// v_mfma_f32_32x32x16_bf16 gives the signs of t - cut for the 32 rows of a
// tile against 32 queries, 16 funnel shifts per lane gather them, and only the
// flagged rows get their exact fp32 distance (from a copy of the tile's
// coordinates in LDS).  Results are those of the reference's scan
// (csrc/cuda/knn_cuda.cu:52-78) bit for bit, as for the other kernels.
//
// A wave owns 32 curve-consecutive queries: lanes l and l + 32 share query
// l % 32 (hi and lo parts of its operand) and split every tile's rows, 16
// each, with a sorted list of their own; the two lists are united at the end.
// The coordinates of the last kBinRing scanned tiles stay in a per-wave ring
// in LDS; a lane parks at most one word (ring slot, sign mask) per tile, and
// the parked rows are resolved exactly, by all lanes together, when the ring
// has gone round.  Rows are met out of row order, so every bound admits an
// equal distance (the 64-bit (distance, row) keys decide), as in the `nearest`
// mode of the scanning kernel.
#pragma once

#include "knn_lowd_mc_impl.hpp"

namespace pca {

constexpr int kBinTile = 32;  // rows per tile
constexpr int kBinGroup = 64; // tiles per group (a box of their own)
constexpr int kBinRing = 8;   // tiles whose coordinates stay in LDS
constexpr int kBinSeedTiles = 16; // most tiles scanned before the sweep

// A box: lower corner, upper corner, the smallest row number inside, a word
// of padding (32 bytes).
struct Box {
  float lo[3];
  float hi[3];
  uint32_t min_row;
  uint32_t pad;
};

struct BinnedParams {
  const float *y;
  const int64_t *ptr_x;
  const int64_t *ptr_y;
  int n, m, d, num_segments, k;
  const int *tile_start;    // first tile of every segment
  const int *wave_start;    // first wave task of every segment
  const uint32_t *keys_x;   // sorted keys of the x rows
  const uint32_t *keys_y;   // sorted keys of the queries
  const uint32_t *perm_y;   // query behind every sorted position
  const float4 *rows;       // x rows in curve order, .w = row number
  const uint4 *packed;      // the same rows as mc_pack_row<3> leaves them,
                            // the fourth coordinate word = row number
  const uint32_t *task_order; // task slots, the longest tasks first
  const int2 *task_desc;      // per slot: first query position, queries
  int task_slots;             // entries of task_order
  int xcd_run_log2;           // log2 of the tasks in a row that one XCD takes
  int code_bits;              // bits of the curve code inside a key
  const Box *box;           // of every tile
  const int *group_start;   // first group of tiles of every segment
  const Box *group_box;     // of every group
  int *out_idx;
  float *out_dist;
  int *out_count;
  int64_t *out_nearest; // the `nearest` search: [m] rows
};

// First position in [lo, hi) whose key is not below `key` (hi if none); the
// wave probes 64 positions per round.
__device__ __forceinline__ int wave_lower_bound(
    const uint32_t *__restrict__ keys, int lo, int hi, uint32_t key,
    int lane) {
  while (hi - lo > kWave) {
    const int step = (hi - lo) / kWave;
    const int probe = lo + (lane + 1) * step - 1;
    const int below = __popcll(__ballot(keys[probe] < key));
    // probes 0 .. below-1 are below the key, probe `below` (if any) is not
    const int new_lo = lo + below * step;
    if (below < kWave)
      hi = lo + (below + 1) * step - 1;
    lo = new_lo;
  }
  const int probe = lo + lane;
  const bool below = probe < hi && keys[probe] < key;
  return lo + __popcll(__ballot(below));
}

// Squared distance between two boxes (a query is a box of one point), with
// the operations of the exact chain on per-axis gaps that are not above
// |row - query| for any row and query of the boxes: never above the computed
// distance of any such pair.
__device__ __forceinline__ float box_gap2(const float (&alo)[3],
                                          const float (&ahi)[3],
                                          const float (&blo)[3],
                                          const float (&bhi)[3]) {
  float acc = 0.0f;
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    const float gap = __builtin_fmaxf(
        __builtin_fmaxf(alo[c] - bhi[c], blo[c] - ahi[c]), 0.0f);
    acc = c == 0 ? gap * gap : __builtin_fmaf(gap, gap, acc);
  }
  return acc;
}

// the set bit of `mask` nearest to position `at` (mask != 0)
__device__ __forceinline__ int nearest_bit(uint64_t mask, int at) {
  const uint64_t up = mask >> at;
  const uint64_t down = at > 0 ? mask & (~(uint64_t)0 >> (64 - at)) : 0;
  const int d_up = up ? (int)__builtin_ctzll(up) : 128;
  const int d_down = down ? at - (63 - (int)__builtin_clzll(down)) : 128;
  return d_up <= d_down ? at + d_up : at - d_down;
}

// ---- pieces shared by the matrix-core searches ------------------------------

// A lane's query: coordinates (zero beyond d and for a lane without one),
// whether it searches at all (a coordinate that is not finite has no distance
// below any limit), its squared norm, and the box around the wave's searching
// queries.
struct BinQuery {
  float y[3];
  bool searching;
  float ysq;
  float lo[3], hi[3];
};

__device__ __forceinline__ BinQuery bin_load_query(const BinnedParams &p,
                                                   bool valid, int q) {
  BinQuery r;
#pragma unroll
  for (int c = 0; c < 3; ++c)
    r.y[c] = (valid && c < p.d) ? p.y[(size_t)q * p.d + c] : 0.0f;
  r.searching = valid && __builtin_fabsf(r.y[0]) < __builtin_inff() &&
                __builtin_fabsf(r.y[1]) < __builtin_inff() &&
                __builtin_fabsf(r.y[2]) < __builtin_inff();
  r.ysq = r.y[0] * r.y[0];
#pragma unroll
  for (int c = 1; c < 3; ++c)
    r.ysq = __builtin_fmaf(r.y[c], r.y[c], r.ysq);
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    float lo = r.searching ? r.y[c] : __builtin_inff();
    float hi = r.searching ? r.y[c] : -__builtin_inff();
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1) {
      lo = __builtin_fminf(lo, __shfl_xor(lo, sh));
      hi = __builtin_fmaxf(hi, __shfl_xor(hi, sh));
    }
    r.lo[c] = lo;
    r.hi[c] = hi;
  }
  return r;
}

// B operand of the filter without the cut: the hi (lanes 0-31) or lo (lanes
// 32-63) parts of (-2 y_0, -2 y_1, -2 y_2, 1), given twice (against the hi
// and the lo parts of the row); see knn_lowd_mc_impl.hpp.  A lane that does
// not search multiplies everything by zero.
__device__ __forceinline__ uint4 bin_query_operand(const BinQuery &q,
                                                   int half) {
  const bool moderate = q.ysq <= kFilterNormLimit;
  uint32_t part[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float v = 0.0f;
    if (e < 3)
      v = (q.searching && moderate) ? -2.0f * q.y[e] : 0.0f;
    else
      v = q.searching ? 1.0f : 0.0f;
    uint32_t hi, lo;
    mc_split(v, hi, lo);
    part[e] = half ? lo : hi;
  }
  const uint32_t w0 = part[0] | (part[1] << 16);
  const uint32_t w1 = part[2] | (part[3] << 16);
  return make_uint4(w0, w1, w0, w1);
}

// ... with -cut riding in the two accumulation slots of w that the zero lo
// part of the query's 1 would leave unused (upper lanes, component 3 of the
// one instruction): -cut' split, cut' = cut + 2^-15 |cut|, so that what the
// split may lose never lowers the cut; an infinite cut (filter switched off)
// enters as the largest finite bf16.
__device__ __forceinline__ mc_bf16x8_t bin_operand_with_cut(uint4 plain,
                                                            float cut,
                                                            int half) {
  if (half) {
    float neg = -__builtin_fmaf(__builtin_fabsf(cut), 3.0517578125e-05f, cut);
    uint32_t hi, lo;
    if (__builtin_fabsf(neg) < 1e38f) {
      mc_split(neg, hi, lo);
    } else {
      hi = neg < 0.0f ? 0xff7fu : 0x7f7fu;
      lo = 0;
    }
    plain.y = (plain.y & 0x0000ffffu) | (hi << 16);
    plain.w = (plain.w & 0x0000ffffu) | (lo << 16);
  }
  return __builtin_bit_cast(mc_bf16x8_t, plain);
}

// The rows of a tile as the lanes fetch them: the operand quad of row `col`
// (both halves), the coordinate quad of row `col` (lower half).  (The packed
// copy is padded by a tile of rows that never pass.)
struct BinFetched {
  uint4 operand, coords;
};

__device__ __forceinline__ BinFetched bin_fetch(const uint4 *__restrict__ packed,
                                                int first_row, int col,
                                                int half) {
  const size_t j = (size_t)(first_row + col);
  BinFetched f;
  f.operand = packed[j * 2];
  f.coords = half ? make_uint4(0u, 0u, 0u, 0u) : packed[j * 2 + 1];
  return f;
}

// Sign mask of t - cut for the lane's 16 rows of a tile (bit 15 - v stands for
// accumulator v = row 8 (v / 4) + 4 half + v % 4): one matrix instruction and
// 16 funnel shifts.  rows < 32: the segment's last tile, whose rows past the
// end belong to the next segment and are masked out.
__device__ __forceinline__ uint32_t bin_tile_signs(uint4 operand,
                                                   mc_bf16x8_t yb, int half,
                                                   int rows) {
  // upper lanes: 1 in place of w_hi and w_lo (times the parts of -cut)
  if (half) {
    operand.y = (operand.y & 0x0000ffffu) | (0x3f80u << 16);
    operand.w = (operand.w & 0x0000ffffu) | (0x3f80u << 16);
  }
  mfma_acc_t acc = {0};
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
      __builtin_bit_cast(mc_bf16x8_t, operand), yb, acc, 0, 0, 0);
  uint32_t mask = 0;
#pragma unroll
  for (int v = 0; v < 16; ++v)
    mask = __builtin_amdgcn_alignbit(mask, __float_as_uint(acc[v]), 31);
  if (rows < kBinTile) {
    uint32_t real = 0;
#pragma unroll
    for (int v = 0; v < 16; ++v)
      real |= (8 * (v / 4) + 4 * half + v % 4 < rows) ? (1u << (15 - v)) : 0u;
    mask &= real;
  }
  return mask;
}

// Exact squared distance of a ring entry (coordinates, row number) to the
// lane's query, as the reference accumulates it.
__device__ __forceinline__ float bin_exact_distance(const uint4 &r4,
                                                    const float (&y)[3]) {
  const float d0 = __uint_as_float(r4.x) - y[0];
  float d = d0 * d0;
  const float d1 = __uint_as_float(r4.y) - y[1];
  d = __builtin_fmaf(d1, d1, d);
  const float d2 = __uint_as_float(r4.z) - y[2];
  return __builtin_fmaf(d2, d2, d);
}

// The box that lane `src` holds, broadcast to the wave.
__device__ __forceinline__ void bin_box_of_lane(const Box &held, int src,
                                                float (&lo)[3],
                                                float (&hi)[3]) {
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    lo[c] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
        (int)__float_as_uint(held.lo[c]), src));
    hi[c] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
        (int)__float_as_uint(held.hi[c]), src));
  }
}

// Tasks of the matrix-core searches.  Normally a block of 32
// curve-consecutive queries is one task (slot = block number).  A block whose
// queries span much more of the curve than the segment's average (4 times:
// measured) lies where
// the points are sparse: its queries are far apart, each with a neighbourhood
// of its own, and one wave would look at several times as many boxes and
// tiles as a wave in a dense region - the tail of the launch.  Such a block is
// split into four tasks of 8 queries: its own slot and three extra slots
// behind the blocks' ones, handed out by an atomic counter while they last
// (`extra` slots; `*extra_used` starts at 0).
//
// Starting order: the used extra slots first (parts of the longest tasks),
// then the blocks by the class of their span - three octaves to a class,
// widest first - and inside a class in curve order: the long tasks start
// early, and tasks keep their neighbours next to them, which look at the same
// tiles.  (One octave to a class orders the lengths more finely and ends no
// sooner, but neighbours along the curve then alternate between two or three
// classes, every class sweeps the whole cloud, and the search kernel of the
// 1 M-point LiDAR-like workload fetched 594 MB instead of 258 MB.)  Unused
// slots come last (their waves leave at once).  It is a counting sort in two
// launches: task_span_kernel leaves every block's class and a histogram of
// the classes per workgroup of kBlock blocks, task_order_kernel turns them
// into places.
constexpr int kTaskClasses = 64; // classes 0..11, 33 = unused block, rest empty

__device__ __forceinline__ uint32_t bin_task_class(uint32_t span) {
  return span != 0 ? (uint32_t)__builtin_clz(span) / 3u : 11u;
}

// cls: [bound] class per block; hist: [workgroups][kTaskClasses].
__global__ __launch_bounds__(kBlock) void task_span_kernel(
    BinnedParams p, int bound, int extra, int *__restrict__ extra_used,
    int2 *__restrict__ desc, uint32_t *__restrict__ cls,
    int *__restrict__ hist) {
  __shared__ int count_of[kTaskClasses];
  if (threadIdx.x < kTaskClasses)
    count_of[threadIdx.x] = 0;
  __syncthreads();
  const int block = blockIdx.x * kBlock + threadIdx.x;
  if (block < bound) {
    int2 mine = make_int2(0, 0);
    uint32_t mine_class = 33u;
    if (block < p.wave_start[p.num_segments]) {
      const int seg = find_segment(p.wave_start, p.num_segments, block);
      const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
      const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
      const int jq0 = y_begin + (block - p.wave_start[seg]) * 32;
      const int count = min(32, y_end - jq0);
      const uint32_t span = p.keys_y[jq0 + count - 1] - p.keys_y[jq0];
      const int blocks = p.wave_start[seg + 1] - p.wave_start[seg];
      const uint64_t average = ((uint64_t)1 << p.code_bits) / (uint64_t)blocks;
      mine = make_int2(jq0, count);
      mine_class = bin_task_class(span);
      if (count == 32 && (uint64_t)span > 4 * average) {
        const int at = atomicAdd(extra_used, 3);
        if (at + 3 <= extra) {
          mine = make_int2(jq0, 8);
          mine_class = bin_task_class(span / 4);
          for (int i = 0; i < 3; ++i)
            desc[bound + at + i] = make_int2(jq0 + 8 * (i + 1), 8);
        }
      }
    }
    desc[block] = mine;
    cls[block] = mine_class;
    atomicAdd(&count_of[mine_class], 1);
  }
  __syncthreads();
  if (threadIdx.x < kTaskClasses)
    hist[blockIdx.x * kTaskClasses + threadIdx.x] = count_of[threadIdx.x];
}

// Same grid as task_span_kernel.  order: [bound + extra] slot numbers.
__global__ __launch_bounds__(kBlock) void task_order_kernel(
    int bound, int extra, const int *__restrict__ extra_used,
    const uint32_t *__restrict__ cls, const int *__restrict__ hist,
    uint32_t *__restrict__ order) {
  constexpr int kParts = kBlock / kTaskClasses;
  constexpr int kWaves = kBlock / kWave;
  __shared__ int before_part[kParts][kTaskClasses];
  __shared__ int total_part[kParts][kTaskClasses];
  __shared__ int base[kTaskClasses];
  __shared__ int wave_count[kWaves][kTaskClasses];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int used = min(*extra_used, extra);

  // the extra slots: used ones first, the others behind everything
  for (int i = blockIdx.x * kBlock + tid; i < extra; i += gridDim.x * kBlock)
    order[i < used ? i : bound + i] = (uint32_t)(bound + i);

  // blocks of every class in the workgroups before this one, and in all
  {
    const int c = tid & (kTaskClasses - 1);
    const int part = tid / kTaskClasses;
    int before = 0, total = 0;
    for (int g = part; g < (int)gridDim.x; g += kParts) {
      const int v = hist[g * kTaskClasses + c];
      total += v;
      before += g < (int)blockIdx.x ? v : 0;
    }
    before_part[part][c] = before;
    total_part[part][c] = total;
    wave_count[tid / kTaskClasses][c] = 0; // (kParts == kWaves)
  }
  static_assert(kParts == kWaves, "one zeroing pass covers wave_count");
  __syncthreads();
  if (tid == 0) {
    int run = used;
    for (int c = 0; c < kTaskClasses; ++c) {
      int before = 0, total = 0;
      for (int part = 0; part < kParts; ++part) {
        before += before_part[part][c];
        total += total_part[part][c];
      }
      base[c] = run + before;
      run += total;
    }
  }
  // place inside the wave among the blocks of the same class
  const int block = blockIdx.x * kBlock + tid;
  const bool valid = block < bound;
  const int mine = valid ? (int)cls[block] : -1;
  int rank = 0;
  uint64_t todo = __ballot(valid);
  while (todo != 0) {
    const int leader = __builtin_ctzll(todo);
    const int c = __shfl(mine, leader);
    const uint64_t same = __ballot(mine == c);
    if (mine == c)
      rank = __builtin_popcountll(same & (((uint64_t)1 << lane) - 1));
    if (lane == leader)
      wave_count[wave][c] = __builtin_popcountll(same);
    todo &= ~same;
  }
  __syncthreads();
  if (valid) {
    int at = base[mine] + rank;
    for (int w = 0; w < wave; ++w)
      at += wave_count[w][mine];
    order[at] = (uint32_t)block;
  }
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: runs
// of 2^run_log2 consecutive tasks (neighbours along the curve, which fetch the
// same tiles) go to the same XCD, one after the other.  Maps a workgroup
// number to its task's place in the order; grids are whole multiples of
// 8 << run_log2.
__device__ __forceinline__ int bin_xcd_run(int workgroup, int run_log2) {
  const int local = workgroup >> 3;
  return ((((local >> run_log2) << 3) + (workgroup & 7)) << run_log2) |
         (local & ((1 << run_log2) - 1));
}

// Waves work on their own (no barrier): a workgroup is one wave, so that its
// place on the SIMD frees up the moment it is done - the tasks differ a lot in
// length.
constexpr int kBinMcBlock = kWave;

// p.wave_start counts blocks of 32 queries, p.task_desc / p.task_order are
// task_span_kernel's.  NEAREST: the search of the
// `nearest` operator - one neighbour, limit 1e38, the reference's order among
// equal distances (device_utils.hpp) - whose result goes to p.out_nearest as
// a row number (0 when nothing qualified).
template <int K, bool NEAREST = false>
__global__ __launch_bounds__(kBinMcBlock, K <= 8 ? 5 : (K <= 16 ? 4 : (K <= 32 ? 3 : 2))) void
knn_binned_mc_kernel(BinnedParams p) {
  static_assert(!NEAREST || K == 1, "nearest keeps one neighbour");
  constexpr int DIM = 3;
  constexpr int REC = McShape<DIM>::REC; // operand quad, coordinate quad
  static_assert(McShape<DIM>::NI == 1 && REC == 2, "one instruction per tile");
  constexpr float kLimit = SearchLimit<NEAREST>::value;
  constexpr int kWaves = kBinMcBlock / kWave;

  // coordinates and row numbers of the last kBinRing tiles of every wave
  __shared__ __attribute__((aligned(16))) uint4 ring[kWaves][kBinRing][kBinTile];
  // parked words: (ring slot << 16) | mask of the lane's 16 rows that passed
  __shared__ uint32_t queue[kBinRing][kBinMcBlock];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int half = lane >> 5;
  const int col = lane & 31;
  const int ordered = bin_xcd_run((int)blockIdx.x, p.xcd_run_log2);
  if (ordered >= p.task_slots)
    return; // (the grid is rounded up to whole runs)
  const int slot = (int)p.task_order[ordered];
  const int2 task = p.task_desc[slot]; // (first query position, queries)
  if (task.y == 0)
    return; // (an unused slot; whole waves leave, no barrier below)
  // (the segment of the task's first query)
  int seg = 0;
  if (p.ptr_y) {
    int lo = 0, hi = p.num_segments;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (p.ptr_y[mid] <= task.x)
        lo = mid;
      else
        hi = mid;
    }
    seg = lo;
  }
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int jq0 = task.x;
  const int jq = jq0 + col;
  const bool valid = col < task.y;
  const int q = valid ? (int)p.perm_y[jq] : 0;
  const int k = p.k;

  const BinQuery me = bin_load_query(p, valid, q);
  const float (&yq)[3] = me.y;
  const float (&q_lo)[3] = me.lo;
  const float (&q_hi)[3] = me.hi;
  const bool searching = me.searching;
  const float ysq = me.ysq;
  const uint4 yb_plain = bin_query_operand(me, half);

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - k) ? lowest_key() : SearchLimit<NEAREST>::empty();
  // exact distances must be strictly below thresh: the limit, or just above
  // the smaller of this lane's and the query's k-th distance (equality still
  // passes); a lane that does not search accepts nothing
  const float ysq_damped = mc_damped_norm(ysq);
  float thresh = searching ? kLimit : -__builtin_inff();
  float cut = searching ? mc_filter_cut(thresh, ysq_damped) : -1e38f;
  float shared = kLimit; // bound learnt from the partner lane
  mc_bf16x8_t yb = bin_operand_with_cut(yb_plain, cut, half);
  auto refresh_cut = [&]() __attribute__((always_inline)) { yb = bin_operand_with_cut(yb_plain, cut, half); };
  auto set_thresh = [&](float v) __attribute__((always_inline)) {
    if (searching) {
      thresh = v;
      cut = mc_filter_cut(v, ysq_damped);
    }
  };

  int qn = 0; // parked words of this lane

  // What the two lanes of a query tell each other about its final k-th
  // distance (see knn_lowd_mc_impl.hpp; equality admitted).
  // this lane's ceil(k/2)-th smallest distance so far (kLimit for k = 1)
  auto own_mid = [&]() __attribute__((always_inline)) {
    float mid = kLimit;
    if (K >= 2) {
      const int c = k >> 1;
#pragma unroll
      for (int cc = (K >= 8 ? K / 2 - 4 : 0); cc <= K / 2; ++cc)
        if (cc >= 1 && cc == c) {
          asm volatile(""); // (keeps this a branch)
          mid = key_dist(best[K - 1 - cc]);
        }
    }
    return mid;
  };
  auto partner_bounds = [&]() __attribute__((always_inline)) {
    const float own = key_dist(best[K - 1]);
    const auto both = __builtin_amdgcn_permlane32_swap(
        __float_as_uint(own), __float_as_uint(own), false, false);
    float partner = __uint_as_float(half ? both[0] : both[1]);
    if (K >= 2) {
      const float mid = own_mid();
      const auto mids = __builtin_amdgcn_permlane32_swap(
          __float_as_uint(mid), __float_as_uint(mid), false, false);
      const float partner_mid = __uint_as_float(half ? mids[0] : mids[1]);
      partner = __builtin_fminf(partner, __builtin_fmaxf(mid, partner_mid));
    }
    if (searching && partner < kLimit) {
      shared = __builtin_fminf(shared, next_up_positive(partner));
      if (shared < thresh)
        set_thresh(shared);
    }
  };

  // Resolves the parked rows exactly: in every round each lane takes the next
  // row of its parked words and all lanes evaluate theirs together.
  auto drain = [&]() __attribute__((always_inline)) {
    bool changed = false; // wave-uniform
    int taken = 0;
    uint32_t pending = 0;
    int slot_base = 0;
    for (;;) {
      if (pending == 0 && taken < qn) {
        const uint32_t word = queue[taken][tid];
        ++taken;
        pending = word & 0xffffu;
        slot_base = (int)(word >> 16) * kBinTile + 4 * half;
      }
      const bool has = pending != 0;
      if (!__any(has))
        break;
      // bit 15 - v of the mask stands for accumulator v = row
      // 8 (v / 4) + 4 half + v % 4 of the tile
      const int bit = 31 - __builtin_clz(has ? pending : 1u);
      const int v = 15 - bit;
      pending &= ~(1u << bit);
      const int j = has ? slot_base + 2 * (v & 12) + (v & 3) : 0;
      const uint4 r4 = (&ring[wave][0][0])[j];
      const float d = bin_exact_distance(r4, yq);
      const bool ok = has && d < thresh;
      if (!__any(ok))
        continue;
      const uint32_t row_id =
          NEAREST ? nearest_tie(r4.w - (uint32_t)x_begin) : r4.w;
      const double key =
          ok ? make_key(d, row_id) : SearchLimit<NEAREST>::empty();
      sorted_insert<K>(best, key);
      float own_bound = key_dist(best[K - 1]);
      // (a row of EQUAL distance and smaller number can still get in)
      if (own_bound < kLimit)
        own_bound = next_up_positive(own_bound);
      // (the filter's cut follows once, after the last round)
      if (searching)
        thresh = __builtin_fminf(own_bound, shared);
      changed = true;
    }
    qn = 0;
    if (!changed)
      return;
    set_thresh(thresh);
    partner_bounds();
    refresh_cut();
  };

  // largest bound among the wave's queries
  auto wave_reach = [&]() __attribute__((always_inline)) {
    float r = searching ? thresh : -1.0f;
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1)
      r = __builtin_fmaxf(r, __shfl_xor(r, sh));
    return r;
  };

  const int tile0 = p.tile_start[seg];
  const int num_tiles = p.tile_start[seg + 1] - tile0;
  int scanned = 0; // tiles since the start: slot = scanned % kBinRing

  typedef BinFetched Fetched;
  auto fetch = [&](int tile) __attribute__((always_inline)) {
    return bin_fetch(p.packed, x_begin + tile * kBinTile, col, half);
  };
  auto scan = [&](int tile, const Fetched &f) __attribute__((always_inline)) {
    const int slot = scanned % kBinRing;
    if (!half)
      ring[wave][slot][col] = f.coords;
    const int rows = min(kBinTile, x_end - (x_begin + tile * kBinTile));
    const uint32_t mask = bin_tile_signs(f.operand, yb, half, rows);
    if (mask != 0) {
      queue[qn][tid] = ((uint32_t)slot << 16) | mask;
      ++qn;
    }
    ++scanned;
    // every kBinRing tiles, and after the first, second and fourth tile of
    // the task: until the lists are full every row passes the filter, and
    // with a first bound after 32 rows instead of 256 the filter passes half
    // as many rows of the seed tiles (the insertions, which dominate, stay:
    // the same time on LiDAR-like clouds, 3 % less on uniform ones)
    if (scanned % kBinRing == 0 ||
        (scanned < kBinRing && (scanned & (scanned - 1)) == 0))
      drain();
  };

  if (num_tiles > 0) {
    // where the wave's first and last query fall in the order of x
    const int last_col = task.y - 1;
    const uint32_t key_first = p.keys_y[jq0];
    const uint32_t key_last = p.keys_y[jq0 + last_col];
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
      const int mid = (seed_lo + seed_hi) / 2;
      seed_lo = max(0, mid - kBinSeedTiles / 2);
      seed_hi = min(num_tiles - 1, seed_lo + kBinSeedTiles - 1);
    }
    {
      Fetched next = fetch(seed_lo);
      for (int t = seed_lo; t <= seed_hi; ++t) {
        const Fetched cur = next;
        if (t < seed_hi)
          next = fetch(t + 1);
        scan(t, cur);
      }
    }
    drain();
    float reach = wave_reach();

    // is the box of lane `src` within reach of some lane's query?  (A NaN -
    // from an infinite or empty box - never rules a box out.)
    auto reachable = [&](const Box &held, int src) __attribute__((always_inline)) {
      float lo[3], hi[3];
      bin_box_of_lane(held, src, lo, hi);
      return __any(searching && !(box_gap2(lo, hi, yq, yq) >= thresh));
    };
    // the same for the boxes of lanes `a` (tested by lanes 0-31) and `b`
    // (lanes 32-63) at once: the ballot of the lanes whose query reaches
    auto reachable_pair = [&](const Box &held, int a, int b) __attribute__((always_inline)) {
      const int src = half ? b : a;
      float lo[3], hi[3];
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        lo[c] = __shfl(held.lo[c], src);
        hi[c] = __shfl(held.hi[c], src);
      }
      return __ballot(searching && !(box_gap2(lo, hi, yq, yq) >= thresh));
    };

    // Groups of tiles, 64 at a time (one box per lane), nearest to the seed
    // tiles first; a group, then a tile, is looked into if its box is within
    // the wave's largest bound of the box around the wave's queries, and then
    // within some query's own bound of that query.
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
                   !(box_gap2(g_box.lo, g_box.hi, q_lo, q_hi) >= reach));
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
            t_ok && !(box_gap2(t_box.lo, t_box.hi, q_lo, q_hi) >= reach));
        // the tiles of the group that some query can reach, by its bound of
        // now; their rows are fetched one tile ahead of the scan
        uint64_t t_pass = 0;
        while (t_todo != 0) {
          // two boxes per step: the two halves of the wave hold the same 32
          // queries, so the lower half tests one box and the upper half the
          // next (a lone last box is tested by both)
          const int t_a = (int)__builtin_ctzll(t_todo);
          t_todo &= t_todo - 1;
          const int t_b = t_todo != 0 ? (int)__builtin_ctzll(t_todo) : t_a;
          t_todo &= t_todo - 1;
          const uint64_t both = reachable_pair(t_box, t_a, t_b);
          if (both & 0xffffffffull)
            t_pass |= (uint64_t)1 << t_a;
          if (both >> 32)
            t_pass |= (uint64_t)1 << t_b;
        }
        if (t_pass != 0) {
          Fetched next = fetch(group * kBinGroup + (int)__builtin_ctzll(t_pass));
          while (t_pass != 0) {
            const int t_lane = (int)__builtin_ctzll(t_pass);
            t_pass &= t_pass - 1;
            const Fetched cur = next;
            if (t_pass != 0)
              next =
                  fetch(group * kBinGroup + (int)__builtin_ctzll(t_pass));
            scan(group * kBinGroup + t_lane, cur);
          }
          if (__any(qn > 0)) {
            drain();
            reach = wave_reach();
          }
        }
      }
    }
    drain();
  }

  unite_halves<K>(best, k, half);
  if (half == 0 && valid) {
    if constexpr (NEAREST)
      write_nearest(best[0], q, x_begin, p.out_nearest);
    else
      write_dense<K>(best, k, q, p.out_idx, p.out_dist, p.out_count);
  }
}

// The binned radius search with the same scan (reference: radius_kernel,
// csrc/cuda/radius_cuda.cu:9-42): every row with a squared distance strictly
// below r2, at most `slots` (= p.k) of them - the ones with the smallest row
// numbers, ascending.  The bound of the filter is fixed (r2), so the query
// operand is built once and there are no seed tiles; flagged rows get their
// exact distance from the ring, and those in range whose number is below the
// largest one of a full list go into the list (row numbers as doubles).
// p.wave_start counts tasks of 32 queries.
template <int K>
__global__ __launch_bounds__(kBinMcBlock, K <= 8 ? 5 : (K <= 16 ? 4 : (K <= 32 ? 3 : 2))) void
radius_binned_mc_kernel(BinnedParams p, float r2, int ignore_same_index) {
  __shared__ __attribute__((aligned(16))) uint4 ring[kBinRing][kBinTile];
  __shared__ uint32_t queue[kBinRing][kBinMcBlock];

  const int lane = threadIdx.x & (kWave - 1);
  const int tid = lane;
  const int half = lane >> 5;
  const int col = lane & 31;
  const int task = bin_xcd_run((int)blockIdx.x, p.xcd_run_log2);
  if (task >= p.wave_start[p.num_segments])
    return; // (also the padding of the grid to whole runs)
  const int seg = find_segment(p.wave_start, p.num_segments, task);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int jq = y_begin + (task - p.wave_start[seg]) * 32 + col;
  const bool valid = jq < y_end;
  const int q = valid ? (int)p.perm_y[jq] : 0;
  const int slots = p.k;

  const BinQuery me = bin_load_query(p, valid, q);
  const float (&yq)[3] = me.y;
  const float (&q_lo)[3] = me.lo;
  const float (&q_hi)[3] = me.hi;
  const bool searching = me.searching;
  // the query operand with -cut for the fixed bound r2 in place; a lane that
  // does not search passes nothing
  const mc_bf16x8_t yb = bin_operand_with_cut(
      bin_query_operand(me, half),
      searching ? mc_filter_cut(r2, mc_damped_norm(me.ysq)) : -1e38f, half);

  double best[K];
#pragma unroll
  for (int j = 0; j < K; ++j)
    best[j] = (j < K - slots) ? -__builtin_inf() : __builtin_inf();
  // rows with a number below `below` can still get in: all while neither of
  // the query's two lists is full, those under the smaller of their largest
  // numbers afterwards
  uint32_t below = searching ? 0xffffffffu : 0u;
  const uint32_t self = ignore_same_index ? (uint32_t)q : 0xffffffffu;
  const float limit = searching ? r2 : -__builtin_inff();
  int qn = 0;
  int scanned = 0;

  auto drain = [&]() __attribute__((always_inline)) {
    bool changed = false;
    int taken = 0;
    uint32_t pending = 0;
    int slot_base = 0;
    for (;;) {
      if (pending == 0 && taken < qn) {
        const uint32_t word = queue[taken][tid];
        ++taken;
        pending = word & 0xffffu;
        slot_base = (int)(word >> 16) * kBinTile + 4 * half;
      }
      const bool has = pending != 0;
      if (!__any(has))
        break;
      const int bit = 31 - __builtin_clz(has ? pending : 1u);
      const int v = 15 - bit;
      pending &= ~(1u << bit);
      const int j = has ? slot_base + 2 * (v & 12) + (v & 3) : 0;
      const uint4 r4 = (&ring[0][0])[j];
      const float d = bin_exact_distance(r4, yq);
      const bool ok = has && d < limit && r4.w < below && r4.w != self;
      if (!__any(ok))
        continue;
      sorted_insert<K>(best, ok ? (double)r4.w : __builtin_inf());
      if (searching && best[K - 1] < __builtin_inf())
        below = min(below, (uint32_t)best[K - 1]);
      changed = true;
    }
    qn = 0;
    if (!changed)
      return;
    // the partner's list bounds the query's final largest number as well
    const auto both = __builtin_amdgcn_permlane32_swap(below, below, false,
                                                       false);
    below = min(below, half ? both[0] : both[1]);
  };

  typedef BinFetched Fetched;
  auto fetch = [&](int tile) __attribute__((always_inline)) {
    return bin_fetch(p.packed, x_begin + tile * kBinTile, col, half);
  };
  auto scan = [&](int tile, const Fetched &f) __attribute__((always_inline)) {
    const int slot = scanned % kBinRing;
    if (!half)
      ring[slot][col] = f.coords;
    const int rows = min(kBinTile, x_end - (x_begin + tile * kBinTile));
    const uint32_t mask = bin_tile_signs(f.operand, yb, half, rows);
    if (mask != 0) {
      queue[qn][tid] = ((uint32_t)slot << 16) | mask;
      ++qn;
    }
    ++scanned;
    if (scanned % kBinRing == 0)
      drain();
  };

  // is the box of lane `src` closer than the radius to the query of some
  // lane that could still use one of its rows (a full list takes only smaller
  // row numbers than it holds)?  (A NaN - from an infinite or empty box -
  // never rules a box out.)
  auto reachable = [&](const Box &held, int src) __attribute__((always_inline)) {
    float lo[3], hi[3];
    bin_box_of_lane(held, src, lo, hi);
    const uint32_t min_row =
        (uint32_t)__builtin_amdgcn_readlane((int)held.min_row, src);
    return __any(searching && min_row < below &&
                 !(box_gap2(lo, hi, yq, yq) >= r2));
  };
  // largest row number any of the wave's queries could still take
  auto wave_below = [&]() __attribute__((always_inline)) {
    uint32_t b = below;
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1)
      b = max(b, (uint32_t)__shfl_xor((int)b, sh));
    return b;
  };

  const int tile0 = p.tile_start[seg];
  const int num_tiles = p.tile_start[seg + 1] - tile0;
  const int group0 = p.group_start[seg];
  const int num_groups = (num_tiles + kBinGroup - 1) / kBinGroup;
  uint32_t any_below = 0xffffffffu;
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
            __ballot(t_mine < num_tiles && t_box.min_row < any_below &&
                     !(box_gap2(t_box.lo, t_box.hi, q_lo, q_hi) >= r2));
        uint64_t t_pass = 0;
        while (t_todo != 0) {
          const int t_lane = (int)__builtin_ctzll(t_todo);
          t_todo &= t_todo - 1;
          if (reachable(t_box, t_lane))
            t_pass |= (uint64_t)1 << t_lane;
        }
        if (t_pass != 0) {
          Fetched next = fetch(group * kBinGroup + (int)__builtin_ctzll(t_pass));
          while (t_pass != 0) {
            const int t_lane = (int)__builtin_ctzll(t_pass);
            t_pass &= t_pass - 1;
            const Fetched cur = next;
            if (t_pass != 0)
              next =
                  fetch(group * kBinGroup + (int)__builtin_ctzll(t_pass));
            scan(group * kBinGroup + t_lane, cur);
          }
          if (__any(qn > 0))
            drain();
          any_below = wave_below();
        }
      }
    }
    drain();
  }

  unite_halves<K>(best, slots, half);
  if (half == 0 && valid) {
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

} // namespace pca
