// Fixed-radius neighbour search for low-dimensional fp32 points (d <= 8) with
// the candidate filter on the gfx950 matrix cores.
//
// Computes what radius_kernel of the reference computes
// (csrc/cuda/radius_cuda.cu:9-42: one thread per query scans its segment of x
// in ascending row order, keeps the first max_num_neighbors rows with
// dist < r^2, stops as soon as it has them) -- same rows, same order.
//
// The machinery is that of knn_lowd_mc_impl.hpp with a threshold that never
// moves: t - cut = w - 2 x.y - cut, cut = r^2 (1 + eps) - fl(|y|^2) (1 - eps),
// comes out of one v_mfma_f32_32x32x16_bf16 per 32 rows x 32 queries
// (split-bf16 operands, -cut in the two spare accumulation slots), the sign
// bits of a lane's 16 results are gathered with funnel shifts, and a lane with
// a non-zero mask parks (step, mask) in its LDS queue.  A candidate with an
// exact distance below r^2 always has its sign bit set (error budget in
// knn_lowd_mc_impl.hpp); whether a row with the bit set IS a neighbour is
// decided by the exact distance (direct differences, one FMA per component in
// ascending order) taken from the fp32 coordinates in the LDS tile.
//
// Lanes l and l + 32 share a query and see interleaved groups of four rows.
// When a queue fills up or the tile ends, the lower lane of each pair walks
// the parked rows of BOTH lanes in ascending row order and appends the
// neighbours to the query's slot row until it holds max_num_neighbors.  A
// query that is full stops parking; a wave whose queries are all full skips
// the matrix-core work, a workgroup whose waves are all done leaves the scan.
//
// A workgroup owns 128 queries of one segment and scans the whole segment
// (rows must be reported in order, so the segment is not sliced).
#pragma once

#include "knn_lowd_mc_impl.hpp"

namespace pca {

struct RadiusMcParams {
  const float *y;
  const int64_t *ptr_x;
  const int64_t *ptr_y;
  const uint4 *x_split; // packed rows of x (mc_pack_rows_kernel)
  int n, m, d_in, num_segments;
  float r2;
  int slots;
  int ignore_same_index;
  const int *work_start; // [num_segments + 1] first 128-query tile per segment
  int *out_idx;          // [m, slots]
  int *out_count;        // [m]
  // for the compaction (DenseResult::edge_sums; NULL: not asked for):
  // neighbours found per kCompactBlockQueries queries
  unsigned long long *edge_sums = nullptr;
};

template <int DIM>
__global__ __launch_bounds__(kBlock) void radius_mc_kernel(RadiusMcParams p) {
  constexpr int NI = McShape<DIM>::NI;
  constexpr int XF = McShape<DIM>::XF;
  constexpr int REC = McShape<DIM>::REC;
  constexpr int TX = McShape<DIM>::TX;
  constexpr int TQ = kMcQueries;
  constexpr int QCAP = kMcQueueCap;
  constexpr int PT = TX / kBlock; // rows staged per thread

  // (every 16-byte unit of a row in a plane of its own, as in
  // knn_lowd_mc_impl.hpp: conflict-free reads)
  __shared__ __attribute__((aligned(16))) uint4 rows_lds[REC][TX];
  // parked steps: (step << 16) | mask of the lane's 16 rows that passed
  // (also carries, between the two barriers at the top of a tile, the four
  // waves' "all my queries are full" flags: one more variable would take the
  // workgroup past 40,960 bytes, the most that lets four of them share a CU)
  __shared__ uint32_t queue[QCAP][kBlock];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int half = lane >> 5;
  const int col = lane & 31;

  const int total_tiles = p.work_start[p.num_segments];
  const int tile = blockIdx.x;
  if (tile >= total_tiles)
    return;
  const int seg = find_segment(p.work_start, p.num_segments, tile);
  const int x_begin = p.ptr_x ? (int)p.ptr_x[seg] : 0;
  const int x_end = p.ptr_x ? (int)p.ptr_x[seg + 1] : p.n;
  const int y_begin = p.ptr_y ? (int)p.ptr_y[seg] : 0;
  const int y_end = p.ptr_y ? (int)p.ptr_y[seg + 1] : p.m;
  const int q = y_begin + (tile - p.work_start[seg]) * TQ + wave * 32 + col;
  const bool valid = q < y_end;
  const int d_in = p.d_in;
  const int slots = p.slots;
  const float r2 = p.r2;
  const int c_count = x_end - x_begin;
  const int num_tiles = (c_count + TX - 1) / TX;

  // ---- per-lane query state ---------------------------------------------
  float yq[DIM];
#pragma unroll
  for (int c = 0; c < DIM; ++c)
    yq[c] = (valid && c < d_in) ? p.y[(size_t)q * d_in + c] : 0.0f;
  float ysq = yq[0] * yq[0];
#pragma unroll
  for (int c = 1; c < DIM; ++c)
    ysq = __builtin_fmaf(yq[c], yq[c], ysq);
  const bool y_moderate = ysq <= kFilterNormLimit;
  // B operands as in knn_lowd_mc_kernel: the hi (lanes 0-31) or lo (lanes
  // 32-63) parts of (-2 y, 1, 0 ...), the upper lanes with the parts of -cut'
  // where the lo part of the 1 would be
  constexpr int WI = DIM / 4;
  constexpr int WE = DIM % 4;
  mc_bf16x8_t yb[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    uint32_t part[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int c = 4 * i + e;
      float v = 0.0f;
      if (c < DIM)
        v = (valid && y_moderate) ? -2.0f * yq[c] : 0.0f;
      else if (c == DIM)
        v = valid ? 1.0f : 0.0f;
      uint32_t hi, lo;
      mc_split(v, hi, lo);
      part[e] = half ? lo : hi;
    }
    uint32_t w0 = part[0] | (part[1] << 16);
    uint32_t w1 = part[2] | (part[3] << 16);
    uint32_t w2 = w0, w3 = w1;
    if (i == WI && half) {
      // a lane without a query never passes: start from +1e38
      const float cut =
          valid ? mc_filter_cut(r2, mc_damped_norm(ysq)) : -1e38f;
      float neg = -__builtin_fmaf(__builtin_fabsf(cut), 3.0517578125e-05f, cut);
      uint32_t hi, lo;
      if (__builtin_fabsf(neg) < 1e38f) {
        mc_split(neg, hi, lo);
      } else {
        hi = neg < 0.0f ? 0xff7fu : 0x7f7fu;
        lo = 0;
      }
      const uint32_t keep = ~(0xffffu << (16 * (WE & 1)));
      const uint32_t sh = 16 * (WE & 1);
      if (WE < 2) {
        w0 = (w0 & keep) | (hi << sh);
        w2 = (w2 & keep) | (lo << sh);
      } else {
        w1 = (w1 & keep) | (hi << sh);
        w3 = (w3 & keep) | (lo << sh);
      }
    }
    yb[i] = __builtin_bit_cast(mc_bf16x8_t, make_uint4(w0, w1, w2, w3));
  }
  const uint32_t one_keep =
      half ? ~(0xffffu << (16 * (WE & 1))) : 0xffffffffu;
  const uint32_t one_bits = half ? (0x3f80u << (16 * (WE & 1))) : 0u;

  // neighbours found so far (kept by the lower lane of a pair, mirrored to
  // the upper one after every drain); a query without a slot left is done
  int count = 0;
  bool done = !valid || slots <= 0;
  int qn = 0; // parked steps of this lane: queue[0 .. qn)[tid]

  // ---- tile staging -------------------------------------------------------
  uint4 stage[PT][REC];
  auto pad_quad = [](int i) {
    uint4 o = make_uint4(0u, 0u, 0u, 0u);
    if (i == DIM / 4) {
      const uint32_t nan_bits = 0x7fc0u << (16 * (DIM % 2));
      if (DIM % 4 < 2)
        o.x = nan_bits;
      else
        o.y = nan_bits;
    }
    return o;
  };
  auto load_tile = [&](int t) {
#pragma unroll
    for (int r = 0; r < PT; ++r) {
      const int pos = t * TX + r * kBlock + tid;
      const size_t g = (size_t)x_begin + pos;
      const bool ok = pos < c_count;
#pragma unroll
      for (int i = 0; i < REC; ++i)
        stage[r][i] = ok ? p.x_split[g * REC + i] : pad_quad(i);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int r = 0; r < PT; ++r)
#pragma unroll
      for (int i = 0; i < REC; ++i)
        rows_lds[i][r * kBlock + tid] = stage[r][i];
  };

  // One lane's walk over parked rows (see knn_lowd_mc_kernel): peek returns
  // the next row of queue column `column` (position in the tile) or a large
  // number if none is left.
  struct Walk {
    int taken;
    uint32_t pending;
    int base;
  };
  auto peek = [&](Walk &w, int column, int entries, int row0) {
    if (w.pending == 0 && w.taken < entries) {
      const uint32_t word = queue[w.taken][column];
      ++w.taken;
      w.pending = word & 0xffffu;
      w.base = (int)(word >> 16) * 32 + row0;
    }
    if (w.pending == 0)
      return 1 << 30;
    const int bit = 31 - __builtin_clz(w.pending);
    const int v = 15 - bit;
    return w.base + 2 * (v & 12) + (v & 3);
  };
  auto pop = [&](Walk &w) { // (only after a successful peek)
    const int bit = 31 - __builtin_clz(w.pending);
    w.pending &= ~(1u << bit);
  };

  // Resolves the parked rows of the tile: the lower lane of every pair takes
  // the rows of both lanes in ascending order.
  auto drain = [&](int g_base, int rows) {
    const auto both = __builtin_amdgcn_permlane32_swap((unsigned)qn,
                                                       (unsigned)qn, false,
                                                       false);
    const int qn_upper = (int)both[1]; // of lane l + 32 (for the lower lanes)
    Walk lo{0, 0u, 0}, hi{0, 0u, 0};
    const bool worker = half == 0 && !done;
    for (;;) {
      int j = 1 << 30;
      if (worker) {
        const int a = peek(lo, tid, qn, 0);
        const int b = peek(hi, tid + 32, qn_upper, 4);
        j = min(a, b);
        if (j < (1 << 30)) {
          if (a <= b)
            pop(lo);
          else
            pop(hi);
        }
      }
      const bool has = j < rows; // (also drops padding rows)
      if (!__any(j < (1 << 30)))
        break;
      if (has && count < slots) {
        float row[XF];
#pragma unroll
        for (int e = 0; e < XF; e += 4) {
          const uint4 q4 = rows_lds[NI + e / 4][j];
          row[e] = __uint_as_float(q4.x);
          row[e + 1] = __uint_as_float(q4.y);
          row[e + 2] = __uint_as_float(q4.z);
          row[e + 3] = __uint_as_float(q4.w);
        }
        const float d0 = row[0] - yq[0];
        float dist = d0 * d0;
#pragma unroll
        for (int c = 1; c < DIM; ++c) {
          const float dc = row[c] - yq[c];
          dist = __builtin_fmaf(dc, dc, dist);
        }
        const int g = g_base + j;
        if (dist < r2 && !(p.ignore_same_index && g == q)) {
          p.out_idx[(size_t)q * slots + count] = g;
          ++count;
        }
      }
    }
    qn = 0;
    // the upper lane learns whether the query still has room
    const bool full = count >= slots;
    const auto f = __builtin_amdgcn_permlane32_swap((unsigned)full,
                                                    (unsigned)full, false,
                                                    false);
    if (f[0]) // the lower lane's verdict, for both lanes
      done = true;
  };

  if (num_tiles > 0)
    load_tile(0);
  bool wave_done = false;

  for (int t = 0; t < num_tiles; ++t) {
    // one LDS buffer: the next tile waits in registers while this one is
    // scanned
    // (no lane has anything parked here)
    if (lane == 0)
      queue[0][wave * kWave] = wave_done ? 1u : 0u;
    __syncthreads();
    bool all_done = true;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w)
      all_done = all_done && queue[0][w * kWave] != 0;
    if (all_done)
      break; // (read between two barriers: the same for every thread)
    store_tile();
    __syncthreads();
    if (t + 1 < num_tiles)
      load_tile(t + 1);
    if (wave_done)
      continue;
    const int g_base = x_begin + t * TX;
    const int rows = min(TX, c_count - t * TX);
    const int steps32 = (rows + 31) / 32;

    uint4 a_next[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i)
      a_next[i] = rows_lds[i][col];
    for (int rt = 0; rt < steps32; ++rt) {
      mfma_acc_t acc = {0};
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        uint4 a = a_next[i];
        if (i == WI) {
          // upper lanes: 1 in place of w_hi and w_lo (times -cut' parts)
          if (WE < 2) {
            a.x = (a.x & one_keep) | one_bits;
            a.z = (a.z & one_keep) | one_bits;
          } else {
            a.y = (a.y & one_keep) | one_bits;
            a.w = (a.w & one_keep) | one_bits;
          }
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            __builtin_bit_cast(mc_bf16x8_t, a), yb[i], acc, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < NI; ++i)
        a_next[i] = rows_lds[i][min(rt + 1, TX / 32 - 1) * 32 + col];

      uint32_t mask = 0;
#pragma unroll
      for (int v = 0; v < 16; ++v)
        mask = __builtin_amdgcn_alignbit(mask, __float_as_uint(acc[v]), 31);
      if (done)
        mask = 0;
      if (__any(mask != 0)) {
        if (mask != 0) {
          queue[qn][tid] = ((uint32_t)rt << 16) | mask;
          ++qn;
        }
        if (__any(qn >= QCAP)) {
          drain(g_base, rows);
          if (!__any(!done))
            break;
        }
      }
    }
    drain(g_base, rows);
    if (!__any(!done))
      wave_done = true;
  }

  if (valid && half == 0) {
    p.out_count[q] = count;
    if (p.edge_sums != nullptr) // (count <= slots; wide lists: one by one)
      if (p.slots < 128)
        add_to_block_sum(p.edge_sums, q / kCompactBlockQueries, count);
      else
        atomicAdd(&p.edge_sums[q / kCompactBlockQueries],
                  (unsigned long long)count);
  }
}

} // namespace pca
