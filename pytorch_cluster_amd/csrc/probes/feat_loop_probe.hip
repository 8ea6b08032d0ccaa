// Stripped loop of the feature-space kNN filter (knn_feat_impl.hpp, knn_feat_wide_impl.hpp): the
// matrix-core chain of csrc/cuda/knn_cuda.cu:52-78's distance loop for 128 features (nine operand blocks
// of 16 halves: the features, the row norm, the folded cut) with everything else taken away, piece by piece
// put back.  It answers what the loop's structure alone allows on this machine, whatever the filter does
// around it: a measurement aid, not part of the search.  Built as a library of its own
// (libpca_probe.so, one entry point) and run by `python bench.py --probe feat_loop`.
//
// Variants (template arguments of loop_kernel):
//   RB     query blocks (of 32) per wave that share one x operand
//   TILE   rows of x per LDS tile
//   SYNC   bit 0: a workgroup barrier per tile; bit 1: tiles staged from global memory with
//          global_load_lds_dwordx4 into a ring of RING tiles
//   VALU   0 nothing, 1 the sign masks and minimum tree over the previous tile's products (cut folded into
//          the product), 2 the same with a subtraction of the cut per value
//   LDSRD  x operands read from LDS (else kept in registers)
//   WGS    workgroups per compute unit asked of the compiler, WAVES waves per workgroup
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float acc_t __attribute__((ext_vector_type(16)));

constexpr int NB = 9;
constexpr int RSU = 2 * NB + 1;

__device__ __forceinline__ float min3f(float a, float b, float c) {
  return __builtin_fminf(__builtin_fminf(a, b), c);
}

// RB query blocks per wave, TILE rows per LDS tile, SYNC: tiles staged from global with a barrier per
// tile, VALU: 0 nothing, 1 sign masks (cut folded), 2 sign masks with subtraction, LDSRD: A operands from LDS
template <int RB, int TILE, int SYNC, int VALU, int LDSRD, int WGS, int RING, int WAVES>
__global__ __launch_bounds__(64 * WAVES, WGS) void loop_kernel(const uint4 *__restrict__ x_pack, int rows_per_wg,
                                                        float cut_in, unsigned *out) {
  constexpr int SUBS = TILE / 32;
  constexpr int TILE_UNITS = TILE * RSU;
  constexpr int PIECES = (TILE_UNITS + 63) / 64;
  constexpr int MAXP = (PIECES + WAVES - 1) / WAVES;
  __shared__ __attribute__((aligned(16))) uint4 xs[RING][TILE_UNITS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, col = lane & 31;
  const int num_tiles = rows_per_wg / TILE;
  const size_t c_begin = (size_t)(blockIdx.x % 61) * 3000; // somewhere in the matrix
  f16x8 yh[RB][NB];
  for (int b = 0; b < RB; ++b)
    for (int i = 0; i < NB; ++i)
      for (int e = 0; e < 8; ++e)
        yh[b][i][e] = (_Float16)(0.001f * ((tid * 7 + i * 3 + e + b) & 63));
  float cut = cut_in;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto request_tile = [&](int t) {
    const uint4 *src = x_pack + (c_begin + (size_t)t * TILE) * RSU;
    const uint32_t dst = (uint32_t)(uintptr_t)&xs[t % RING][0];
#pragma unroll
    for (int e = 0; e < MAXP; ++e) {
      const int piece = wave_u + WAVES * e;
      const int u = piece * 64 + lane;
      if (piece < PIECES && (TILE_UNITS % 64 == 0 || u < TILE_UNITS)) {
        const uint4 *g = src + u;
        const uint32_t base = dst + (uint32_t)piece * (64 * 16);
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(base) : "memory");
      }
    }
  };
  // all but the `newer` newest tiles of this wave have arrived
  auto await_tile = [&](int newer) {
    if (newer >= RING - 1 && RING >= 2)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(MAXP * (RING - 1) > 63 ? 63 : MAXP * (RING - 1)) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  for (int i = tid; i < RING * TILE_UNITS; i += 64 * WAVES)
    xs[0][i] = make_uint4(0x3c003c00u + i, 0x3c003c00u, 0x38003800u, 0x34003400u);
  __syncthreads();
  if (SYNC & 2) {
#pragma unroll
    for (int r = 0; r < RING; ++r)
      request_tile(r);
    await_tile(RING - 1);
  }
  unsigned sink = 0;
  float sinkf = 1e30f;
  f16x8 areg;
  for (int e = 0; e < 8; ++e)
    areg[e] = (_Float16)(0.01f * (lane + e));

  auto pass = [&](acc_t (&cur)[SUBS][RB], acc_t (&old)[SUBS][RB], int t) __attribute__((always_inline)) {
    if (SYNC & 1)
      __syncthreads();
    if (SYNC & 2) {
      if (t >= 1 && t + RING - 1 < num_tiles)
        request_tile(t + RING - 1);
    }
    asm volatile("" : "+v"(areg));
    const uint4 *arow = &xs[t % RING][col * RSU + half];
    constexpr int OPS = SUBS * NB;
    constexpr int AHEAD = 4;
    uint4 window[AHEAD];
    if (LDSRD) {
#pragma unroll
      for (int o = 0; o < AHEAD && o < OPS; ++o)
        window[o] = arow[(o / NB) * 32 * RSU + 2 * (o % NB)];
    }
#pragma unroll
    for (int sub = 0; sub < SUBS; ++sub)
#pragma unroll
      for (int b = 0; b < RB; ++b)
        cur[sub][b] = acc_t{0};
    __builtin_amdgcn_sched_barrier(0);
    unsigned mask[SUBS][RB];
    float lo[SUBS][RB];
#pragma unroll
    for (int sub = 0; sub < SUBS; ++sub)
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        mask[sub][b] = 0;
        lo[sub][b] = 0;
        if (VALU) {
          const acc_t &a = old[sub][b];
          float m0 = min3f(a[0], a[1], a[2]);
          float m1 = min3f(a[3], a[4], a[5]);
          float m2 = min3f(a[6], a[7], a[8]);
          float m3 = min3f(a[9], a[10], a[11]);
          float m4 = min3f(a[12], a[13], a[14]);
          m0 = min3f(m0, m1, m2);
          m3 = min3f(m3, m4, a[15]);
          lo[sub][b] = __builtin_fminf(m0, m3);
          if (VALU == 2) {
            unsigned part[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              unsigned mk = __float_as_uint(a[4 * g] - cut) >> 31;
#pragma unroll
              for (int v = 1; v < 4; ++v)
                mk = __builtin_amdgcn_alignbit(mk, __float_as_uint(a[4 * g + v] - cut), 31);
              part[g] = mk & 15u;
            }
            mask[sub][b] = (part[0] << 12) | (part[1] << 8) | (part[2] << 4) | part[3];
          } else {
            unsigned mk = __float_as_uint(a[0]) >> 31;
#pragma unroll
            for (int v = 1; v < 16; ++v)
              mk = __builtin_amdgcn_alignbit(mk, __float_as_uint(a[v]), 31);
            mask[sub][b] = mk & 0xffffu;
          }
        }
      }
#pragma unroll
    for (int o = 0; o < OPS; ++o) {
      // (a register operand the compiler cannot prove equal from one product to the next: equal
      // products of the two sub-tiles would be computed once)
      asm volatile("" : "+v"(areg));
      f16x8 a = areg;
      if (LDSRD) {
        a = __builtin_bit_cast(f16x8, window[o % AHEAD]);
        if (o + AHEAD < OPS) {
          const int n = o + AHEAD;
          window[o % AHEAD] = arow[(n / NB) * 32 * RSU + 2 * (n % NB)];
        }
      }
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        cur[o / NB][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, yh[b][o % NB], cur[o / NB][b], 0, 0, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (b == 0 && LDSRD)
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (VALU)
          __builtin_amdgcn_sched_group_barrier(0x002, VALU == 2 ? 6 : 3, 0);
      }
    }
#pragma unroll
    for (int sub = 0; sub < SUBS; ++sub)
#pragma unroll
      for (int b = 0; b < RB; ++b)
        asm volatile("" : "+v"(mask[sub][b]), "+v"(lo[sub][b]));
    __builtin_amdgcn_sched_barrier(0);
    // tile t + 1 of this wave: all but the RING - 2 newest requests (tiles t + 2 .. t + RING - 1)
    if ((SYNC & 2) && t + 1 < num_tiles) {
      if (t + RING - 1 < num_tiles)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(MAXP * (RING - 2) > 63 ? 63 : MAXP * (RING - 2)) : "memory");
      else
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    bool any_low = false;
#pragma unroll
    for (int sub = 0; sub < SUBS; ++sub)
#pragma unroll
      for (int b = 0; b < RB; ++b)
        any_low |= mask[sub][b] != 0;
    if (__any(any_low)) {
#pragma unroll
      for (int sub = 0; sub < SUBS; ++sub)
#pragma unroll
        for (int b = 0; b < RB; ++b) {
          sink ^= mask[sub][b];
          sinkf = __builtin_fminf(sinkf, lo[sub][b]);
        }
    }
  };
  acc_t acc_a[SUBS][RB], acc_b[SUBS][RB];
#pragma unroll
  for (int sub = 0; sub < SUBS; ++sub)
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      acc_a[sub][b] = acc_t{0};
      acc_b[sub][b] = acc_t{0};
    }
#pragma unroll 1
  for (int t = 0; t < num_tiles; t += 2) {
    pass(acc_a, acc_b, t);
    pass(acc_b, acc_a, t + 1);
  }
  float r = sinkf;
#pragma unroll
  for (int sub = 0; sub < SUBS; ++sub)
#pragma unroll
    for (int b = 0; b < RB; ++b)
      for (int j = 0; j < 16; ++j)
        r += acc_a[sub][b][j] + acc_b[sub][b][j];
  if (r == 12345.678f || sink == 0xdeadbeefu)
    out[tid] = sink;
}


struct Result {
  const char *name;
  int rb, tile, sync, valu, ldsrd, wgs, ring, waves, regs;
  size_t lds;
  double ms, flops;
};

template <int RB, int TILE, int SYNC, int VALU, int LDSRD, int WGS, int RING = 3, int WAVES = 4>
int run(const uint4 *x, unsigned *out, int reps, const char *name, std::vector<Result> &results) {
  const int rows_per_wg = 24576 / RB; // the same matrix work per wave in every variant
  const int grid = 3072 * 4 / WAVES;  // and the same number of waves
  hipEvent_t a, b;
  if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess)
    return -1;
  auto k = loop_kernel<RB, TILE, SYNC, VALU, LDSRD, WGS, RING, WAVES>;
  hipLaunchKernelGGL(k, dim3(grid), dim3(64 * WAVES), 0, 0, x, rows_per_wg, -1e30f, out);
  if (hipDeviceSynchronize() != hipSuccess)
    return -1;
  float best = 1e9f;
  for (int rep = 0; rep < reps; ++rep) {
    (void)hipEventRecord(a, 0);
    hipLaunchKernelGGL(k, dim3(grid), dim3(64 * WAVES), 0, 0, x, rows_per_wg, -1e30f, out);
    (void)hipEventRecord(b, 0);
    if (hipEventSynchronize(b) != hipSuccess)
      return -1;
    float ms;
    (void)hipEventElapsedTime(&ms, a, b);
    best = ms < best ? ms : best;
  }
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
  hipFuncAttributes attr;
  (void)hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(k));
  // every wave: rows / 32 sub-tiles x NB operand blocks x RB query blocks, 32*32*16*2 flops each
  const double mfma = (double)grid * WAVES * (rows_per_wg / 32) * NB * RB;
  results.push_back({name, RB, TILE, SYNC, VALU, LDSRD, WGS, RING, WAVES, attr.numRegs,
                     (size_t)attr.sharedSizeBytes, (double)best, mfma * 32768.0});
  return 0;
}

} // namespace

// Runs every variant `reps` times (best time kept) on the current device's default stream and writes one
// line per variant, as JSON objects separated by newlines, into `text` (at most `text_len` bytes).
// Returns the number of variants, or -1 when a HIP call failed or the text did not fit.
extern "C" int pca_probe_feat_loop(int reps, char *text, int text_len) {
  const size_t rows = 200064 + 64;
  uint4 *x = nullptr;
  unsigned *out = nullptr;
  if (hipMalloc(&x, rows * RSU * 16) != hipSuccess || hipMalloc(&out, 4096) != hipSuccess)
    return -1;
  {
    std::vector<uint32_t> h(rows * RSU * 4);
    for (size_t i = 0; i < h.size(); ++i)
      h[i] = 0x34003400u + (uint32_t)((i * 2654435761u) >> 22 & 0x03ff03ffu);
    if (hipMemcpy(x, h.data(), h.size() * 4, hipMemcpyHostToDevice) != hipSuccess)
      return -1;
  }
  std::vector<Result> results;
  int rc = 0;
  reps = reps < 1 ? 1 : reps;
  // the chain alone, operands in registers; then operands from LDS; then a barrier per tile
  rc |= run<1, 64, 0, 0, 0, 2>(x, out, reps, "chain only, operands in registers", results);
  rc |= run<1, 64, 0, 0, 1, 2>(x, out, reps, "+ x operands from LDS", results);
  rc |= run<1, 64, 1, 0, 1, 2>(x, out, reps, "+ barrier per tile", results);
  // tiles staged from global memory: the four-wave kernel's shape, then what else was tried
  rc |= run<1, 64, 3, 0, 1, 2, 3, 4>(x, out, reps, "staged, 2 x 4 waves, ring 3 (four-wave kernel)", results);
  rc |= run<1, 64, 3, 1, 1, 2, 3, 4>(x, out, reps, "  + sign masks and minimum tree", results);
  rc |= run<1, 64, 3, 2, 1, 2, 3, 4>(x, out, reps, "  + the cut subtracted per value", results);
  rc |= run<1, 64, 3, 1, 1, 1, 4, 8>(x, out, reps, "staged, 1 x 8 waves, ring 4 (eight-wave kernel)", results);
  rc |= run<1, 64, 3, 1, 1, 1, 4, 16>(x, out, reps, "staged, 1 x 16 waves, ring 4", results);
  rc |= run<1, 32, 3, 1, 1, 1, 6, 8>(x, out, reps, "staged, 1 x 8 waves, tile 32, ring 6", results);
  rc |= run<2, 32, 3, 1, 1, 2, 4, 4>(x, out, reps, "two query blocks per wave, 2 x 4 waves, tile 32", results);
  rc |= run<2, 32, 3, 1, 1, 1, 4, 8>(x, out, reps, "two query blocks per wave, 1 x 8 waves, tile 32", results);
  rc |= run<2, 64, 3, 1, 1, 1, 4, 8>(x, out, reps, "two query blocks per wave, 1 x 8 waves, tile 64", results);
  (void)hipFree(x);
  (void)hipFree(out);
  if (rc != 0)
    return -1;
  size_t used = 0;
  for (const Result &r : results) {
    const int n = snprintf(text + used, used < (size_t)text_len ? (size_t)text_len - used : 0,
                           "{\"variant\": \"%s\", \"query_blocks\": %d, \"tile_rows\": %d, \"sync\": %d, "
                           "\"valu\": %d, \"lds_operands\": %d, \"wgs_per_cu\": %d, \"ring\": %d, \"waves\": %d, "
                           "\"vgprs\": %d, \"lds_bytes\": %zu, \"ms\": %.4f, \"tflops\": %.1f, "
                           "\"frac_of_2500\": %.3f}\n",
                           r.name, r.rb, r.tile, r.sync, r.valu, r.ldsrd, r.wgs, r.ring, r.waves, r.regs, r.lds, r.ms,
                           r.flops / (r.ms * 1e-3) / 1e12, r.flops / (r.ms * 1e-3) / 2.5e15);
    if (n < 0 || used + (size_t)n >= (size_t)text_len)
      return -1;
    used += (size_t)n;
  }
  return (int)results.size();
}
