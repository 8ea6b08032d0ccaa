// Farthest point sampling: the `fps` operator of the reference
// (csrc/cuda/fps_cuda.cu:10-66, fps_kernel), one workgroup of 1,024 threads
// per example.
//
// What the reference computes, and what is reproduced bit for bit: the first
// sample of an example is its start row; every further sample is the row with
// the largest running minimum distance to the samples so far, where
//   * distances are squared, accumulated with one fused multiply-add per
//     dimension (`dd += tmp * tmp`; every operator rounds to 16 bits for
//     fp16), and the running minimum starts at 5e4 for every row (the `dist`
//     array of the host wrapper, :91) -- larger distances count as 5e4;
//   * among rows of equal value the reference's block of 256 threads returns
//     the one with the smallest (row - start) % 256, then the smallest row:
//     thread t scans rows start + t, start + t + 256, ... and keeps its first
//     strict maximum (:35-47), the reduction keeps the lower thread on ties
//     (:52-59, read as lock-step rounds);
//   * `best` starts at -1 and `best_idx` at 0: when no row has a value above
//     -1 (every distance NaN) the sample is row 0.
//
// The sampling is a chain of dependent steps, each a pass over the example's
// rows plus a workgroup-wide arg-max, so the time per sample is what counts.
// fps_reg_kernel keeps the rows and their running minima in REGISTERS (up to
// 16 rows per thread: examples of up to 16,384 rows of up to 4 dimensions),
// and needs one barrier per sample: every wave finds its best row with two
// reductions of 32-bit keys by data-parallel lane shifts (value, then tie),
// the lane that holds it writes value, tie and coordinates to LDS, and after
// the barrier every row of 16 lanes picks the winner among the 16 wave
// results the same way and reads its coordinates.  fps_any_kernel (any size,
// dimension and element type) streams the rows and a `dist` array from memory
// instead.
#include "device_utils.hpp"
#include "launchers.hpp"

#include <hip/hip_fp16.h>

namespace pca {

namespace {

constexpr int kFpsThreads = 1024;
constexpr int kFpsWaves = kFpsThreads / kWave;
constexpr uint32_t kFpsNoTie = 0xffffffffu;

// Order among equal values: (row - start) % 256 first, then the row
__device__ __forceinline__ uint32_t fps_tie(uint32_t rel) {
  return ((rel & 255u) << 24) | (rel >> 8);
}
__device__ __forceinline__ uint32_t fps_rel(uint32_t tie) {
  return ((tie & 0xffffffu) << 8) | (tie >> 24);
}

// (value, tie) a beats b
template <typename T>
__device__ __forceinline__ bool fps_better(T ad, uint32_t at, T bd,
                                           uint32_t bt) {
  return ad > bd || (ad == bd && at < bt);
}

__device__ __forceinline__ float shfl_xor_t(float v, int m) {
  return __shfl_xor(v, m);
}
__device__ __forceinline__ double shfl_xor_t(double v, int m) {
  return __shfl_xor(v, m);
}

// Largest value of a wave / of every row of 16 lanes, by data-parallel
// primitives (one fused shift-and-max instruction per step; lanes without a
// source take 0, the smallest value).  The wave's result is uniform.
#define PCA_DPP_UMAX(v, ctrl, rows)                                            \
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(v), ctrl, rows,    \
                                                   0xf, false))
__device__ __forceinline__ uint32_t row16_umax(uint32_t v) {
  PCA_DPP_UMAX(v, 0x111, 0xf); // row_shr:1
  PCA_DPP_UMAX(v, 0x112, 0xf); // row_shr:2
  PCA_DPP_UMAX(v, 0x114, 0xf); // row_shr:4
  PCA_DPP_UMAX(v, 0x118, 0xf); // row_shr:8
  return v; // lane 15 of every row holds the row's maximum
}
__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
  v = row16_umax(v);
  PCA_DPP_UMAX(v, 0x142, 0xa); // row_bcast:15 into rows 1 and 3
  PCA_DPP_UMAX(v, 0x143, 0xc); // row_bcast:31 into rows 2 and 3
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
#undef PCA_DPP_UMAX

// ---- element types ----------------------------------------------------------

struct FpsF32 {
  typedef float store_t;
  typedef float calc_t;
  static __device__ __forceinline__ calc_t load(store_t v) { return v; }
  static __device__ __forceinline__ calc_t step(calc_t a, calc_t b,
                                                calc_t acc) {
    const calc_t t = a - b;
    return __builtin_fmaf(t, t, acc);
  }
  static __device__ __forceinline__ calc_t lower(calc_t a, calc_t b) {
    return __builtin_fminf(a, b);
  }
  static __device__ __forceinline__ calc_t limit() { return 5e4f; }
};

struct FpsF64 {
  typedef double store_t;
  typedef double calc_t;
  static __device__ __forceinline__ calc_t load(store_t v) { return v; }
  static __device__ __forceinline__ calc_t step(calc_t a, calc_t b,
                                                calc_t acc) {
    const calc_t t = a - b;
    return __builtin_fma(t, t, acc);
  }
  static __device__ __forceinline__ calc_t lower(calc_t a, calc_t b) {
    return __builtin_fmin(a, b);
  }
  static __device__ __forceinline__ calc_t limit() { return 5e4; }
};

// c10::Half arithmetic: every operator computes in float and rounds to 16
// bits; values travel as floats that are representable halves
struct FpsF16 {
  typedef uint16_t store_t;
  typedef float calc_t;
  static __device__ __forceinline__ float r16(float v) {
    return __half2float(__float2half_rn(v));
  }
  static __device__ __forceinline__ calc_t load(store_t v) {
    return __half2float(__ushort_as_half(v));
  }
  static __device__ __forceinline__ calc_t step(calc_t a, calc_t b,
                                                calc_t acc) {
    const float t = r16(a - b);
    const float p = r16(t * t);
    return r16(acc + p);
  }
  static __device__ __forceinline__ calc_t lower(calc_t a, calc_t b) {
    return __builtin_fminf(a, b);
  }
  static __device__ __forceinline__ calc_t limit() { return r16(5e4f); }
};

// ---- any size, dimension and element type -------------------------------------

// dist: [n] running minima (initialised here); one workgroup per example.
template <typename Tr>
__global__ __launch_bounds__(kFpsThreads) void fps_any_kernel(
    const typename Tr::store_t *__restrict__ src,
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ out_ptr,
    const int64_t *__restrict__ start, int d,
    typename Tr::calc_t *__restrict__ dist, int64_t *__restrict__ out) {
  typedef typename Tr::calc_t calc_t;
  __shared__ calc_t s_d[2][kFpsWaves];
  __shared__ uint32_t s_t[2][kFpsWaves];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int b = blockIdx.x;
  const int64_t start_idx = ptr[b];
  const int64_t end_idx = ptr[b + 1];
  const int64_t o_begin = out_ptr[b];
  const int64_t o_end = out_ptr[b + 1];
  if (o_begin >= o_end)
    return;

  for (int64_t n = start_idx + tid; n < end_idx; n += kFpsThreads)
    dist[n] = Tr::limit();
  int64_t old = start_idx + (start ? start[b] : 0);
  if (tid == 0)
    out[o_begin] = old;

  for (int64_t m = o_begin + 1; m < o_end; ++m) {
    const int par = (int)(m & 1);
    const typename Tr::store_t *cur = src + (size_t)old * d;
    calc_t best = (calc_t)-1;
    uint32_t best_tie = kFpsNoTie;
    // a thread's rows share (row - start) % 256, so its first strict
    // maximum is its best by the tie rule as well
    for (int64_t n = start_idx + tid; n < end_idx; n += kFpsThreads) {
      const typename Tr::store_t *row = src + (size_t)n * d;
      calc_t dd = 0;
      for (int c = 0; c < d; ++c)
        dd = Tr::step(Tr::load(cur[c]), Tr::load(row[c]), dd);
      dd = Tr::lower(dist[n], dd);
      dist[n] = dd;
      if (dd > best) {
        best = dd;
        best_tie = fps_tie((uint32_t)(n - start_idx));
      }
    }
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1) {
      const calc_t od = shfl_xor_t(best, sh);
      const uint32_t ot = __shfl_xor(best_tie, sh);
      if (fps_better(od, ot, best, best_tie)) {
        best = od;
        best_tie = ot;
      }
    }
    if (lane == 0) {
      s_d[par][wave] = best;
      s_t[par][wave] = best_tie;
    }
    __syncthreads();
    best = s_d[par][0];
    best_tie = s_t[par][0];
#pragma unroll
    for (int w = 1; w < kFpsWaves; ++w) {
      const calc_t od = s_d[par][w];
      const uint32_t ot = s_t[par][w];
      if (fps_better(od, ot, best, best_tie)) {
        best = od;
        best_tie = ot;
      }
    }
    // nothing above -1: the reference's `best_idx` is still 0
    old = best_tie != kFpsNoTie ? start_idx + (int64_t)fps_rel(best_tie) : 0;
    if (tid == 0)
      out[m] = old;
  }
}

// ---- fp32, up to 4 dimensions, up to T * P rows per example -------------------

// T threads hold P rows each.  With T = 256 S, thread t has the rows
// t / S + 256 * ((t % S) * P + i), i < P, of its example; a single wave
// (T = 64) gives thread t the rows 4 t + i / (P / 4) + 256 * (i % (P / 4)).
// Among equal values the reference's order is "(row - start) % 256, then the
// row", which in these layouts reads "t, then i": the first thread wins, and
// inside it the first slot.  Every "first of the equal ones" is therefore a
// count of trailing zeros of a ballot, and only the values themselves go
// through a reduction.  A step costs every wave the same few dozen
// instructions of reduction and hand-over on top of its 8 P of distances,
// and the waves of a SIMD take turns: the launcher picks the shape that
// measured fastest for the row count.  The single wave needs neither the
// hand-over through shared memory nor a barrier.
template <int DIM, int P, int T>
__global__ __launch_bounds__(T) void fps_reg_kernel(
    const float *__restrict__ src, const int64_t *__restrict__ ptr,
    const int64_t *__restrict__ out_ptr, const int64_t *__restrict__ start,
    int d, int64_t *__restrict__ out) {
  // per wave and parity: value (as an ordered unsigned number,
  // 0 = none), row (relative to the example) and coordinates of the wave's best
  __shared__ uint32_t s_v[2][kFpsWaves];
  __shared__ uint32_t s_rel[2][kFpsWaves];
  __shared__ float s_x[2][DIM][kFpsWaves];
  static_assert(kFpsWaves == 16 && (T % 256 == 0 || T == kWave) &&
                    T <= kFpsThreads,
                "one row of 16 lanes picks the winner among up to 16 waves");
  static_assert(T != kWave || P % 4 == 0, "four tie classes per lane");

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  constexpr int S = T >= 256 ? T / 256 : 1; // threads per tie class
  constexpr int C = T >= 256 ? 1 : 256 / T; // tie classes per thread
  constexpr int PARTS = P / C;              // slots per tie class
  const int rel0 = (tid / S) * C + 256 * ((tid % S) * P);
  // row of slot i, relative to rel0
  auto slot_row = [](int i) { return i / PARTS + 256 * (i % PARTS); };
  const int b = blockIdx.x;
  const int64_t start_idx = ptr[b];
  const int count = (int)(ptr[b + 1] - start_idx);
  const int64_t o_begin = out_ptr[b];
  const int64_t o_end = out_ptr[b + 1];
  if (o_begin >= o_end)
    return;
  if (T < kFpsThreads && T > kWave) {
    // the entries of waves that do not run stay "nothing"
    if (tid < 2 * kFpsWaves)
      s_v[tid / kFpsWaves][tid % kFpsWaves] = 0u;
    __syncthreads();
  }

  float px[P][DIM];
  // A slot's running minimum is the high word of a 64-bit pattern whose low
  // word is 15 - i.  Minima are -1 (no row) or in [0, 5e4]: read as doubles,
  // the patterns of rows order by minimum first and smaller slot second, and
  // none is a NaN or an infinity, so one 64-bit maximum per slot tracks the
  // thread's best (the first of its largest minima) and where it is.
  double slot_key[P];
  static_assert(P <= 16, "low words 15 - i");
#pragma unroll
  for (int i = 0; i < P; ++i) {
    const int rel = rel0 + slot_row(i);
#pragma unroll
    for (int c = 0; c < DIM; ++c)
      px[i][c] = (rel < count && c < d)
                     ? src[(size_t)(start_idx + rel) * d + c]
                     : 0.0f;
    slot_key[i] = __hiloint2double(
        __float_as_int(rel < count ? 5e4f : -1.0f), 15 - i);
  }
  const int64_t first = start_idx + (start ? start[b] : 0);
  if (tid == 0)
    out[o_begin] = first;
  float cur[DIM];
#pragma unroll
  for (int c = 0; c < DIM; ++c)
    cur[c] = c < d ? src[(size_t)first * d + c] : 0.0f;

  for (int64_t m = o_begin + 1; m < o_end; ++m) {
    const int par = (int)(m & 1);
    // (below every slot's pattern: -1 with the largest low word)
    double best_key = __hiloint2double(__float_as_int(-1.0f), -1);
    // (component by component over all slots: independent instructions
    // follow each other, a slot's own chain is spread out)
    float dd[P];
#pragma unroll
    for (int i = 0; i < P; ++i) {
      const float t0 = cur[0] - px[i][0];
      dd[i] = t0 * t0;
    }
#pragma unroll
    for (int c = 1; c < DIM; ++c) {
#pragma unroll
      for (int i = 0; i < P; ++i) {
        // (zero components beyond d add fma(0, 0, acc) = acc)
        const float tc = cur[c] - px[i][c];
        dd[i] = __builtin_fmaf(tc, tc, dd[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < P; ++i) {
      // fminf without its quieting of signalling NaNs, which neither operand
      // can be (5e4, -1, or the result of arithmetic): a NaN loses to a number
      const float before = __int_as_float(__double2hiint(slot_key[i]));
      asm("v_min_f32 %0, %1, %2" : "=v"(dd[i]) : "v"(before), "v"(dd[i]));
      slot_key[i] = __hiloint2double(__float_as_int(dd[i]),
                                     __double2loint(slot_key[i]));
    }
    double part_key[2] = {best_key, best_key};
#pragma unroll
    for (int i = 0; i < P; ++i)
      asm("v_max_f64 %0, %1, %2"
          : "=v"(part_key[i & 1])
          : "v"(part_key[i & 1]), "v"(slot_key[i]));
    asm("v_max_f64 %0, %1, %2"
        : "=v"(best_key)
        : "v"(part_key[0]), "v"(part_key[1]));
    const uint32_t best_bits = (uint32_t)__double2hiint(best_key);
    const int best_i = best_bits != __float_as_uint(-1.0f)
                           ? 15 - __double2loint(best_key)
                           : -1;
    // values are -1 (nothing) or >= 0: their bit patterns, with the top bit
    // set, order like the values
    const uint32_t key = best_i >= 0 ? (best_bits | 0x80000000u) : 0u;
    const uint32_t wave_key = wave_umax(key);
    const int src_lane = (int)__builtin_ctzll(__ballot(key == wave_key));
    // which of its rows that lane means: a uniform number, so every lane
    // picks that slot of its own registers with scalar branches (no per-row
    // bookkeeping of coordinates in the loop above)
    const int slot = __builtin_amdgcn_readlane(best_i, src_lane);
    float bx[DIM];
#pragma unroll
    for (int c = 0; c < DIM; ++c)
      bx[c] = 0.0f;
    switch (slot) {
#define PCA_FPS_SLOT(i_)                                                       \
  case i_:                                                                     \
    if (i_ < P) {                                                              \
      _Pragma("unroll") for (int c = 0; c < DIM; ++c) bx[c] =                  \
          px[i_ < P ? i_ : 0][c];                                              \
    }                                                                          \
    break;
      PCA_FPS_SLOT(0) PCA_FPS_SLOT(1) PCA_FPS_SLOT(2) PCA_FPS_SLOT(3)
      PCA_FPS_SLOT(4) PCA_FPS_SLOT(5) PCA_FPS_SLOT(6) PCA_FPS_SLOT(7)
      PCA_FPS_SLOT(8) PCA_FPS_SLOT(9) PCA_FPS_SLOT(10) PCA_FPS_SLOT(11)
      PCA_FPS_SLOT(12) PCA_FPS_SLOT(13) PCA_FPS_SLOT(14) PCA_FPS_SLOT(15)
#undef PCA_FPS_SLOT
    default:
      break;
    }
    static_assert(P <= 16, "slots of the switch above");
    int64_t chosen;
    if (T == kWave) {
      if (wave_key != 0u) {
        chosen = start_idx + __builtin_amdgcn_readlane(rel0, src_lane) +
                 slot_row(slot);
#pragma unroll
        for (int c = 0; c < DIM; ++c)
          cur[c] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
              (int)__float_as_uint(bx[c]), src_lane));
      } else {
        // nothing above -1: the reference's `best_idx` is still 0
        chosen = 0;
#pragma unroll
        for (int c = 0; c < DIM; ++c)
          cur[c] = c < d ? src[c] : 0.0f;
      }
    } else {
      if (lane == src_lane) {
        s_v[par][wave] = wave_key;
        s_rel[par][wave] = (uint32_t)(rel0 + slot_row(slot));
#pragma unroll
        for (int c = 0; c < DIM; ++c)
          s_x[par][c][wave] = bx[c];
      }
      __syncthreads();
      // every row of 16 lanes looks at the 16 wave results
      const uint32_t ev = s_v[par][lane & 15];
      const uint32_t erel = s_rel[par][lane & 15];
      float ex[DIM];
#pragma unroll
      for (int c = 0; c < DIM; ++c) {
        ex[c] = s_x[par][c][lane & 15];
        asm volatile("" : "+v"(ex[c])); // (read now, not after the reduction)
      }
      const uint32_t top_key =
          (uint32_t)__builtin_amdgcn_readlane((int)row16_umax(ev), 15);
      if (top_key != 0u) {
        const int win = (int)__builtin_ctzll(__ballot(ev == top_key));
        chosen =
            start_idx + (int64_t)__builtin_amdgcn_readlane((int)erel, win);
#pragma unroll
        for (int c = 0; c < DIM; ++c)
          cur[c] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
              (int)__float_as_uint(ex[c]), win));
      } else {
        // nothing above -1: the reference's `best_idx` is still 0
        chosen = 0;
#pragma unroll
        for (int c = 0; c < DIM; ++c)
          cur[c] = c < d ? src[c] : 0.0f;
      }
    }
    if (tid == 0)
      out[m] = chosen;
    // (in vector registers: the distance code then interleaves its rows)
#pragma unroll
    for (int c = 0; c < DIM; ++c)
      asm volatile("" : "+v"(cur[c]));
  }
}

template <int DIM>
hipError_t launch_fps_reg(const float *src, const int64_t *ptr,
                          const int64_t *out_ptr, const int64_t *start, int d,
                          int num_segments, int64_t max_rows, int64_t *out,
                          hipStream_t stream) {
#define PCA_FPS_REG(P_, T_)                                                    \
  hipLaunchKernelGGL((fps_reg_kernel<DIM, P_, T_>), dim3(num_segments),        \
                     dim3(T_), 0, stream, src, ptr, out_ptr, start, d, out)
  // (shapes by measurement: 16 examples of each size on one device)
  if (max_rows <= 256)
    PCA_FPS_REG(4, 64);
  else if (max_rows <= 512)
    PCA_FPS_REG(8, 64);
  else if (max_rows <= 1024)
    PCA_FPS_REG(2, 512);
  else if (max_rows <= 2048)
    PCA_FPS_REG(4, 512);
  else if (max_rows <= 4096)
    PCA_FPS_REG(8, 512);
  else if (max_rows <= 8192)
    PCA_FPS_REG(16, 512);
  else
    PCA_FPS_REG(16, 1024);
#undef PCA_FPS_REG
  return hipGetLastError();
}

template <typename Tr>
hipError_t launch_fps_any(const void *src, const int64_t *ptr,
                          const int64_t *out_ptr, const int64_t *start, int d,
                          int num_segments, void *dist, int64_t *out,
                          hipStream_t stream) {
  hipLaunchKernelGGL((fps_any_kernel<Tr>), dim3(num_segments),
                     dim3(kFpsThreads), 0, stream,
                     static_cast<const typename Tr::store_t *>(src), ptr,
                     out_ptr, start, d,
                     static_cast<typename Tr::calc_t *>(dist), out);
  return hipGetLastError();
}

} // namespace

bool fps_in_registers(int dtype, int d, int64_t max_rows) {
  return dtype == 0 && d >= 1 && d <= 4 && max_rows >= 1 &&
         max_rows <= 16 * kFpsThreads;
}

size_t fps_dist_bytes(int64_t n) { return sizeof(double) * (size_t)n; }

hipError_t launch_fps(int dtype, const void *src, const int64_t *ptr,
                      const int64_t *out_ptr, const int64_t *start, int d,
                      int num_segments, int64_t max_rows, void *dist,
                      int64_t *out, hipStream_t stream) {
  if (fps_in_registers(dtype, d, max_rows)) {
    const float *s = static_cast<const float *>(src);
    if (d <= 2)
      return launch_fps_reg<2>(s, ptr, out_ptr, start, d, num_segments,
                               max_rows, out, stream);
    if (d == 3)
      return launch_fps_reg<3>(s, ptr, out_ptr, start, d, num_segments,
                               max_rows, out, stream);
    return launch_fps_reg<4>(s, ptr, out_ptr, start, d, num_segments, max_rows,
                             out, stream);
  }
  switch (dtype) {
  case 0:
    return launch_fps_any<FpsF32>(src, ptr, out_ptr, start, d, num_segments,
                                  dist, out, stream);
  case 1:
    return launch_fps_any<FpsF64>(src, ptr, out_ptr, start, d, num_segments,
                                  dist, out, stream);
  case 2:
    return launch_fps_any<FpsF16>(src, ptr, out_ptr, start, d, num_segments,
                                  dist, out, stream);
  default:
    return hipErrorInvalidValue;
  }
}

} // namespace pca
