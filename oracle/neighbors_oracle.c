/*
 * TEST INFRASTRUCTURE ONLY -- the product never links, loads or calls this.
 *
 * CPU restatement of the reference's GPU semantics for the kNN / radius
 * neighbour-search path, in plain C.  It is the checker for the HIP kernels
 * (tests/, the smoke check and the cpu_baseline leg of the benchmark may use
 * it; nothing else may).
 *
 * What is restated (reference file:line):
 *   oracle_knn_dense_*     csrc/cuda/knn_cuda.cu:30-84   (knn_kernel) with the
 *                          default ptr of the host wrapper (:100-112) and
 *                          csrc/cuda/utils.cuh:11-19     (get_example_idx)
 *   cosine distance        csrc/cuda/knn_cuda.cu:9-28,55-59
 *   oracle_radius_dense_*  csrc/cuda/radius_cuda.cu:9-42 (radius_kernel); the
 *                          caller passes r*r formed in double and narrowed to
 *                          the element type as the host wrapper does (:90)
 *   oracle_compact         csrc/cuda/knn_cuda.cu:133-134 and
 *                          csrc/cuda/radius_cuda.cu:94-95 (mask on -1, two
 *                          masked_selects, stack)
 *   oracle_nearest_*       csrc/cuda/nearest_cuda.cu:10-66 (nearest_kernel):
 *                          the block of 1,024 threads is played through
 *                          literally -- strided scan per thread (:31-44),
 *                          then the pairwise reduction over shared memory
 *                          (:46-59) -- so that the candidate chosen among
 *                          equal distances is the reference's
 *   oracle_fps_*           csrc/cuda/fps_cuda.cu:10-66 (fps_kernel): the block
 *                          of 256 threads played through in the same way, per
 *                          sample: strided scan with the running minimum
 *                          distances (:35-47), then the reduction over shared
 *                          memory (:52-59), read as lock-step rounds
 *
 * Arithmetic: `fma_mode` = 1 evaluates every `acc += a * b` of the reference
 * kernels as one fused multiply-add (what a GPU compiler emits for that
 * source, and what the HIP kernels of this repository do explicitly), 0 rounds
 * the product and the sum separately (what a CPU build without FMA
 * contraction does).  The file is compiled with -ffp-contract=off so nothing
 * else is fused.
 *
 * Parity pins (see tests/test_oracle_*.py): the reference's inline fixtures
 * test/test_knn.py:16-52,57-75, test/test_radius.py:25-116, the ordered README
 * outputs README.md:188-191,217-220, the reference's compiled CPU operators
 * (oracle/_ref), scipy's cKDTree as in test/test_knn.py:84-88 and
 * test/test_radius.py:129-133, and float64 brute force.  oracle_nearest_*:
 * the fixture test/test_nearest.py:11-35, scipy.cluster.vq.vq (the
 * reference's own CPU route, torch_cluster/nearest.py:122-124), float64
 * brute force, and a closed form of the tie rule (smallest distance, then
 * smallest (row - segment start) % 1024, then smallest row).
 * oracle_fps_*: the fixture test/test_fps.py:16-63, float64 brute-force
 * farthest point sampling on data without ties, the reference's compiled CPU
 * operator (oracle/_ref, csrc/cpu/fps_cpu.cpp) on such data, and a closed form
 * of the tie rule (largest clipped distance, then smallest
 * (row - start) % 256, then smallest row).
 * PARITY UNPINNED, two details of oracle_fps_*: the reference's reduction
 * (csrc/cuda/fps_cuda.cu:52-59) reads and writes its shared arrays within a
 * round without a barrier, so which of several rows of EQUAL value it returns
 * can depend on the timing of its warps -- the lock-step reading restated here
 * is one of its possible outcomes (the reference's own test sorts the result
 * where ties occur, test/test_fps.py:46-60); and `min` with a NaN operand for
 * fp16 (restated as fmin, as for the other element types).  Neither can be
 * checked without an NVIDIA toolchain.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* csrc/cuda/utils.cuh:11-19 -- first i with ptr[i+1] > idx, else the last
 * segment. */
static int64_t example_idx(int64_t idx, const int64_t *ptr,
                           int64_t num_examples) {
  for (int64_t i = 0; i < num_examples; i++) {
    if (ptr[i + 1] > idx)
      return i;
  }
  return num_examples - 1;
}

#define DEFINE_ORACLE(SUFFIX, T, FMA, SQRT)                                    \
                                                                               \
  static T sqdist_##SUFFIX(const T *x, const T *y, int64_t n_x, int64_t n_y,   \
                           int64_t dim, int fma_mode) {                        \
    T acc = 0;                                                                 \
    for (int64_t d = 0; d < dim; d++) {                                        \
      T diff = x[n_x * dim + d] - y[n_y * dim + d];                            \
      if (fma_mode)                                                            \
        acc = FMA(diff, diff, acc);                                            \
      else {                                                                   \
        T sq = diff * diff;                                                    \
        acc = acc + sq;                                                        \
      }                                                                        \
    }                                                                          \
    return acc;                                                                \
  }                                                                            \
                                                                               \
  static T dot_##SUFFIX(const T *a, const T *b, int64_t n_a, int64_t n_b,      \
                        int64_t size, int fma_mode) {                          \
    T result = 0;                                                              \
    for (int64_t i = 0; i < size; i++) {                                       \
      if (fma_mode)                                                            \
        result = FMA(a[n_a * size + i], b[n_b * size + i], result);            \
      else {                                                                   \
        T p = a[n_a * size + i] * b[n_b * size + i];                           \
        result = result + p;                                                   \
      }                                                                        \
    }                                                                          \
    return result;                                                             \
  }                                                                            \
                                                                               \
  static T norm_##SUFFIX(const T *a, int64_t n_a, int64_t size,                \
                         int fma_mode) {                                       \
    return SQRT(dot_##SUFFIX(a, a, n_a, n_a, size, fma_mode));                 \
  }                                                                            \
                                                                               \
  /* One query of knn_kernel: sorted insertion list with the strict `>` test   \
   * (an equal distance never displaces an earlier, lower-index entry), 1e10   \
   * sentinel, -1 padded indices. */                                           \
  static void knn_query_##SUFFIX(const T *x, const T *y, int64_t n_y,          \
                                 int64_t x_begin, int64_t x_end, int64_t dim,  \
                                 int64_t k, int cosine, int fma_mode,          \
                                 T *best_dist, int64_t *best_idx) {            \
    for (int64_t e = 0; e < k; e++) {                                          \
      best_dist[e] = (T)1e10;                                                  \
      best_idx[e] = -1;                                                        \
    }                                                                          \
    for (int64_t n_x = x_begin; n_x < x_end; n_x++) {                          \
      T tmp_dist;                                                              \
      if (cosine) {                                                            \
        T den = norm_##SUFFIX(x, n_x, dim, fma_mode) *                         \
                norm_##SUFFIX(y, n_y, dim, fma_mode);                          \
        tmp_dist = dot_##SUFFIX(x, y, n_x, n_y, dim, fma_mode) / den;          \
        /* `1. - tmp_dist`: the literal is a double in the reference */        \
        tmp_dist = (T)(1. - (double)tmp_dist);                                 \
      } else {                                                                 \
        tmp_dist = sqdist_##SUFFIX(x, y, n_x, n_y, dim, fma_mode);             \
      }                                                                        \
      for (int64_t e1 = 0; e1 < k; e1++) {                                     \
        if (best_dist[e1] > tmp_dist) {                                        \
          for (int64_t e2 = k - 1; e2 > e1; e2--) {                            \
            best_dist[e2] = best_dist[e2 - 1];                                 \
            best_idx[e2] = best_idx[e2 - 1];                                   \
          }                                                                    \
          best_dist[e1] = tmp_dist;                                            \
          best_idx[e1] = n_x;                                                  \
          break;                                                               \
        }                                                                      \
      }                                                                        \
    }                                                                          \
  }                                                                            \
                                                                               \
  /* row/col: [m*k] as the kernel leaves them (col -1 where fewer than k       \
   * candidates exist).  dist: optional [m*k] distances (1e10 where empty). */ \
  int oracle_knn_dense_##SUFFIX(                                               \
      const T *x, const T *y, const int64_t *ptr_x, const int64_t *ptr_y,      \
      int64_t n, int64_t m, int64_t dim, int64_t num_examples, int64_t k,      \
      int cosine, int fma_mode, int64_t *row, int64_t *col, T *dist) {         \
    int64_t default_ptr_x[2] = {0, n}, default_ptr_y[2] = {0, m};              \
    if (ptr_x == NULL || ptr_y == NULL) {                                      \
      ptr_x = default_ptr_x;                                                   \
      ptr_y = default_ptr_y;                                                   \
      num_examples = 1;                                                        \
    }                                                                          \
    if (k <= 0)                                                                \
      return 1;                                                                \
    _Pragma("omp parallel") {                                                  \
      T *best_dist = (T *)malloc(sizeof(T) * (size_t)k);                       \
      int64_t *best_idx = (int64_t *)malloc(sizeof(int64_t) * (size_t)k);      \
      _Pragma("omp for schedule(dynamic, 64)") for (int64_t n_y = 0; n_y < m;  \
                                                    n_y++) {                   \
        int64_t b = example_idx(n_y, ptr_y, num_examples);                     \
        knn_query_##SUFFIX(x, y, n_y, ptr_x[b], ptr_x[b + 1], dim, k, cosine,  \
                           fma_mode, best_dist, best_idx);                     \
        for (int64_t e = 0; e < k; e++) {                                      \
          row[n_y * k + e] = n_y;                                              \
          col[n_y * k + e] = best_idx[e];                                      \
          if (dist)                                                            \
            dist[n_y * k + e] = best_dist[e];                                  \
        }                                                                      \
      }                                                                        \
      free(best_dist);                                                         \
      free(best_idx);                                                          \
    }                                                                          \
    return 0;                                                                  \
  }                                                                            \
                                                                               \
  /* row/col: [m*max_num_neighbors], pre-filled with -1 like the host wrapper  \
   * (radius_cuda.cu:75-78).  scanned: optional [m], the number of x rows the  \
   * query visited before it stopped (for the required-pairs work count). */   \
  int oracle_radius_dense_##SUFFIX(                                            \
      const T *x, const T *y, const int64_t *ptr_x, const int64_t *ptr_y,      \
      int64_t n, int64_t m, int64_t dim, int64_t num_examples, T r2,           \
      int64_t max_num_neighbors, int ignore_same_index, int fma_mode,          \
      int64_t *row, int64_t *col, int64_t *scanned) {                          \
    int64_t default_ptr_x[2] = {0, n}, default_ptr_y[2] = {0, m};              \
    if (ptr_x == NULL || ptr_y == NULL) {                                      \
      ptr_x = default_ptr_x;                                                   \
      ptr_y = default_ptr_y;                                                   \
      num_examples = 1;                                                        \
    }                                                                          \
    if (max_num_neighbors <= 0)                                                \
      return 1; /* the reference writes out of bounds here: undefined */       \
    for (int64_t i = 0; i < m * max_num_neighbors; i++) {                      \
      row[i] = -1;                                                             \
      col[i] = -1;                                                             \
    }                                                                          \
    _Pragma("omp parallel for schedule(dynamic, 64)") for (int64_t n_y = 0;    \
                                                           n_y < m; n_y++) {   \
      int64_t count = 0;                                                       \
      int64_t b = example_idx(n_y, ptr_y, num_examples);                       \
      int64_t n_x = ptr_x[b];                                                  \
      for (; n_x < ptr_x[b + 1]; n_x++) {                                      \
        T d = sqdist_##SUFFIX(x, y, n_x, n_y, dim, fma_mode);                  \
        if (d < r2 && !(ignore_same_index && n_y == n_x)) {                    \
          row[n_y * max_num_neighbors + count] = n_y;                          \
          col[n_y * max_num_neighbors + count] = n_x;                          \
          count++;                                                             \
        }                                                                      \
        if (count >= max_num_neighbors) {                                      \
          n_x++;                                                               \
          break;                                                               \
        }                                                                      \
      }                                                                        \
      if (scanned)                                                             \
        scanned[n_y] = n_x - ptr_x[b];                                         \
    }                                                                          \
    return 0;                                                                  \
  }

DEFINE_ORACLE(f32, float, fmaf, sqrtf)
DEFINE_ORACLE(f64, double, fma, sqrt)

/* ------------------------------------------------------------------------
 * nearest_kernel (csrc/cuda/nearest_cuda.cu:10-66): for every row of x the
 * row of y of the same example with the smallest squared distance.  One
 * block of NEAREST_THREADS threads per x row; thread t looks at the y rows
 * y_start + t, y_start + t + 1024, ... and keeps the first strictly smaller
 * distance (:31-44; `best` starts at 1e38 narrowed to scalar_t and
 * `best_idx` at 0, so a row whose candidates all fail `dist < best` --
 * NaN, overflow, an empty example of y -- yields index 0); the block then
 * halves the number of live entries ten times, an entry taking its right
 * neighbour's value only when that one is strictly smaller (:46-59).
 * The loops below run in exactly that order.
 * ------------------------------------------------------------------------ */
#define NEAREST_THREADS 1024

/* :17-23 -- the example whose range of ptr_x holds the row; -1 if none (the
 * reference then reads an uninitialised variable). */
static int64_t nearest_example(int64_t n_x, const int64_t *ptr_x,
                               int64_t batch_size) {
  for (int64_t b = 0; b < batch_size; b++) {
    if (n_x >= ptr_x[b] && n_x < ptr_x[b + 1])
      return b;
  }
  return -1;
}

#define DEFINE_NEAREST(SUFFIX, T, XT, DIST_EXPR, LIMIT_EXPR)                   \
  int oracle_nearest_##SUFFIX(const XT *x, const XT *y, const int64_t *ptr_x,  \
                              const int64_t *ptr_y, int64_t n, int64_t m,      \
                              int64_t dim, int64_t batch_size, int mode,       \
                              int64_t *out) {                                  \
    int64_t default_ptr_x[2] = {0, n}, default_ptr_y[2] = {0, m};              \
    if (ptr_x == NULL || ptr_y == NULL) {                                      \
      ptr_x = default_ptr_x;                                                   \
      ptr_y = default_ptr_y;                                                   \
      batch_size = 1;                                                          \
    }                                                                          \
    int bad = 0;                                                               \
    _Pragma("omp parallel") {                                                  \
      T *best_dist = (T *)malloc(sizeof(T) * NEAREST_THREADS);                 \
      int64_t *best_dist_idx =                                                 \
          (int64_t *)malloc(sizeof(int64_t) * NEAREST_THREADS);                \
      _Pragma("omp for schedule(dynamic, 16)") for (int64_t n_x = 0; n_x < n;  \
                                                    n_x++) {                   \
        const int64_t batch_idx = nearest_example(n_x, ptr_x, batch_size);     \
        if (batch_idx < 0) {                                                   \
          bad = 1;                                                             \
          out[n_x] = -1;                                                       \
          continue;                                                            \
        }                                                                      \
        const int64_t y_start_idx = ptr_y[batch_idx];                          \
        const int64_t y_end_idx = ptr_y[batch_idx + 1];                        \
        for (int64_t thread_idx = 0; thread_idx < NEAREST_THREADS;             \
             thread_idx++) {                                                   \
          T best = (LIMIT_EXPR);                                               \
          int64_t best_idx = 0;                                                \
          for (int64_t n_y = y_start_idx + thread_idx; n_y < y_end_idx;        \
               n_y += NEAREST_THREADS) {                                       \
            T dist = (DIST_EXPR);                                              \
            if (dist < best) {                                                 \
              best = dist;                                                     \
              best_idx = n_y;                                                  \
            }                                                                  \
          }                                                                    \
          best_dist[thread_idx] = best;                                        \
          best_dist_idx[thread_idx] = best_idx;                                \
        }                                                                      \
        for (int64_t u = 0; (1 << u) < NEAREST_THREADS; u++) {                 \
          for (int64_t thread_idx = 0;                                         \
               thread_idx < (NEAREST_THREADS >> (u + 1)); thread_idx++) {      \
            int64_t idx_1 = (thread_idx * 2) << u;                             \
            int64_t idx_2 = (thread_idx * 2 + 1) << u;                         \
            if (best_dist[idx_1] > best_dist[idx_2]) {                         \
              best_dist[idx_1] = best_dist[idx_2];                             \
              best_dist_idx[idx_1] = best_dist_idx[idx_2];                     \
            }                                                                  \
          }                                                                    \
        }                                                                      \
        out[n_x] = best_dist_idx[0];                                           \
      }                                                                        \
      free(best_dist);                                                         \
      free(best_dist_idx);                                                     \
    }                                                                          \
    return bad;                                                                \
  }

/* mode: fma_mode for the float and double versions */
DEFINE_NEAREST(f32, float, float, sqdist_f32(x, y, n_x, n_y, dim, mode),
               (float)1e38)
DEFINE_NEAREST(f64, double, double, sqdist_f64(x, y, n_x, n_y, dim, mode),
               (double)1e38)

/* ------------------------------------------------------------------------
 * 16-bit element types (IEEE half, bfloat16).
 *
 * In the reference's kernels `scalar_t` is c10::Half / c10::BFloat16, whose
 * arithmetic operators convert to float, operate, and round the result back
 * to 16 bits (torch/headeronly/util/Half.h:501-560, BFloat16.h): every
 * `x - y`, every product and every `+=` of knn_kernel / radius_kernel rounds
 * once, and nothing is fused.  The functions below restate exactly that:
 * values are carried as floats that are representable in the 16-bit type.
 * kind: 0 = IEEE half, 1 = bfloat16.
 * ------------------------------------------------------------------------ */

static float half_bits_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int shift = 0;
      while (!(man & 0x400u)) {
        man <<= 1;
        shift++;
      }
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* float -> nearest half (ties to even) -> float */
static float round_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = x & 0x80000000u;
  uint32_t ax = x & 0x7fffffffu;
  uint16_t h;
  if (ax > 0x7f800000u) { /* NaN */
    h = 0x7e00u;
  } else if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    h = 0x7c00u;
  } else if (ax < 0x33000001u) { /* below half of the smallest subnormal */
    h = 0;
  } else if (ax < 0x38800000u) { /* subnormal half */
    int e = (int)(ax >> 23);          /* biased float exponent */
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    int shift = 126 - e;              /* bits dropped below 2^-24 */
    uint32_t kept = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1u)))
      kept++;
    h = (uint16_t)kept;
  } else {
    uint32_t man = ax & 0x7fffffu;
    uint32_t e = (ax >> 23) - 127 + 15;
    uint32_t kept = (e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (kept & 1u)))
      kept++;
    h = (uint16_t)kept;
  }
  float r = half_bits_to_float(h);
  uint32_t rb;
  memcpy(&rb, &r, 4);
  rb |= sign;
  memcpy(&r, &rb, 4);
  return r;
}

static float bf16_bits_to_float(uint16_t b) {
  uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* float -> nearest bfloat16 (ties to even) -> float */
static float round_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) {
    x = 0x7fc00000u;
  } else {
    x += 0x7fffu + ((x >> 16) & 1u);
    x &= 0xffff0000u;
  }
  memcpy(&f, &x, 4);
  return f;
}

static float load16(const uint16_t *p, int64_t i, int kind) {
  return kind ? bf16_bits_to_float(p[i]) : half_bits_to_float(p[i]);
}

static float round16(float v, int kind) {
  return kind ? round_to_bf16(v) : round_to_half(v);
}

float oracle_round16(float v, int kind) { return round16(v, kind); }

static float sqdist16(const uint16_t *x, const uint16_t *y, int64_t n_x,
                      int64_t n_y, int64_t dim, int kind) {
  float acc = 0;
  for (int64_t d = 0; d < dim; d++) {
    float diff = round16(
        load16(x, n_x * dim + d, kind) - load16(y, n_y * dim + d, kind), kind);
    float prod = round16(diff * diff, kind);
    acc = round16(acc + prod, kind);
  }
  return acc;
}

static float dot16(const uint16_t *a, const uint16_t *b, int64_t n_a,
                   int64_t n_b, int64_t size, int kind) {
  float result = 0;
  for (int64_t i = 0; i < size; i++) {
    float prod = round16(
        load16(a, n_a * size + i, kind) * load16(b, n_b * size + i, kind),
        kind);
    result = round16(result + prod, kind);
  }
  return result;
}

static float norm16(const uint16_t *a, int64_t n_a, int64_t size, int kind) {
  return round16(sqrtf(dot16(a, a, n_a, n_a, size, kind)), kind);
}

/* knn_kernel with a 16-bit scalar_t; dist (optional) receives the distances
 * as floats holding 16-bit-representable values. */
int oracle_knn_dense_16(const uint16_t *x, const uint16_t *y,
                        const int64_t *ptr_x, const int64_t *ptr_y, int64_t n,
                        int64_t m, int64_t dim, int64_t num_examples,
                        int64_t k, int cosine, int kind, int64_t *row,
                        int64_t *col, float *dist) {
  int64_t default_ptr_x[2] = {0, n}, default_ptr_y[2] = {0, m};
  if (ptr_x == NULL || ptr_y == NULL) {
    ptr_x = default_ptr_x;
    ptr_y = default_ptr_y;
    num_examples = 1;
  }
  if (k <= 0)
    return 1;
  const float sentinel = round16(1e10f, kind); /* half: +inf */
#pragma omp parallel
  {
    float *best_dist = (float *)malloc(sizeof(float) * (size_t)k);
    int64_t *best_idx = (int64_t *)malloc(sizeof(int64_t) * (size_t)k);
#pragma omp for schedule(dynamic, 64)
    for (int64_t n_y = 0; n_y < m; n_y++) {
      int64_t b = example_idx(n_y, ptr_y, num_examples);
      for (int64_t e = 0; e < k; e++) {
        best_dist[e] = sentinel;
        best_idx[e] = -1;
      }
      for (int64_t n_x = ptr_x[b]; n_x < ptr_x[b + 1]; n_x++) {
        float tmp_dist;
        if (cosine) {
          float den = round16(norm16(x, n_x, dim, kind) *
                                  norm16(y, n_y, dim, kind),
                              kind);
          tmp_dist =
              round16(dot16(x, y, n_x, n_y, dim, kind) / den, kind);
          /* `1. - tmp_dist`: double arithmetic, narrowed through float */
          tmp_dist = round16((float)(1. - (double)tmp_dist), kind);
        } else {
          tmp_dist = sqdist16(x, y, n_x, n_y, dim, kind);
        }
        for (int64_t e1 = 0; e1 < k; e1++) {
          if (best_dist[e1] > tmp_dist) {
            for (int64_t e2 = k - 1; e2 > e1; e2--) {
              best_dist[e2] = best_dist[e2 - 1];
              best_idx[e2] = best_idx[e2 - 1];
            }
            best_dist[e1] = tmp_dist;
            best_idx[e1] = n_x;
            break;
          }
        }
      }
      for (int64_t e = 0; e < k; e++) {
        row[n_y * k + e] = n_y;
        col[n_y * k + e] = best_idx[e];
        if (dist)
          dist[n_y * k + e] = best_dist[e];
      }
    }
    free(best_dist);
    free(best_idx);
  }
  return 0;
}

/* radius_kernel with a 16-bit scalar_t; r2 = (scalar_t)(r * r) as a float. */
int oracle_radius_dense_16(const uint16_t *x, const uint16_t *y,
                           const int64_t *ptr_x, const int64_t *ptr_y,
                           int64_t n, int64_t m, int64_t dim,
                           int64_t num_examples, float r2,
                           int64_t max_num_neighbors, int ignore_same_index,
                           int kind, int64_t *row, int64_t *col) {
  int64_t default_ptr_x[2] = {0, n}, default_ptr_y[2] = {0, m};
  if (ptr_x == NULL || ptr_y == NULL) {
    ptr_x = default_ptr_x;
    ptr_y = default_ptr_y;
    num_examples = 1;
  }
  if (max_num_neighbors <= 0)
    return 1;
  for (int64_t i = 0; i < m * max_num_neighbors; i++) {
    row[i] = -1;
    col[i] = -1;
  }
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t n_y = 0; n_y < m; n_y++) {
    int64_t count = 0;
    int64_t b = example_idx(n_y, ptr_y, num_examples);
    for (int64_t n_x = ptr_x[b]; n_x < ptr_x[b + 1]; n_x++) {
      float d = sqdist16(x, y, n_x, n_y, dim, kind);
      if (d < r2 && !(ignore_same_index && n_y == n_x)) {
        row[n_y * max_num_neighbors + count] = n_y;
        col[n_y * max_num_neighbors + count] = n_x;
        count++;
      }
      if (count >= max_num_neighbors)
        break;
    }
  }
  return 0;
}

/* nearest_kernel with scalar_t = c10::Half (mode: kind, 0 = IEEE half; the
 * reference does not instantiate it for bfloat16, csrc/cuda/nearest_cuda.cu:
 * 87); `best = 1e38` narrows to +inf. */
DEFINE_NEAREST(16, float, uint16_t, sqdist16(x, y, n_x, n_y, dim, mode),
               round16(1e38f, mode))

/* ------------------------------------------------------------------------
 * fps_kernel (csrc/cuda/fps_cuda.cu:10-66): farthest point sampling, one block
 * of FPS_THREADS threads per example.  out[out_ptr[b]] is the start row
 * (:26-28); for every further sample the threads update the running minimum
 * distance of their rows n = start + t, start + t + 256, ... to the last
 * sample (`dist`, initialised to 5e4 by the host wrapper, :91; squared
 * distance by `dd += tmp * tmp` per dimension) and keep the first strictly
 * larger value, `best` starting at -1 and `best_idx` at 0 (:32-47); the block
 * then takes, in rounds i = 1, 2, 4, .., 128, for every t with t + i < 256
 * the entry t + i when it is strictly larger (:52-59).  Within a round the
 * reference's threads read and write the shared arrays without a barrier in
 * between; the rounds are played here with all reads before all writes (the
 * race-free reading, which is also what a block running in lock step does).
 * `min(dist[n], dd)` is fmin (a NaN distance leaves `dist` as it is and is
 * never `> best`).
 * ------------------------------------------------------------------------ */
#define FPS_THREADS 256

#define DEFINE_FPS(SUFFIX, T, XT, DIST_EXPR, MIN_EXPR, INIT_EXPR)              \
  int oracle_fps_##SUFFIX(const XT *src, const int64_t *ptr,                   \
                          const int64_t *out_ptr, const int64_t *start,        \
                          int64_t n_rows, int64_t dim, int64_t batch_size,     \
                          int mode, int64_t *out) {                            \
    T *dist = (T *)malloc(sizeof(T) * (size_t)(n_rows > 0 ? n_rows : 1));      \
    for (int64_t i = 0; i < n_rows; i++)                                       \
      dist[i] = (INIT_EXPR);                                                   \
    _Pragma("omp parallel for schedule(dynamic, 1)") for (                     \
        int64_t batch_idx = 0; batch_idx < batch_size; batch_idx++) {          \
      T best_dist[FPS_THREADS], next_dist[FPS_THREADS];                        \
      int64_t best_dist_idx[FPS_THREADS], next_idx[FPS_THREADS];               \
      const int64_t start_idx = ptr[batch_idx];                                \
      const int64_t end_idx = ptr[batch_idx + 1];                              \
      if (out_ptr[batch_idx] >= out_ptr[batch_idx + 1])                        \
        continue; /* (the reference writes one entry even then) */             \
      out[out_ptr[batch_idx]] = start_idx + start[batch_idx];                  \
      for (int64_t m = out_ptr[batch_idx] + 1; m < out_ptr[batch_idx + 1];     \
           m++) {                                                              \
        const int64_t old = out[m - 1];                                        \
        for (int64_t thread_idx = 0; thread_idx < FPS_THREADS; thread_idx++) { \
          T best = (T)-1.;                                                     \
          int64_t best_idx = 0;                                                \
          for (int64_t n = start_idx + thread_idx; n < end_idx;                \
               n += FPS_THREADS) {                                             \
            T dd = (DIST_EXPR);                                                \
            dd = (MIN_EXPR);                                                   \
            dist[n] = dd;                                                      \
            if (dd > best) {                                                   \
              best = dd;                                                       \
              best_idx = n;                                                    \
            }                                                                  \
          }                                                                    \
          best_dist[thread_idx] = best;                                        \
          best_dist_idx[thread_idx] = best_idx;                                \
        }                                                                      \
        for (int64_t i = 1; i < FPS_THREADS; i *= 2) {                         \
          for (int64_t t = 0; t < FPS_THREADS; t++) {                          \
            next_dist[t] = best_dist[t];                                       \
            next_idx[t] = best_dist_idx[t];                                    \
            if ((t + i) < FPS_THREADS && best_dist[t] < best_dist[t + i]) {    \
              next_dist[t] = best_dist[t + i];                                 \
              next_idx[t] = best_dist_idx[t + i];                              \
            }                                                                  \
          }                                                                    \
          memcpy(best_dist, next_dist, sizeof(best_dist));                     \
          memcpy(best_dist_idx, next_idx, sizeof(best_dist_idx));              \
        }                                                                      \
        out[m] = best_dist_idx[0];                                             \
      }                                                                        \
    }                                                                          \
    free(dist);                                                                \
    return 0;                                                                  \
  }

/* mode: fma_mode (float, double) or the 16-bit kind (0 = IEEE half) */
DEFINE_FPS(f32, float, float, sqdist_f32(src, src, old, n, dim, mode),
           fminf(dist[n], dd), (float)5e4)
DEFINE_FPS(f64, double, double, sqdist_f64(src, src, old, n, dim, mode),
           fmin(dist[n], dd), (double)5e4)
DEFINE_FPS(16, float, uint16_t, sqdist16(src, src, old, n, dim, mode),
           fminf(dist[n], dd), round16(5e4f, mode))

/* Host-wrapper epilogue: keep the slots whose `mask_src` entry is not -1, in
 * slot order, and stack them as [2, E] (row-major, leading dimension E).
 * Returns E; writes nothing when out is NULL. */
int64_t oracle_compact(const int64_t *row, const int64_t *col,
                       const int64_t *mask_src, int64_t slots, int64_t *out,
                       int64_t capacity) {
  int64_t e = 0;
  for (int64_t i = 0; i < slots; i++)
    e += mask_src[i] != -1;
  if (out == NULL || e > capacity)
    return e;
  int64_t j = 0;
  for (int64_t i = 0; i < slots; i++) {
    if (mask_src[i] != -1) {
      out[j] = row[i];
      out[e + j] = col[i];
      j++;
    }
  }
  return e;
}
