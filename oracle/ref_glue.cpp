// TEST INFRASTRUCTURE ONLY -- never linked into or called by the product.
//
// C-ABI glue around the reference's own CPU operators so that tests and the
// CPU-baseline leg of bench.py can call them through ctypes without going
// through the TorchScript operator registry (which the product library also
// registers `torch_cluster::knn` / `torch_cluster::radius` in, so both cannot
// be registered in one process).
//
// This file contains no reference code.  It is compiled together with the
// reference sources where they lie:
//   /root/reference/csrc/cpu/knn_cpu.cpp     (knn_cpu,    :7-105)
//   /root/reference/csrc/cpu/radius_cpu.cpp  (radius_cpu, :7-117)
//   /root/reference/csrc/cpu/fps_cpu.cpp     (fps_cpu,    :13-68)
// whose prototypes come from the reference headers included below
// (csrc/cpu/knn_cpu.h:5-8, csrc/cpu/radius_cpu.h:5-9, csrc/cpu/fps_cpu.h).
#include "cpu/fps_cpu.h"
#include "cpu/knn_cpu.h"
#include "cpu/radius_cpu.h"

#include <cstdint>
#include <cstring>
#include <optional>

namespace {

// dtype codes shared with oracle/oracle.py
at::ScalarType to_scalar_type(int dtype) {
  switch (dtype) {
  case 0:
    return at::kFloat;
  case 1:
    return at::kDouble;
  case 2:
    return at::kHalf;
  case 3:
    return at::kBFloat16;
  default:
    TORCH_CHECK(false, "unknown dtype code ", dtype);
  }
}

torch::Tensor wrap(const void *p, int64_t rows, int64_t cols, int dtype) {
  return torch::from_blob(const_cast<void *>(p), {rows, cols},
                          torch::TensorOptions().dtype(to_scalar_type(dtype)));
}

std::optional<torch::Tensor> wrap_ptr(const int64_t *p, int64_t num_segments) {
  if (p == nullptr)
    return std::nullopt;
  return torch::from_blob(const_cast<int64_t *>(p), {num_segments + 1},
                          torch::TensorOptions().dtype(torch::kLong));
}

// Copies a [2, E] int64 tensor into out (row-major, leading dimension E) when
// it fits; always returns E.
int64_t emit(const torch::Tensor &edges, int64_t *out, int64_t capacity) {
  auto e = edges.contiguous();
  const int64_t E = e.size(1);
  if (out != nullptr && E <= capacity && E > 0)
    std::memcpy(out, e.data_ptr<int64_t>(), sizeof(int64_t) * 2 * E);
  return E;
}

} // namespace

extern "C" {

// Returns E (number of edges) or -1 on a C++ exception.  `out` receives
// row 0 = query (y) index, row 1 = x index, each of length E, back to back.
int64_t ref_knn_cpu(const void *x, const void *y, const int64_t *ptr_x,
                    const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                    int64_t num_segments, int64_t k, int dtype, int64_t *out,
                    int64_t capacity) {
  try {
    auto e = knn_cpu(wrap(x, n, d, dtype), wrap(y, m, d, dtype),
                     wrap_ptr(ptr_x, num_segments),
                     wrap_ptr(ptr_y, num_segments), k, /*num_workers=*/1);
    return emit(e, out, capacity);
  } catch (const std::exception &) {
    return -1;
  }
}

int64_t ref_radius_cpu(const void *x, const void *y, const int64_t *ptr_x,
                       const int64_t *ptr_y, int64_t n, int64_t m, int64_t d,
                       int64_t num_segments, double r,
                       int64_t max_num_neighbors, int ignore_same_index,
                       int dtype, int64_t *out, int64_t capacity) {
  try {
    auto e = radius_cpu(wrap(x, n, d, dtype), wrap(y, m, d, dtype),
                        wrap_ptr(ptr_x, num_segments),
                        wrap_ptr(ptr_y, num_segments), r, max_num_neighbors,
                        /*num_workers=*/1, ignore_same_index != 0);
    return emit(e, out, capacity);
  } catch (const std::exception &) {
    return -1;
  }
}

// fps_cpu with random_start = false; returns the number of samples or -1.
int64_t ref_fps_cpu(const void *src, const int64_t *ptr, int64_t n, int64_t d,
                    int64_t num_segments, double ratio, int dtype,
                    int64_t *out, int64_t capacity) {
  try {
    auto r = torch::tensor(ratio, torch::TensorOptions().dtype(torch::kFloat));
    auto idx = fps_cpu(wrap(src, n, d, dtype), *wrap_ptr(ptr, num_segments), r,
                       /*random_start=*/false)
                   .contiguous();
    const int64_t count = idx.numel();
    if (out != nullptr && count <= capacity && count > 0)
      std::memcpy(out, idx.data_ptr<int64_t>(), sizeof(int64_t) * count);
    return count;
  } catch (const std::exception &) {
    return -1;
  }
}

} // extern "C"
