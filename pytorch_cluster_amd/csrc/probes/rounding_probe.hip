// Every float rounded to bfloat16 by round_to_16<true> and round_in_chain<true>
// (the device's conversion instruction, what the 16-bit searches use) and by
// the integer formula of c10::BFloat16.  Counts the bit patterns on which
// they differ; round_in_chain may answer a NaN with any NaN.
#include "../device_utils.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

// workgroup b takes the 65,536 floats whose upper half is b
__global__ __launch_bounds__(256) void rounding_kernel(
    unsigned long long *differ, uint32_t *first) {
  const uint32_t hi = blockIdx.x;
  unsigned mine = 0;
  for (uint32_t lo = threadIdx.x; lo < 65536u; lo += blockDim.x) {
    const uint32_t bits = (hi << 16) | lo;
    const float v = __uint_as_float(bits);
    const uint32_t want = __float_as_uint(pca::round_to_bf16_by_integers(v));
    const uint32_t chain = __float_as_uint(pca::round_in_chain<true>(v));
    const bool is_nan = (bits & 0x7fffffffu) > 0x7f800000u;
    if (__float_as_uint(pca::round_to_16<true>(v)) != want ||
        (is_nan ? (chain & 0x7fffffffu) <= 0x7f800000u : chain != want)) {
      ++mine;
      atomicMin(first, bits);
    }
  }
  if (mine != 0)
    atomicAdd(differ, (unsigned long long)mine);
}

} // namespace

// out[0]: floats on which the two differ (of 2^32); out[1]: the smallest such
// bit pattern (0xffffffff: none).  Returns 0, or -1 when a HIP call failed.
extern "C" int pca_probe_bf16_rounding(unsigned long long out[2]) {
  unsigned long long *differ = nullptr;
  uint32_t *first = nullptr;
  if (hipMalloc(&differ, 8) != hipSuccess)
    return -1;
  if (hipMalloc(&first, 4) != hipSuccess) {
    (void)hipFree(differ);
    return -1;
  }
  int rc = -1;
  unsigned long long host_differ = 0;
  uint32_t host_first = 0;
  if (hipMemset(differ, 0, 8) == hipSuccess &&
      hipMemset(first, 0xff, 4) == hipSuccess) {
    hipLaunchKernelGGL(rounding_kernel, dim3(65536), dim3(256), 0, 0, differ,
                       first);
    if (hipGetLastError() == hipSuccess &&
        hipMemcpy(&host_differ, differ, 8, hipMemcpyDeviceToHost) ==
            hipSuccess &&
        hipMemcpy(&host_first, first, 4, hipMemcpyDeviceToHost) ==
            hipSuccess) {
      out[0] = host_differ;
      out[1] = host_first;
      rc = 0;
    }
  }
  (void)hipFree(differ);
  (void)hipFree(first);
  return rc;
}
