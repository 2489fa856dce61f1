// Unsigned 32-bit division by a run-time constant with one multiply-high and two shifts
// (Granlund-Montgomery): q = (t + ((n - t) >> s1)) >> s2 with t = mulhi(m, n).  Exact for
// every 32-bit n.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace tsplit {

struct FastDiv {
  uint32_t d, m, s1, s2;
  __host__ __device__ FastDiv(uint32_t div = 1) : d(div) {
    uint32_t l = 0;
    while ((1ull << l) < div) ++l;
    m = static_cast<uint32_t>(((1ull << 32) * ((1ull << l) - div)) / div + 1);
    s1 = l < 1 ? l : 1;
    s2 = l > 1 ? l - 1 : 0;
  }
  __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
#ifdef __HIP_DEVICE_COMPILE__
    const uint32_t t = __umulhi(m, n);
#else
    const uint32_t t = static_cast<uint32_t>((static_cast<uint64_t>(m) * n) >> 32);
#endif
    return (t + ((n - t) >> s1)) >> s2;
  }
};

}  // namespace tsplit
