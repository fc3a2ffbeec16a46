// Division by a number known when the kernel is launched.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace amos {

// n / d for 0 <= n < 2^31 with a host-built multiplier: two scalar (or vector) instructions
// where a hardware-less integer division costs dozens
struct FastDiv {
  uint32_t magic, shift, one;
};
inline FastDiv make_fast_div(uint32_t d) {
  FastDiv f = {0, 0, 0};
  if (d <= 1) { f.one = 1; return f; }
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;               // ceil(log2 d), >= 1
  const uint64_t s = 31 + l;
  f.magic = (uint32_t)(((1ull << s) + d - 1) / d);   // ceil(2^s / d) < 2^32
  f.shift = (uint32_t)(s - 32);
  return f;
}
// (branch-free: a branch per division would keep the scalar loads of the kernel arguments from
// being issued together, and each then costs its full latency)
__device__ __forceinline__ int fast_div(int n, const FastDiv& f) {
  return (int)((__umulhi((unsigned)n, f.magic) + (unsigned)n * f.one) >> f.shift);
}

}  // namespace amos
