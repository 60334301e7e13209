// Launcher of the skinny-m ("decode") forward kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rd {

struct DecodeArgs {
  const uint16_t* x;   // [m, k] bf16
  const uint16_t* A;   // [g, k, n] bf16
  uint16_t* y;         // [m, n] bf16
  const int32_t* group_sizes;
  int m, k, n, g;
};

// nb: columns per work-group (32, 64 or 128).  Needs k % 8 == 0, n % 8 == 0 and k <= kDecodeMaxK.
constexpr int kDecodeMaxK = 16384;
int launch_gmm_decode(hipStream_t s, const DecodeArgs& a, int nb);

}  // namespace rd
