// Developer probe, not part of the library: where the cycles of the ping-pong K loop go.
//
// rd_gemm_pp.h calls RD_MARK(id) at the phase boundaries of gemm_tile_pingpong_mixed (empty macros in the library).
// Here they accumulate shader-clock deltas per wave for one chosen work-group of a Mixtral-shaped forward launch:
//   0 memory phase, 1 barrier after it, 2 compute phase, 3 barrier after it, 4 after the last barrier, 5 epilogue.
// Each mark costs a few tens of cycles itself, so read the numbers as proportions.
//
//   make -C gpu_ragged_dot_amd/csrc probe_phase_times
//   gpu_ragged_dot_amd/csrc/build/probe_phase_times [zeros=0|1] [work-group index]
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <algorithm>
#include <vector>

__device__ unsigned long long* g_marks;  // [8 waves][8]
__device__ int g_marked_block;
#define RD_MARK_DECL                                                                   \
  const bool rd_mark_on = ((int)blockIdx.x == g_marked_block);                         \
  unsigned long long rd_mark_last = __builtin_readcyclecounter(), rd_mark_sum[6] = {0, 0, 0, 0, 0, 0}; \
  const unsigned long long rd_mark_start = rd_mark_last
#define RD_MARK(id)                                                                    \
  do {                                                                                 \
    if (rd_mark_on) {                                                                  \
      const unsigned long long now_ = __builtin_readcyclecounter();                    \
      rd_mark_sum[(id)] += now_ - rd_mark_last;                                        \
      rd_mark_last = now_;                                                             \
      if ((id) == 5 && (threadIdx.x & 63) == 0) {                                      \
        unsigned long long* p_ = g_marks + (threadIdx.x >> 6) * 8;                     \
        for (int q_ = 0; q_ < 6; ++q_) p_[q_] = rd_mark_sum[q_];                       \
        p_[6] = now_ - rd_mark_start;                                                  \
      }                                                                                \
    }                                                                                  \
  } while (0)
#include "rd_kernels.h"
#include "rd_sched.h"

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); return 1; } } while (0)

typedef rd::PpCfg<256, 256, 2, 4, true, false, 64, 3, 32, 4> Cfg;  // the forward kernel of the 256 x 256 per-operand-ring variant

int main(int argc, char** argv) {
  const int m = 16384, k = 4096, n = 14336, g = 8;
  const int zeros = argc > 1 ? atoi(argv[1]) : 0;
  const int block = argc > 2 ? atoi(argv[2]) : 2000;
  const std::vector<int32_t> gs = {2012, 2069, 2038, 2100, 2032, 2052, 2039, 2042};
  uint16_t *x, *A, *y; int32_t *dgs, *ws;
  CK(hipMalloc(&x, (size_t)m * k * 2)); CK(hipMalloc(&A, (size_t)g * k * n * 2)); CK(hipMalloc(&y, (size_t)m * n * 2));
  CK(hipMalloc(&dgs, g * 4)); CK(hipMalloc(&ws, 1 << 20));
  CK(hipMemcpy(dgs, gs.data(), g * 4, hipMemcpyHostToDevice));
  if (zeros) {
    CK(hipMemset(x, 0, (size_t)m * k * 2)); CK(hipMemset(A, 0, (size_t)g * k * n * 2));
  } else {  // bf16 values of magnitude 1..2 with random sign and mantissa
    std::vector<uint16_t> h((size_t)k * n);
    for (auto& v : h) v = (uint16_t)((0x3f80 + (rand() & 0x7f)) ^ ((rand() & 1) << 15));
    for (int gi = 0; gi < g; ++gi) CK(hipMemcpy(A + (size_t)gi * k * n, h.data(), h.size() * 2, hipMemcpyHostToDevice));
    for (size_t off = 0; off < (size_t)m * k; off += h.size())
      CK(hipMemcpy(x + off, h.data(), std::min(h.size(), (size_t)m * k - off) * 2, hipMemcpyHostToDevice));
  }
  unsigned long long* marks;
  CK(hipMalloc(&marks, 64 * 8)); CK(hipMemset(marks, 0, 64 * 8));
  CK(hipMemcpyToSymbol(HIP_SYMBOL(g_marks), &marks, sizeof(marks)));
  const int U = (m + 255) / 256 + g;
  int32_t *off = ws, *t2g = ws + g, *t2it = ws + g + U, *tot = ws + g + 2 * U;
  rd::GmmArgs a{};
  a.x = x; a.A = A; a.y = y; a.group_sizes = dgs; a.group_offsets = off; a.tile2group = t2g; a.tile2it = t2it; a.total_tiles = tot;
  a.m = m; a.k = k; a.n = n; a.g = g; a.U = U; a.n_tiles = (n + 255) / 256; a.group_m = 4; a.group_n = 8;
  a.num_cus = 256;
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  for (int rep = 0; rep < 30; ++rep) {
    const int b = rep == 29 ? block : -1;  // only the last launch is marked
    CK(hipMemcpyToSymbol(HIP_SYMBOL(g_marked_block), &b, sizeof(int)));
    rd::launch_sched_map(0, dgs, g, m, 256, off, t2g, t2it, tot);
    CK(hipEventRecord(e0));
    const int rc = rd::launch_gmm<Cfg, false>(0, a);
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    if (rep >= 27) printf("launch %d rc %d %.3f ms %.1f TFLOP/s\n", rep, rc, ms, 2.0 * m * k * n / ms / 1e9);
  }
  std::vector<unsigned long long> h(64);
  CK(hipMemcpy(h.data(), marks, 64 * 8, hipMemcpyDeviceToHost));
  const double phases = k / 32;
  printf("cycles per 32-wide phase (%d phases; 16 MFMA = 512 cycles of matrix-core work per wave and phase)\n", k / 32);
  for (int w = 0; w < 8; ++w) {
    const unsigned long long* p = &h[w * 8];
    printf("wave %d: memory %5.0f  barrier %4.0f  compute %5.0f  barrier %4.0f | after loop %llu  epilogue %llu  tile %llu\n", w,
           p[0] / phases, p[1] / phases, p[2] / phases, p[3] / phases, p[4], p[5], p[6]);
  }
  return 0;
}
