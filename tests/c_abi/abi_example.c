/* The C ABI used from plain C, with nothing but the HIP runtime: what a non-Python host of the library looks like.
 * Builds a small ragged problem on the host, runs rd_sched_map, rd_gmm and rd_tgmm on the device, and checks the
 * results against triple loops (bit-exact for the map, 1e-2 * max|ref| for the products).
 *
 *   make -C gpu_ragged_dot_amd/csrc abi_example        (built by `all`; binary: tests/c_abi/abi_example)
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/ragged_dot_hip.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); return 2; } } while (0)
#define CHECK_RD(x) do { int s_ = (x); if (s_ != RD_OK) { printf("%s: status %d: %s\n", #x, s_, rd_last_error()); return 3; } } while (0)

static uint16_t to_bf16(float f) {  /* round to nearest even */
  uint32_t u; memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
static float frand(uint32_t* s) { *s = *s * 1664525u + 1013904223u; return ((*s >> 8) & 0xffff) / 32768.0f - 1.0f; }

int main(void) {
  enum { M = 300, K = 64, N = 72, G = 3, CHUNK = 128 };
  const int32_t gs[G] = {130, 0, 150}; /* 20 rows past sum(group_sizes), one empty group */
  static uint16_t x[M * K], A[G * K * N], dy[M * N], y[M * N], dA[G * K * N];
  static float yref[M * N], dAref[G * K * N];
  uint32_t seed = 1;
  for (int i = 0; i < M * K; ++i) x[i] = to_bf16(frand(&seed));
  for (int i = 0; i < G * K * N; ++i) A[i] = to_bf16(frand(&seed) / 8);
  for (int i = 0; i < M * N; ++i) dy[i] = to_bf16(frand(&seed));

  /* reference on the host */
  int off[G + 1]; off[0] = 0;
  for (int g = 0; g < G; ++g) off[g + 1] = off[g] + gs[g];
  float ymax = 0, amax = 0;
  for (int g = 0; g < G; ++g)
    for (int r = off[g]; r < off[g + 1]; ++r)
      for (int c = 0; c < N; ++c) {
        float s = 0;
        for (int kk = 0; kk < K; ++kk) s += from_bf16(x[r * K + kk]) * from_bf16(A[(g * K + kk) * N + c]);
        yref[r * N + c] = s; if (fabsf(s) > ymax) ymax = fabsf(s);
      }
  for (int g = 0; g < G; ++g)
    for (int kk = 0; kk < K; ++kk)
      for (int c = 0; c < N; ++c) {
        float s = 0;
        for (int r = off[g]; r < off[g + 1]; ++r) s += from_bf16(x[r * K + kk]) * from_bf16(dy[r * N + c]);
        dAref[(g * K + kk) * N + c] = s; if (fabsf(s) > amax) amax = fabsf(s);
      }

  void *dx, *dAw, *ddy, *dyo, *ddA, *dgs, *ws;
  CHECK_HIP(hipMalloc(&dx, sizeof x)); CHECK_HIP(hipMalloc(&dAw, sizeof A)); CHECK_HIP(hipMalloc(&ddy, sizeof dy));
  CHECK_HIP(hipMalloc(&dyo, sizeof y)); CHECK_HIP(hipMalloc(&ddA, sizeof dA)); CHECK_HIP(hipMalloc(&dgs, sizeof gs));
  CHECK_HIP(hipMemcpy(dx, x, sizeof x, hipMemcpyHostToDevice)); CHECK_HIP(hipMemcpy(dAw, A, sizeof A, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(ddy, dy, sizeof dy, hipMemcpyHostToDevice)); CHECK_HIP(hipMemcpy(dgs, gs, sizeof gs, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemset(dyo, 0xff, sizeof y)); CHECK_HIP(hipMemset(ddA, 0xff, sizeof dA)); /* outputs arrive uninitialised */

  if (rd_abi_version() != RD_ABI_VERSION) { printf("ABI version %d, header %d\n", rd_abi_version(), RD_ABI_VERSION); return 4; }

  /* scheduling map */
  const int U = rd_sched_map_len(M, G, CHUNK);
  int32_t *d_off, *d_t2g, *d_t2it, *d_tot;
  CHECK_HIP(hipMalloc((void**)&d_off, G * 4)); CHECK_HIP(hipMalloc((void**)&d_t2g, U * 4));
  CHECK_HIP(hipMalloc((void**)&d_t2it, U * 4)); CHECK_HIP(hipMalloc((void**)&d_tot, 4));
  CHECK_RD(rd_sched_map(NULL, (const int32_t*)dgs, G, M, CHUNK, d_off, d_t2g, d_t2it, d_tot));
  int32_t h_off[G], h_t2g[16], h_t2it[16], h_tot;
  CHECK_HIP(hipMemcpy(h_off, d_off, G * 4, hipMemcpyDeviceToHost)); CHECK_HIP(hipMemcpy(h_t2g, d_t2g, U * 4, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(h_t2it, d_t2it, U * 4, hipMemcpyDeviceToHost)); CHECK_HIP(hipMemcpy(&h_tot, d_tot, 4, hipMemcpyDeviceToHost));
  /* by hand: tiles per group ceil(130/128)=2, 0, ceil(150/128)=2; U = ceil(300/128)+3 = 6 */
  const int32_t want_g[6] = {0, 0, 2, 2, 0, 0}, want_it[6] = {0, 1, 0, 1, 0, 0};
  if (U != 6 || h_tot != 4 || h_off[0] != 0 || h_off[1] != 130 || h_off[2] != 130 || memcmp(h_t2g, want_g, 24) || memcmp(h_t2it, want_it, 24)) {
    printf("scheduling map differs\n"); return 5;
  }

  /* the two products, library defaults (plan = NULL) */
  size_t ws_bytes = rd_gmm_workspace_bytes(M, G, NULL);
  if (rd_tgmm_workspace_bytes(M, G, NULL) > ws_bytes) ws_bytes = rd_tgmm_workspace_bytes(M, G, NULL);
  CHECK_HIP(hipMalloc(&ws, ws_bytes));
  CHECK_RD(rd_gmm(NULL, dx, dAw, (const int32_t*)dgs, dyo, M, K, N, G, 0, RD_DTYPE_BF16, NULL, ws, ws_bytes));
  CHECK_RD(rd_tgmm(NULL, dx, ddy, (const int32_t*)dgs, ddA, M, K, N, G, RD_DTYPE_BF16, NULL, ws, ws_bytes));
  CHECK_HIP(hipDeviceSynchronize());
  CHECK_HIP(hipMemcpy(y, dyo, sizeof y, hipMemcpyDeviceToHost)); CHECK_HIP(hipMemcpy(dA, ddA, sizeof dA, hipMemcpyDeviceToHost));

  float ydiff = 0, adiff = 0;
  for (int r = 0; r < M; ++r)
    for (int c = 0; c < N; ++c) {
      const float got = from_bf16(y[r * N + c]);
      if (r >= off[G]) { if (y[r * N + c] != 0) { printf("row %d past sum(group_sizes) is not zero\n", r); return 6; } continue; }
      if (fabsf(got - yref[r * N + c]) > ydiff) ydiff = fabsf(got - yref[r * N + c]);
    }
  for (int i = 0; i < G * K * N; ++i) {
    const int g = i / (K * N);
    if (gs[g] == 0) { if (dA[i] != 0) { printf("slice of the empty group is not zero\n"); return 7; } continue; }
    if (fabsf(from_bf16(dA[i]) - dAref[i]) > adiff) adiff = fabsf(from_bf16(dA[i]) - dAref[i]);
  }
  printf("y: max|diff| %.4g (max|ref| %.4g)   dA: max|diff| %.4g (max|ref| %.4g)\n", ydiff, ymax, adiff, amax);
  if (ydiff > 1e-2f * ymax || adiff > 1e-2f * amax) { printf("outside 1e-2 * max|ref|\n"); return 8; }

  /* error channel: a negative status and a message, no abort */
  if (rd_gmm(NULL, dx, dAw, (const int32_t*)dgs, dyo, -1, K, N, G, 0, RD_DTYPE_BF16, NULL, ws, ws_bytes) != RD_ERR_INVALID_ARGUMENT ||
      strlen(rd_last_error()) == 0) { printf("bad-shape call was not rejected\n"); return 9; }
  printf("abi_example ok\n");
  return 0;
}
