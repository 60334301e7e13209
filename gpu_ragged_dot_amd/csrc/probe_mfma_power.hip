// Developer probe, not part of the library: what the matrix cores sustain under the chip's power limit when nothing
// else runs.  One wave per SIMD on every compute unit issues back-to-back independent bf16 MFMAs on fragments held in
// registers - no LDS, no memory traffic inside the loop - for about half a second per case, on all-zero operands,
// on uniform random operands in (-2, 2) and on all-one operands, with v_mfma_f32_32x32x16_bf16 and with
// v_mfma_f32_16x16x32_bf16.  The random-operand figure is the ceiling a GEMM on such data can approach on this part
// however its data movement is arranged.
//
//   make -C gpu_ragged_dot_amd/csrc probe_mfma_power
//   gpu_ragged_dot_amd/csrc/build/probe_mfma_power
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); exit(1); } } while (0)

constexpr int kSrcVectors = 1 << 20;  // 16-byte vectors of operand data
constexpr int kBlocks = 256, kThreads = 256;

// SHAPE 32: 16 accumulators of 32x32; SHAPE 16: 64 accumulators of 16x16 - both fill the 256 accumulator registers and
// do 2 x 16 x 32768 FLOP per wave and pair of iterations.
template <int SHAPE>
__global__ __launch_bounds__(kThreads, 1) void mfma_loop(const uint4* __restrict__ src, float* __restrict__ out, int iters) {
  bf16x8 a[8], b[8];
  const int tid = blockIdx.x * kThreads + threadIdx.x;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = __builtin_bit_cast(bf16x8, src[(tid * 16 + i) % kSrcVectors]);
    b[i] = __builtin_bit_cast(bf16x8, src[(tid * 16 + 8 + i) % kSrcVectors]);
  }
  float s = 0.f;
  if (SHAPE == 32) {
    f32x16 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    for (int it = 0; it < iters; it += 2) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i + 4 * h], b[j + 4 * h], acc[i * 4 + j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) s += acc[i][v];
  } else {
    f32x4 acc[64];
#pragma unroll
    for (int i = 0; i < 64; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][v] = 0.f;
    for (int it = 0; it < iters; it += 2) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i * 8 + j + 4 * h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j + 4 * h], acc[i * 8 + j + 4 * h], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 64; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) s += acc[i][v];
  }
  if (s == 123.456f) out[tid] = s;  // keeps the loop alive; practically never true
}

int main() {
  std::vector<uint16_t> h((size_t)kSrcVectors * 8);
  uint4* d;
  float* o;
  CHECK(hipMalloc(&d, (size_t)kSrcVectors * 16));
  CHECK(hipMalloc(&o, (size_t)kBlocks * kThreads * sizeof(float)));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  const int iters = 8000;  // 16 MFMAs of 32 cycles per iteration: about 2 ms per launch
  static const char* kData[] = {"zeros", "uniform(-2,2)", "ones"};
  for (int mode = 0; mode < 3; ++mode) {
    srand(1);
    for (size_t i = 0; i < h.size(); ++i) {
      if (mode == 0) h[i] = 0;
      else if (mode == 2) h[i] = 0x3f80;
      else { const float f = ((rand() % 2001) - 1000) / 500.0f; uint32_t u; memcpy(&u, &f, 4); h[i] = (uint16_t)(u >> 16); }
    }
    CHECK(hipMemcpy(d, h.data(), (size_t)kSrcVectors * 16, hipMemcpyHostToDevice));
    for (int shape = 0; shape < 2; ++shape) {
      auto launch = [&]() {
        if (shape == 0) hipLaunchKernelGGL(mfma_loop<32>, dim3(kBlocks), dim3(kThreads), 0, 0, d, o, iters);
        else hipLaunchKernelGGL(mfma_loop<16>, dim3(kBlocks), dim3(kThreads), 0, 0, d, o, iters);
      };
      for (int w = 0; w < 100; ++w) launch();  // lets the clock settle under load
      CHECK(hipDeviceSynchronize());
      const int reps = 200;
      CHECK(hipEventRecord(e0));
      for (int r = 0; r < reps; ++r) launch();
      CHECK(hipEventRecord(e1));
      CHECK(hipEventSynchronize(e1));
      float ms;
      CHECK(hipEventElapsedTime(&ms, e0, e1));
      const double flops = (double)reps * kBlocks * 4 * iters * 16 * 32768.0;
      printf("operands %-14s %s : %7.1f TFLOP/s (%.2f ms per launch)\n", kData[mode], shape == 0 ? "32x32x16" : "16x16x32",
             flops / (ms * 1e-3) / 1e12, ms / reps);
      fflush(stdout);
    }
  }
  return 0;
}
