// Developer probe, not part of the library: what the matrix cores sustain under the chip's power limit when nothing
// else runs.  One wave per SIMD on every compute unit issues back-to-back independent bf16 MFMAs on fragments held in
// registers - no LDS, no memory traffic inside the loop - for about half a second per case, on all-zero operands,
// on uniform random operands in (-2, 2) and on all-one operands, with v_mfma_f32_32x32x16_bf16 and with
// v_mfma_f32_16x16x32_bf16.  The random-operand figure is the ceiling a GEMM on such data can approach on this part
// however its data movement is arranged.  A second kernel then adds, per 32 MFMAs, what the four-wave GEMM core issues
// per K-slab - 16 ds_read_b128 of fragments, 8 direct-to-LDS loads of 1 KB (from a 64 KB window per work-group, i.e.
// always L2 hits) and one barrier - to show what each of them costs under the power limit.
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
typedef __attribute__((address_space(3))) void* lds_void_ptr;
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); exit(1); } } while (0)

constexpr int kSrcVectors = 1 << 20;  // 16-byte vectors of operand data
constexpr int kBlocks = 256, kThreads = 256;
constexpr int kRegion = 64 * 1024;  // bytes of global data per work-group that the direct loads cycle through

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

// 32 MFMAs of 32x32x16 per iteration in two halves, as the four-wave core runs a K-slab; optionally with its LDS
// fragment reads (LDSR: into the fragment set the other half uses), its direct-to-LDS loads (DMA) and its barrier (BAR).
template <bool LDSR, bool DMA, bool BAR>
__global__ __launch_bounds__(kThreads, 1) void mix(const uint4* __restrict__ src, const unsigned char* __restrict__ src2, float* __restrict__ out, int iters) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int gtid = blockIdx.x * kThreads + tid;
  for (int i = 0; i < 16; ++i) reinterpret_cast<uint4*>(smem)[tid + 256 * i] = src[(gtid * 16 + i) % kSrcVectors];
  __syncthreads();
  bf16x8 f[2][8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    f[0][i] = __builtin_bit_cast(bf16x8, src[(gtid * 16 + i) % kSrcVectors]);
    f[1][i] = __builtin_bit_cast(bf16x8, src[(gtid * 16 + 8 + i) % kSrcVectors]);
  }
  f32x16 acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(src2 + (size_t)blockIdx.x * kRegion), 0, kRegion, 0x00020000);
  int cnt = __builtin_amdgcn_readfirstlane(tid >> 6) * 16;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        if (LDSR && t < 8) f[h ^ 1][t] = *reinterpret_cast<const bf16x8*>(smem + (((it * 16 + h * 8 + t) & 63) << 10) + lane * 16);
        if (DMA && (t & 3) == 3) {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)(smem + 65536 + ((cnt & 63) << 10)), 16, lane * 16, (cnt & 63) << 10, 0, 0);
          ++cnt;
        }
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[h][t & 3], f[h][4 + (t >> 2)], acc[t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (h == 0) {
        if (DMA) __builtin_amdgcn_s_waitcnt((24 & 0xf) | ((24 >> 4) << 14) | (0x7 << 4) | (0xf << 8));  // vmcnt(24)
        if (BAR) { __builtin_amdgcn_s_waitcnt(0xc07f); __builtin_amdgcn_s_barrier(); }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[i][v];
  if (s == 123.456f) out[gtid] = s;
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
  // ---- the same matrix-core work with the data movement of a K-slab around it --------------------------------------
  unsigned char* d2;
  CHECK(hipMalloc(&d2, (size_t)kBlocks * kRegion));
  static const char* kMix[] = {"MFMA only", "+ 16 ds_read_b128 per 32 MFMA", "+ reads + 8 direct loads per 32 MFMA",
                               "+ reads + loads + barrier", "+ 8 direct loads only"};
  const int mix_iters = 4000;  // 32 MFMAs per iteration
  for (int mode = 0; mode < 2; ++mode) {
    srand(1);
    for (size_t i = 0; i < h.size(); ++i) {
      if (mode == 0) h[i] = 0;
      else { const float f = ((rand() % 2001) - 1000) / 500.0f; uint32_t u; memcpy(&u, &f, 4); h[i] = (uint16_t)(u >> 16); }
    }
    CHECK(hipMemcpy(d, h.data(), (size_t)kSrcVectors * 16, hipMemcpyHostToDevice));
    CHECK(hipMemcpy(d2, h.data(), (size_t)kBlocks * kRegion, hipMemcpyHostToDevice));
    for (int cfg = 0; cfg < 5; ++cfg) {
      void (*kern)(const uint4*, const unsigned char*, float*, int) =
          cfg == 0 ? mix<false, false, false> : cfg == 1 ? mix<true, false, false> : cfg == 2 ? mix<true, true, false>
          : cfg == 3 ? mix<true, true, true> : mix<false, true, false>;
      CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      auto launch = [&]() { hipLaunchKernelGGL(kern, dim3(kBlocks), dim3(kThreads), 160 * 1024, 0, d, d2, o, mix_iters); };
      for (int w = 0; w < 100; ++w) launch();
      CHECK(hipDeviceSynchronize());
      const int reps = 200;
      CHECK(hipEventRecord(e0));
      for (int r = 0; r < reps; ++r) launch();
      CHECK(hipEventRecord(e1));
      CHECK(hipEventSynchronize(e1));
      float ms;
      CHECK(hipEventElapsedTime(&ms, e0, e1));
      const double flops = (double)reps * kBlocks * 4 * mix_iters * 32 * 32768.0;
      printf("operands %-14s %-38s : %7.1f TFLOP/s (%.2f ms per launch)\n", mode == 0 ? "zeros" : "uniform(-2,2)", kMix[cfg],
             flops / (ms * 1e-3) / 1e12, ms / reps);
      fflush(stdout);
    }
  }
  return 0;
}
