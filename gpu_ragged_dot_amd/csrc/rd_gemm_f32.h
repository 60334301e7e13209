// fp32 operands: one 64x64 tile of C = sum_kk Aop(i,kk)*Bop(j,kk) on v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate).
// A plain, any-shape routine (element-granular masked loads, single LDS buffer): it exists so that float32 inputs -
// which the reference accepts - give float32-accurate results; the bf16 cores are where the speed is.
#pragma once
#include "rd_common.h"

namespace rd {

template <bool A_KMAJOR_, bool B_KMAJOR_>
struct F32Cfg {
  typedef float Elem;
  static constexpr int BM = 64, BN = 64, BK = 16, WAVES_M = 2, WAVES_N = 2;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, VEC = false, DLDS = false, PINGPONG = false, MIXED = false,
                        SPLITK = false;
  static constexpr bool F32 = true;
  static constexpr int STAGES = 1;
  static constexpr int NT = 256, WAVES_PER_EU = 1;
  static constexpr int PITCH = BK + 1;  // floats per LDS row: odd pitch, conflict-free column reads
  static constexpr int LDS_BYTES = (BM + BN) * PITCH * (int)sizeof(float);
};

// Stage one operand's [64 x 16] slab into LDS as [row][kk], zero outside the tile's limits / the contraction length.
template <bool KMAJOR, int PITCH>
__device__ __forceinline__ void stage_f32(const float* __restrict__ p, int ld, int lim, int k0, int klen, float* lds) {
#pragma unroll
  for (int e = threadIdx.x; e < 64 * 16; e += 256) {
    int i, kk;
    if (KMAJOR) { i = e >> 4; kk = e & 15; }   // consecutive threads walk the contraction index: contiguous in memory
    else { i = e & 63; kk = e >> 6; }           // consecutive threads walk rows of the tile: contiguous in memory
    const bool ok = i < lim && k0 + kk < klen;
    const size_t off = KMAJOR ? (size_t)(ok ? i : 0) * ld + (ok ? k0 + kk : 0) : (size_t)(ok ? k0 + kk : 0) * ld + (ok ? i : 0);
    const float v = p[off];  // always a valid address; masked below
    lds[i * PITCH + kk] = ok ? v : 0.f;
  }
}

template <class C>
__device__ __forceinline__ void gemm_tile_f32(const float* __restrict__ Ap, int lda, int a_lim,
                                              const float* __restrict__ Bp, int ldb, int b_lim, int klen,
                                              float* __restrict__ Op, int ldo, float* smem) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  float* As = smem;
  float* Bs = smem + C::BM * C::PITCH;
  f32x16_t acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;

  for (int k0 = 0; k0 < klen; k0 += C::BK) {
    __syncthreads();  // previous slab fully consumed
    stage_f32<C::A_KMAJOR, C::PITCH>(Ap, lda, a_lim, k0, klen, As);
    stage_f32<C::B_KMAJOR, C::PITCH>(Bp, ldb, b_lim, k0, klen, Bs);
    __syncthreads();
    // v_mfma_f32_32x32x2_f32: lane l feeds row/column (l & 31), contraction element (l >> 5) of each pair
#pragma unroll
    for (int s = 0; s < C::BK / 2; ++s) {
      const float a = As[(wm * 32 + (lane & 31)) * C::PITCH + 2 * s + (lane >> 5)];
      const float b = Bs[(wn * 32 + (lane & 31)) * C::PITCH + 2 * s + (lane >> 5)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
  }
  const int col = wn * 32 + (lane & 31);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = wm * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
    if (row < a_lim && col < b_lim) Op[(size_t)row * ldo + col] = acc[v];
  }
}

}  // namespace rd
