// fp32 operands: one BM x BN tile of C = sum_kk Aop(i,kk)*Bop(j,kk) on v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate),
// so that float32 inputs - which the reference accepts - give float32-accurate results.
//
// Any shape is taken.  Four waves in a 2 x 2 grid, each holding (BM/2) x (BN/2) of the tile in 32 x 32 blocks; the
// contraction runs in slabs of 16 through two LDS buffers: the loads of slab s+1 are issued into registers before the
// MFMAs of slab s and written to the other buffer after them, one barrier per slab.  LDS holds a slab as [kk][row]
// (pitch BM + 4), which is what the MFMA wants lane by lane and lets the row-contiguous operands go in as 16-byte
// stores.  Operands are loaded 16 bytes at a time when the pitch, base address and masked extent of both allow it
// (decided per tile, uniformly), else element by element.
#pragma once
#include "rd_common.h"

namespace rd {

template <int BM_, int BN_, bool A_KMAJOR_, bool B_KMAJOR_>
struct F32Cfg {
  typedef float Elem;
  static constexpr int BM = BM_, BN = BN_, BK = 16, WAVES_M = 2, WAVES_N = 2;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, VEC = false, DLDS = false, PINGPONG = false, MIXED = false,
                        SPLITK = false;
  static constexpr bool F32 = true;
  static constexpr int STAGES = 2;
  static constexpr int NT = 256, WAVES_PER_EU = BM * BN >= 128 * 128 ? 3 : 4;
  static constexpr int PITCH_A = BM + 4, PITCH_B = BN + 4;  // floats per LDS row of one contraction index
  static constexpr int SLAB_FLOATS = BK * (PITCH_A + PITCH_B);
  static constexpr int LDS_BYTES = 2 * SLAB_FLOATS * (int)sizeof(float);
  static_assert(BM % 64 == 0 && BN % 64 == 0, "each wave holds whole 32 x 32 blocks");
};

// One operand's [ROWS x 16] slab, in flight between global memory and LDS: ROWS * 16 / 256 floats per thread.
template <int ROWS>
struct F32Slab {
  static constexpr int N = ROWS * 16 / 256;
  float v[N];
};

// Issue the loads of one slab; `ps` points at the slab (the tile's base advanced along the contraction, wave-uniform),
// `krem` contraction elements remain from there.  Everything outside the tile's limits / the contraction length reads
// as zero.  VEC: 16-byte loads (legal per f32_vec_ok).  In-slab offsets fit 32 bits: at most 128 rows of pitch `ld`.
template <bool KMAJOR, int ROWS, bool VEC>
__device__ __forceinline__ void f32_load(F32Slab<ROWS>& r, const float* __restrict__ ps, int ld, int lim, int krem) {
  constexpr int N = F32Slab<ROWS>::N;
  const int tid = threadIdx.x;
  if constexpr (VEC) {
#pragma unroll
    for (int j = 0; j < N / 4; ++j) {
      const int q = tid + 256 * j;
      int i, kk;
      if (KMAJOR) { i = q >> 2; kk = (q & 3) * 4; }              // four lanes cover the 64 bytes of one row
      else { i = (q % (ROWS / 4)) * 4; kk = q / (ROWS / 4); }    // ROWS/4 lanes cover one contraction index
      const bool ok = i < lim && kk < krem;
      const unsigned off = !ok ? 0u : KMAJOR ? (unsigned)i * ld + kk : (unsigned)kk * ld + i;
      float4 t = *reinterpret_cast<const float4*>(ps + off);  // always a valid address; masked below
      r.v[4 * j + 0] = ok ? t.x : 0.f;
      r.v[4 * j + 1] = ok ? t.y : 0.f;
      r.v[4 * j + 2] = ok ? t.z : 0.f;
      r.v[4 * j + 3] = ok ? t.w : 0.f;
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const int e = tid + 256 * j;
      int i, kk;
      if (KMAJOR) { i = e >> 4; kk = e & 15; }
      else { i = e % ROWS; kk = e / ROWS; }
      const bool ok = i < lim && kk < krem;
      const unsigned off = !ok ? 0u : KMAJOR ? (unsigned)i * ld + kk : (unsigned)kk * ld + i;
      const float t = ps[off];
      r.v[j] = ok ? t : 0.f;
    }
  }
}

// Write a loaded slab to LDS as [kk][row]; the same index arithmetic as f32_load.
template <bool KMAJOR, int ROWS, bool VEC>
__device__ __forceinline__ void f32_store(const F32Slab<ROWS>& r, float* lds) {
  constexpr int N = F32Slab<ROWS>::N, PITCH = ROWS + 4;
  const int tid = threadIdx.x;
  if constexpr (VEC) {
#pragma unroll
    for (int j = 0; j < N / 4; ++j) {
      const int q = tid + 256 * j;
      if (KMAJOR) {
        const int i = q >> 2, kk = (q & 3) * 4;
#pragma unroll
        for (int c = 0; c < 4; ++c) lds[(kk + c) * PITCH + i] = r.v[4 * j + c];
      } else {
        const int i = (q % (ROWS / 4)) * 4, kk = q / (ROWS / 4);
        *reinterpret_cast<float4*>(lds + kk * PITCH + i) = make_float4(r.v[4 * j], r.v[4 * j + 1], r.v[4 * j + 2], r.v[4 * j + 3]);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const int e = tid + 256 * j;
      int i, kk;
      if (KMAJOR) { i = e >> 4; kk = e & 15; }
      else { i = e % ROWS; kk = e / ROWS; }
      lds[kk * PITCH + i] = r.v[j];
    }
  }
}

// 16-byte loads are legal for an operand when its pitch and base keep every vector aligned and no vector straddles
// the masked extent: along the contraction for a K-major operand, along the tile's rows otherwise.
template <bool KMAJOR>
__device__ __forceinline__ bool f32_vec_ok(const float* p, int ld, int lim, int klen) {
  const bool aligned = (ld & 3) == 0 && (reinterpret_cast<uintptr_t>(p) & 15) == 0;
  return aligned && (((KMAJOR ? klen : lim) & 3) == 0);
}

// The contraction loop for one way of loading (both operands by 16 bytes, or both by element).
template <class C, bool VEC, int MI, int NI>
__device__ __forceinline__ void f32_mainloop(const float* __restrict__ Ap, int lda, int a_lim, const float* __restrict__ Bp,
                                             int ldb, int b_lim, int klen, float* smem, f32x16_t (&acc)[MI][NI]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const size_t a_step = C::A_KMAJOR ? (size_t)C::BK : (size_t)C::BK * lda;  // one slab further along the contraction
  const size_t b_step = C::B_KMAJOR ? (size_t)C::BK : (size_t)C::BK * ldb;
  F32Slab<C::BM> ra;
  F32Slab<C::BN> rb;
  f32_load<C::A_KMAJOR, C::BM, VEC>(ra, Ap, lda, a_lim, klen);
  f32_load<C::B_KMAJOR, C::BN, VEC>(rb, Bp, ldb, b_lim, klen);
  f32_store<C::A_KMAJOR, C::BM, VEC>(ra, smem);
  f32_store<C::B_KMAJOR, C::BN, VEC>(rb, smem + C::BK * C::PITCH_A);
  __syncthreads();

  int cur = 0;
  for (int k0 = 0; k0 < klen; k0 += C::BK) {
    const bool more = k0 + C::BK < klen;
    if (more) {
      Ap += a_step;
      Bp += b_step;
      f32_load<C::A_KMAJOR, C::BM, VEC>(ra, Ap, lda, a_lim, klen - k0 - C::BK);
      f32_load<C::B_KMAJOR, C::BN, VEC>(rb, Bp, ldb, b_lim, klen - k0 - C::BK);
    }
    const float* As = smem + cur * C::SLAB_FLOATS;
    const float* Bs = As + C::BK * C::PITCH_A;
    // v_mfma_f32_32x32x2_f32: lane l feeds row/column (l & 31), contraction element (l >> 5) of each pair
#pragma unroll
    for (int s = 0; s < C::BK / 2; ++s) {
      float a[MI], b[NI];
#pragma unroll
      for (int i = 0; i < MI; ++i) a[i] = As[(2 * s + (lane >> 5)) * C::PITCH_A + wm * (C::BM / 2) + 32 * i + (lane & 31)];
#pragma unroll
      for (int j = 0; j < NI; ++j) b[j] = Bs[(2 * s + (lane >> 5)) * C::PITCH_B + wn * (C::BN / 2) + 32 * j + (lane & 31)];
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      float* An = smem + (cur ^ 1) * C::SLAB_FLOATS;
      f32_store<C::A_KMAJOR, C::BM, VEC>(ra, An);
      f32_store<C::B_KMAJOR, C::BN, VEC>(rb, An + C::BK * C::PITCH_A);
    }
    __syncthreads();  // the other buffer is complete, and this one is free for the slab after next
    cur ^= 1;
  }
}

template <class C>
__device__ __forceinline__ void gemm_tile_f32(const float* __restrict__ Ap, int lda, int a_lim,
                                              const float* __restrict__ Bp, int ldb, int b_lim, int klen,
                                              float* __restrict__ Op, int ldo, float* smem) {
  constexpr int MI = C::BM / 64, NI = C::BN / 64;  // 32 x 32 blocks per wave, down and across
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  f32x16_t acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  if (klen > 0) {
    const bool vec = __builtin_amdgcn_readfirstlane(f32_vec_ok<C::A_KMAJOR>(Ap, lda, a_lim, klen) &&
                                                    f32_vec_ok<C::B_KMAJOR>(Bp, ldb, b_lim, klen));
    if (vec) f32_mainloop<C, true, MI, NI>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, smem, acc);
    else f32_mainloop<C, false, MI, NI>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, smem, acc);
  }

#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int col = wn * (C::BN / 2) + 32 * j + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = wm * (C::BM / 2) + 32 * i + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (row < a_lim && col < b_lim) Op[(size_t)row * ldo + col] = acc[i][j][v];
      }
    }
}

}  // namespace rd
