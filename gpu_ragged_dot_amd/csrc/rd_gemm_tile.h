// One macro-tile of a bf16 x bf16 -> fp32 GEMM on gfx950 matrix cores, shared by the three grouped products:
//   gmm  NN : y[rows]  = x[rows, :]   . A[g]      (A[g] is [k, n], the contraction index is the slow one)
//   gmm  NT : y[rows]  = x[rows, :]   . A[g]^T    (A[g] is [n, k], the contraction index is the fast one)
//   tgmm TN : dA[g]    = x[rows, :]^T . dy[rows, :] (both operands have the contraction index slow)
//
// The tile computes  C[BM, BN] = sum_kk  Aop(i, kk) * Bop(j, kk)  with v_mfma_f32_32x32x16_bf16.  Each operand is
// either "K-major" (element (i, kk) at p[i*ld + kk]) or "MN-major" (element (i, kk) at p[kk*ld + i]).  K-major tiles
// sit in LDS as [rows][BK] and feed the matrix core with plain 128-bit reads; MN-major tiles sit as [BK][rows] and are
// read with the transposing LDS read (ds_read_b64_tr_b16), which hands every lane the 4 consecutive contraction
// elements of its own column.  Global -> LDS staging goes through registers: the next K-slab is fetched while the
// current one is multiplied, so there is one barrier per K-step and LDS is double-buffered.
//
// Raggedness: a tile never spans two groups.  Rows/columns of the tile past its limit are fetched from a clamped
// (always valid) address and simply not stored; only the contraction remainder is zero-filled.
#pragma once
#include <type_traits>
#include "rd_common.h"

namespace rd {

// Src: element type of the operands and the output in HBM.  bf16_bits: bf16 in, bf16 out.  float: float32 arrays whose
// elements are rounded to bf16 (nearest even) on their way into LDS, multiplied on the bf16 matrix cores with fp32
// accumulation and stored as float32 - the reference's compute_dtype = bfloat16 on float32 arrays
// (gpu_ragged_dot.py:116-119, 145, 149).  fp8_bits: float8 e4m3fn operands, widened (exactly) to bf16 on their way into
// LDS, bf16 matrix cores with fp32 accumulation, bf16 out.
// f16_t: float16 arrays on the float16 matrix-core instruction (v_mfma_f32_32x32x16_f16), fp32 accumulation, float16 out
// (rounded to nearest even); the 16-bit patterns move through the stager and LDS exactly as bf16 ones do.
template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, bool A_KMAJOR_, bool B_KMAJOR_, bool VEC_,
          typename Src = bf16_bits>
struct TileCfg {
  typedef Src Elem;
  typedef typename std::conditional<sizeof(Src) == 1, bf16_bits, Src>::type Out;  // element type of the output
  static constexpr bool F32 = false;
  static constexpr bool HALF = std::is_same<Src, f16_t>::value;  // float16 operands and matrix-core instruction
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, VEC = VEC_, DLDS = false, PINGPONG = false, MIXED = false,
                        SPLITK = false;
  static constexpr int STAGES = 2;
  static constexpr int NT = 64 * WAVES_M * WAVES_N;      // threads per work-group
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // per-wave tile
  static constexpr int TM = WM / 32, TN = WN / 32;       // 32x32 MFMA tiles per wave
  static constexpr int KSTEPS = BK / 16;
  static constexpr int WAVES_PER_EU = NT >= 256 ? NT / 256 : 1;
  // LDS row pitches (elements).  K-major rows get 16 B of padding: 16 consecutive rows then start in 16 different
  // 16-byte bank groups.  MN-major rows get 64 B: the 4 rows touched by one transposing read land in different
  // quarters of the 256-byte bank window.
  static constexpr int KM_PAD = 8, MN_PAD = 32;
  static constexpr int A_STRIDE = A_KMAJOR ? BK + KM_PAD : BM + MN_PAD;
  static constexpr int B_STRIDE = B_KMAJOR ? BK + KM_PAD : BN + MN_PAD;
  static constexpr int A_ELEMS = (A_KMAJOR ? BM : BK) * A_STRIDE;
  static constexpr int B_ELEMS = (B_KMAJOR ? BN : BK) * B_STRIDE;
  static constexpr int STAGE_ELEMS = A_ELEMS + B_ELEMS;
  static constexpr int LDS_BYTES = 2 * STAGE_ELEMS * (int)sizeof(bf16_bits);
  static_assert(BM % (32 * WAVES_M) == 0 && BN % (32 * WAVES_N) == 0 && BK % 16 == 0, "tile shape");
};

// Moves one operand's [T x BK] slab HBM -> registers -> LDS in 16-byte chunks, NT threads cooperating.
template <int T, int BK, int NT, bool KMAJOR, int STRIDE, bool VEC, typename Src = bf16_bits>
struct OperandStager {
  static constexpr int CPR = KMAJOR ? BK / 8 : T / 8;  // 16-byte chunks per LDS row
  static constexpr int ROWS = KMAJOR ? T : BK;
  static constexpr int NCHUNK = ROWS * CPR;
  static constexpr int PER = NCHUNK / NT;       // chunks per thread
  static constexpr int ROW_STEP = NT / CPR;     // LDS rows between two chunks of one thread
  static_assert(NCHUNK % NT == 0 && NT % CPR == 0 && PER >= 1, "tile too small for this many threads");

  const Src* base;  // tile origin in HBM
  int ld, lim, klen, c, r0;
  int off[PER];  // K-major: element offset of each chunk's (clamped) row; MN-major: row * ld

  // 8 consecutive elements at p as one 16-byte chunk of bf16 (VEC: p is 16-byte aligned)
  static __device__ __forceinline__ u32x4_t chunk8(const Src* p) {
    if constexpr (sizeof(Src) == 2) {
      return *reinterpret_cast<const u32x4_t*>(p);
    } else if constexpr (sizeof(Src) == 1) {
      const u32x2_t raw = *reinterpret_cast<const u32x2_t*>(p);  // 8 bytes: p is 8-byte aligned
      const u32x4_t r = {fp8e4m3x2_to_bf16x2<false>(raw[0]), fp8e4m3x2_to_bf16x2<true>(raw[0]),
                         fp8e4m3x2_to_bf16x2<false>(raw[1]), fp8e4m3x2_to_bf16x2<true>(raw[1])};
      return r;
    } else {
      const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(p), hi = *reinterpret_cast<const f32x4_t*>(p + 4);
      return u32x4_t{pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3])};
    }
  }
  static __device__ __forceinline__ bf16_bits elem(const Src* p) {
    if constexpr (std::is_same<Src, f16_t>::value) return __builtin_bit_cast(bf16_bits, *p);
    else if constexpr (sizeof(Src) == 2) return *p;
    else if constexpr (sizeof(Src) == 1) return (bf16_bits)fp8e4m3_to_bf16(*p);
    else return f32_to_bf16(*p);
  }

  __device__ __forceinline__ void init(const Src* p, int ld_, int lim_, int klen_, int tid) {
    base = p; ld = ld_; lim = lim_; klen = klen_;
    c = tid % CPR; r0 = tid / CPR;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int row = r0 + i * ROW_STEP;
      if (KMAJOR) off[i] = imin(row, lim - 1) * ld + c * 8;
      else off[i] = row * ld + (VEC ? imin(c * 8, lim - 8) : c * 8);
    }
  }

  template <bool PRED>
  __device__ __forceinline__ void load(int k0, u32x4_t (&r)[PER]) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      if (VEC) {
        if (KMAJOR) {
          const bool ok = !PRED || (k0 + c * 8 < klen);
          r[i] = ok ? chunk8(base + off[i] + k0) : u32x4_t{0, 0, 0, 0};
        } else {
          const bool ok = !PRED || (k0 + r0 + i * ROW_STEP < klen);
          r[i] = ok ? chunk8(base + (size_t)k0 * ld + off[i]) : u32x4_t{0, 0, 0, 0};
        }
      } else {
        // element-granular path for pitches that are not a multiple of 16 bytes
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          bf16_bits v = 0;
          if (KMAJOR) {
            const int kk = k0 + c * 8 + e;
            if (kk < klen) v = elem(base + off[i] + k0 + e);
          } else {
            const int kk = k0 + r0 + i * ROW_STEP;
            if (kk < klen && c * 8 + e < lim) v = elem(base + (size_t)k0 * ld + off[i] + e);
          }
          w[e >> 1] |= (uint32_t)v << ((e & 1) * 16);
        }
        r[i] = u32x4_t{w[0], w[1], w[2], w[3]};
      }
    }
  }

  __device__ __forceinline__ void store(const u32x4_t (&r)[PER], bf16_bits* lds) const {
#pragma unroll
    for (int i = 0; i < PER; ++i)
      *reinterpret_cast<u32x4_t*>(lds + (r0 + i * ROW_STEP) * STRIDE + c * 8) = r[i];
  }
};

// The 8 contraction-consecutive bf16 values one lane feeds to v_mfma_f32_32x32x16_bf16 for 32x32 tile `t32` of the
// wave, K-substep `ks`: lane l owns row/column (l & 31) and contraction elements 8*(l >> 5) .. +7.
template <bool KMAJOR, int STRIDE>
__device__ __forceinline__ bf16x8_t read_fragment(const bf16_bits* lds, int idx0, int ks, int lane) {
  if (KMAJOR) {
    const bf16_bits* p = lds + (idx0 + (lane & 31)) * STRIDE + ks * 16 + (lane >> 5) * 8;
    return *reinterpret_cast<const bf16x8_t*>(p);
  } else {
    // Transposing read: within each 16-lane group, lane i supplies the address of 4 consecutive columns
    // (4*(i&3) ..) of row (i>>2) and receives column i of rows 0..3.
    const int q = lane >> 4, i = lane & 15;
    const int row = ks * 16 + 8 * (q >> 1) + (i >> 2);
    const int col = idx0 + 16 * (q & 1) + 4 * (i & 3);
    typedef __attribute__((address_space(3))) s16x4_t* lds_v4_ptr;
    const bf16_bits* p = lds + row * STRIDE + col;
    s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_ptr)(p));
    s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_ptr)(p + 4 * STRIDE));
    s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, v);
  }
}

// C[i, j] (i < a_lim, j < b_lim) -> Op[i*ldo + j] in the element type of the configuration.  `smem` must hold
// C::LDS_BYTES.
template <class C>
__device__ __forceinline__ void gemm_tile(const typename C::Elem* __restrict__ Ap, int lda, int a_lim,
                                          const typename C::Elem* __restrict__ Bp, int ldb, int b_lim, int klen,
                                          typename C::Out* __restrict__ Op, int ldo, bf16_bits* smem) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;

  typedef OperandStager<C::BM, C::BK, C::NT, C::A_KMAJOR, C::A_STRIDE, C::VEC, typename C::Elem> StA;
  typedef OperandStager<C::BN, C::BK, C::NT, C::B_KMAJOR, C::B_STRIDE, C::VEC, typename C::Elem> StB;
  StA sa; StB sb;
  sa.init(Ap, lda, a_lim, klen, tid);
  sb.init(Bp, ldb, b_lim, klen, tid);

  f32x16_t acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  u32x4_t ra[StA::PER], rb[StB::PER];
  const int nk = (klen + C::BK - 1) / C::BK;

  if (nk > 0) {
    if (C::BK <= klen) { sa.template load<false>(0, ra); sb.template load<false>(0, rb); }
    else { sa.template load<true>(0, ra); sb.template load<true>(0, rb); }
    sa.store(ra, smem);
    sb.store(rb, smem + C::A_ELEMS);
  }
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    bf16_bits* cur = smem + (kt & 1) * C::STAGE_ELEMS;
    bf16_bits* nxt = smem + ((kt + 1) & 1) * C::STAGE_ELEMS;
    const bool more = kt + 1 < nk;
    if (more) {
      const int k0 = (kt + 1) * C::BK;
      if (k0 + C::BK <= klen) { sa.template load<false>(k0, ra); sb.template load<false>(k0, rb); }
      else { sa.template load<true>(k0, ra); sb.template load<true>(k0, rb); }
    }
    const bf16_bits* la = cur;
    const bf16_bits* lb = cur + C::A_ELEMS;
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ++ks) {
      bf16x8_t fa[C::TM], fb[C::TN];
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
        fa[i] = read_fragment<C::A_KMAJOR, C::A_STRIDE>(la, wm * C::WM + i * 32, ks, lane);
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
        fb[j] = read_fragment<C::B_KMAJOR, C::B_STRIDE>(lb, wn * C::WN + j * 32, ks, lane);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          if constexpr (C::HALF)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, fa[i]), __builtin_bit_cast(f16x8_t, fb[j]),
                                                              acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      sa.store(ra, nxt);
      sb.store(rb, nxt + C::A_ELEMS);
    }
    __syncthreads();
  }

  // Epilogue.  Accumulator register v of lane l is C[8*(v>>2) + 4*(l>>5) + (v&3)][l & 31] of its 32x32 tile.
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
      const int col = wn * C::WN + j * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = wm * C::WM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (row < a_lim && col < b_lim) {
          if constexpr (C::HALF) Op[(size_t)row * ldo + col] = (f16_t)acc[i][j][v];
          else if constexpr (sizeof(typename C::Out) == 2) Op[(size_t)row * ldo + col] = f32_to_bf16(acc[i][j][v]);
          else Op[(size_t)row * ldo + col] = acc[i][j][v];
        }
      }
    }
  }
}

// Zero rows [0, rows) x cols [0, cols) of a bf16 matrix with pitch ld, all threads of the work-group cooperating
// (nontemporal stores, like the epilogue of the tiles that compute).
template <int NT, bool VEC, typename E>
__device__ __forceinline__ void zero_tile(E* __restrict__ Op, int ld, int rows, int cols) {
  if (VEC && sizeof(E) == 2) {  // cols % 8 == 0 and 16-byte aligned rows
    const int cpr = cols >> 3;
    for (int idx = threadIdx.x; idx < rows * cpr; idx += NT) {
      const int r = idx / cpr, c = idx - r * cpr;
      __builtin_nontemporal_store(u32x4_t{0, 0, 0, 0}, reinterpret_cast<u32x4_t*>(Op + (size_t)r * ld + c * 8));
    }
  } else {
    for (int idx = threadIdx.x; idx < rows * cols; idx += NT) {
      const int r = idx / cols, c = idx - r * cols;
      Op[(size_t)r * ld + c] = 0;
    }
  }
}

}  // namespace rd
