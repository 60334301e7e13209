// One compiled tile shape.  Built once per entry of the variant list in the Makefile, with
//   -DRD_BM= -DRD_BN= -DRD_BK= -DRD_WAVES_M= -DRD_WAVES_N= -DRD_VEC= -DRD_NAME= [-DRD_DLDS=1|2|3 -DRD_STAGES= -DRD_PINGPONG=1
//   -DRD_F32=1|2|3|4]
// and exports a getter rd_variant_<name>() for its TileVariant record that the C-ABI file collects.
#include "rd_kernels.h"

#define RD_CAT2(a, b) a##b
#define RD_CAT(a, b) RD_CAT2(a, b)
#define RD_STR2(a) #a
#define RD_STR(a) RD_STR2(a)

#ifndef RD_DLDS
#define RD_DLDS 0
#endif
#ifndef RD_STAGES
#define RD_STAGES 2
#endif
#ifndef RD_PINGPONG
#define RD_PINGPONG 0
#endif

#ifndef RD_F32
#define RD_F32 0
#endif

namespace rd {
#if RD_F32 == 4 && RD_DLDS == 3
// float16 arrays on the four-wave direct-to-LDS core: the bf16 core's data movement with the float16 instruction
typedef W4Cfg<RD_BM, RD_BN, /*A K-major*/ true, /*B K-major*/ false, RD_STAGES, true> CfgNN;
typedef W4RCfg<RD_BM, RD_BN, true> CfgNT;
typedef W4Cfg<RD_BM, RD_BN, false, false, RD_STAGES, true> CfgTN;
#elif RD_F32 == 3 && RD_DLDS
// float8 e4m3fn arrays on the float8 matrix-core instruction, direct-to-LDS (rd_gemm_f8.h).  tgmm reads x^T as an
// MN-major operand, whose slab rows span the tile's rows: only for tile heights that are multiples of 256.
typedef F8Cfg<RD_BM, RD_BN, RD_WAVES_M, RD_WAVES_N, RD_STAGES, 64, 0, /*A K-major*/ true, /*B K-major*/ false, RD_PINGPONG != 0> CfgNN;
typedef F8Cfg<RD_BM, RD_BN, RD_WAVES_M, RD_WAVES_N, RD_STAGES, 64, 0, true, true, RD_PINGPONG != 0> CfgNT;
#if RD_BM % 256 == 0
typedef F8Cfg<RD_BM, RD_BN, RD_WAVES_M, RD_WAVES_N, RD_STAGES, 64, 0, false, false, RD_PINGPONG != 0> CfgTN;
#else
#define RD_NO_TGMM 1
#endif
#elif RD_F32 == 3
// float8 e4m3fn arrays, widened to bf16 on the way into LDS, bf16 matrix cores, bf16 out
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, /*A K-major*/ true, /*B K-major*/ false, RD_VEC != 0, fp8_bits> CfgNN;
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, true, true, RD_VEC != 0, fp8_bits> CfgNT;
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, false, false, RD_VEC != 0, fp8_bits> CfgTN;
#elif RD_F32 == 4
// float16 arrays on the float16 matrix-core instruction, float16 out
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, /*A K-major*/ true, /*B K-major*/ false, RD_VEC != 0, f16_t> CfgNN;
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, true, true, RD_VEC != 0, f16_t> CfgNT;
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, false, false, RD_VEC != 0, f16_t> CfgTN;
#elif RD_F32 == 2
// float32 arrays, rounded to bf16 on the way into LDS, bf16 matrix cores, float32 out (compute_dtype = bfloat16)
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, /*A K-major*/ true, /*B K-major*/ false, RD_VEC != 0, float> CfgNN;
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, true, true, RD_VEC != 0, float> CfgNT;
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, false, false, RD_VEC != 0, float> CfgTN;
#elif RD_F32
typedef F32Cfg<RD_BM, RD_BN, /*A K-major*/ true, /*B K-major*/ false> CfgNN;
typedef F32Cfg<RD_BM, RD_BN, true, true> CfgNT;
typedef F32Cfg<RD_BM, RD_BN, false, false> CfgTN;
#elif RD_DLDS == 3
typedef W4Cfg<RD_BM, RD_BN, /*A K-major*/ true, /*B K-major*/ false, RD_STAGES> CfgNN;
// both operands K-major: the 64-wide, register-staged form of the core (rd_gemm_w4r.h)
typedef W4RCfg<RD_BM, RD_BN> CfgNT;
typedef W4Cfg<RD_BM, RD_BN, false, false, RD_STAGES> CfgTN;
#elif RD_DLDS == 2
// one LDS ring per operand: one K-major operand in 64-wide slabs (3 slots) - the activations in the forward product,
// the weights A[g,n,k] with trans_rhs (measured 1-3 % ahead of giving them to dout) - everything else in 32-wide
// slabs (4 slots)
typedef PpCfg<RD_BM, RD_BN, RD_WAVES_M, RD_WAVES_N, /*A K-major*/ true, /*B K-major*/ false, 64, 3, 32, 4> CfgNN;
typedef PpCfg<RD_BM, RD_BN, RD_WAVES_M, RD_WAVES_N, true, true, 32, 4, 64, 3> CfgNT;
typedef PpCfg<RD_BM, RD_BN, RD_WAVES_M, RD_WAVES_N, false, false, 32, 4, 32, 4> CfgTN;
#elif RD_DLDS
typedef DldsCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, /*A K-major*/ true, /*B K-major*/ false, RD_STAGES, RD_PINGPONG != 0> CfgNN;
typedef DldsCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, true, true, RD_STAGES, RD_PINGPONG != 0> CfgNT;
typedef DldsCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, false, false, RD_STAGES, RD_PINGPONG != 0> CfgTN;
#else
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, /*A K-major*/ true, /*B K-major*/ false, RD_VEC != 0> CfgNN;
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, true, true, RD_VEC != 0> CfgNT;
typedef TileCfg<RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, false, false, RD_VEC != 0> CfgTN;
#endif
}  // namespace rd

extern "C" const rd::TileVariant* RD_CAT(rd_variant_, RD_NAME)() {
  static const rd::TileVariant v = {
      RD_STR(RD_NAME), RD_BM, RD_BN, RD_BK, RD_WAVES_M, RD_WAVES_N, RD_VEC, /*dtype: RD_DTYPE_* */ RD_F32, RD_DLDS != 0, RD_STAGES,
      /*splitk*/ RD_DLDS != 0 && (!RD_F32 || RD_F32 == 3 || RD_F32 == 4),
#ifdef RD_NO_TGMM
      &rd::launch_gmm<rd::CfgNN, false>, &rd::launch_gmm<rd::CfgNT, true>, nullptr};
#else
      &rd::launch_gmm<rd::CfgNN, false>, &rd::launch_gmm<rd::CfgNT, true>, &rd::launch_tgmm<rd::CfgTN>};
#endif
  return &v;
}
