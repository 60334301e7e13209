// Shared device-side helpers for the ragged_dot HIP kernels (gfx950 / CDNA4 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rd {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

typedef uint16_t bf16_bits;  // storage type of a bf16 element in HBM / LDS
typedef _Float16 f16_t;      // a float16 (IEEE half) element; in LDS its 16 bits travel as bf16_bits
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

// fp32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ bf16_bits f32_to_bf16(float f) {
  __bf16 h = (__bf16)f;
  return __builtin_bit_cast(bf16_bits, h);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
}

// fp32 -> float16, round to nearest even (v_cvt_f16_f32), and two of them in one word
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  const f16_t l = (f16_t)lo, h = (f16_t)hi;
  return (uint32_t)__builtin_bit_cast(uint16_t, l) | ((uint32_t)__builtin_bit_cast(uint16_t, h) << 16);
}
// two accumulator values as two 16-bit output elements: float16 (HALF) or bf16
template <bool HALF>
__device__ __forceinline__ uint32_t pack_out_x2(float lo, float hi) {
  if constexpr (HALF) return pack_f16x2(lo, hi);
  else return pack_bf16x2(lo, hi);
}
// One 32x32x16 matrix-core instruction on 16-bit operands: 8 contraction-consecutive elements per lane and operand, as
// bf16 or (HALF) as float16 - the same bits in the same places, another instruction.
template <bool HALF>
__device__ __forceinline__ f32x16_t mfma_32x32x16(bf16x8_t a, bf16x8_t b, f32x16_t c) {
  if constexpr (HALF)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

typedef uint8_t fp8_bits;  // storage type of an OCP float8 e4m3fn element in HBM

// float8 e4m3fn (1 sign, 4 exponent bits of bias 7, 3 mantissa bits; no infinities, S.1111.111 is NaN) -> bf16.  Every
// e4m3 value is a bf16 value, so this is exact (gfx950's float8 is this format).
// The two float8 bytes of the lower (HI = false) or upper half of w, as a pair of bf16: v_cvt_scalef32_pk_bf16_fp8 with
// a scale of one (checked on all 65536 pairs of codes against v_cvt_pk_f32_fp8 and the upper halves of its fp32 words).
template <bool HI>
__device__ __forceinline__ uint32_t fp8e4m3x2_to_bf16x2(uint32_t w) {
  typedef __bf16 bf16x2_raw_t __attribute__((ext_vector_type(2)));
  const bf16x2_raw_t v = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, HI);
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ uint32_t fp8e4m3_to_bf16(uint32_t b) {
  return fp8e4m3x2_to_bf16x2<false>(b & 0xff) & 0xffff;
}

__device__ __forceinline__ float bf16_to_f32(bf16_bits b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

__device__ __forceinline__ int imin(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ int imax(int a, int b) { return a > b ? a : b; }

// Work-groups are dealt to the 8 XCDs round-robin by launch index.  Remap the launch index so that each XCD
// (own 4 MB L2) walks one contiguous range of logical tile ids.  Returns -1 for the padding of the last range.
__device__ __forceinline__ int xcd_contiguous_id(int launch_id, int n_logical) {
  const int per_xcd = (n_logical + 7) >> 3;
  const int id = (launch_id & 7) * per_xcd + (launch_id >> 3);
  return id < n_logical ? id : -1;
}

static inline int xcd_padded_grid(int n_logical) { return ((n_logical + 7) / 8) * 8; }

}  // namespace rd
