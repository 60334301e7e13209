// Forward ragged_dot for a handful of rows per group (token-by-token decoding through a mixture of experts).
// The op is then a stream over the weights of the non-empty experts: each weight element is used by <= a few
// rows, so the matrix cores are pointless and HBM bandwidth is everything.  One launch does the whole op: every
// work-group finds its group's row range itself (a 128-entry sum), so no scheduling-map kernel runs first.
//
// Work-group (group gi, column block jb): streams A[gi][:, jb*NB .. +NB) once with 16-byte loads, ROWS rows of x at
// a time held in LDS, fp32 accumulation on the vector ALU, one cross-lane + cross-wave reduction at the end.
#include "rd_common.h"
#include "rd_decode.h"

namespace rd {

namespace {

constexpr int kThreads = 256;
constexpr int kRows = 4;    // rows of x handled per pass over the weights
constexpr int kUnroll = 8;  // 16-byte weight loads in flight per thread

template <int NB>
__global__ __launch_bounds__(kThreads) void gmm_decode_kernel(DecodeArgs p) {
  constexpr int TPR = NB / 8;          // threads across one weight row segment
  constexpr int KR = kThreads / TPR;   // weight rows fetched per step by the work-group
  constexpr int KR_WAVE = 64 / TPR;    // of which per wave
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __shared__ int red[2][kThreads / 64];
  bf16_bits* xs = reinterpret_cast<bf16_bits*>(smem_raw);                    // [kRows][k]
  float* part = reinterpret_cast<float*>(smem_raw + (size_t)kRows * p.k * 2);  // [waves][kRows][NB]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_blocks = (p.n + NB - 1) / NB;
  const int gi = blockIdx.x / n_blocks, jb = blockIdx.x - gi * n_blocks;

  // row range of this group, and the end of the last group (start of the zero tail)
  int before = 0, all = 0;
  for (int j = tid; j < p.g; j += kThreads) {
    const int s = p.group_sizes[j];
    all += s;
    if (j < gi) before += s;
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) { before += __shfl_xor(before, d, 64); all += __shfl_xor(all, d, 64); }
  if (lane == 0) { red[0][wave] = before; red[1][wave] = all; }
  __syncthreads();
  before = red[0][0] + red[0][1] + red[0][2] + red[0][3];
  all = red[1][0] + red[1][1] + red[1][2] + red[1][3];

  const int tc = tid % TPR, kr = tid / TPR;
  const int col0 = jb * NB;
  const int cols = imin(NB, p.n - col0);            // multiple of 8
  const int ccol = col0 + imin(tc * 8, cols - 8);   // clamped: always a valid 16-byte chunk
  const bool col_ok = tc * 8 < cols;

  if (gi == p.g - 1) {  // rows past sum(group_sizes) are zero
    const int t0 = imax(imin(all, p.m), 0);
    const int cpr = cols >> 3;
    for (int idx = tid; idx < (p.m - t0) * cpr; idx += kThreads) {
      const int r = idx / cpr, c = idx - r * cpr;
      *reinterpret_cast<u32x4_t*>(p.y + (size_t)(t0 + r) * p.n + col0 + c * 8) = u32x4_t{0, 0, 0, 0};
    }
  }

  const int row0 = before;
  const int rows = imin(p.group_sizes[gi], p.m - row0);
  if (rows <= 0 || row0 < 0) return;

  const bf16_bits* W = p.A + (size_t)gi * p.k * p.n + ccol;

  for (int rc = 0; rc < rows; rc += kRows) {
    const int nr = imin(kRows, rows - rc);
    __syncthreads();  // previous pass done with xs / part
    // stage x rows (zero rows past nr so the FMA loop needs no row predicate)
    const int kch = p.k >> 3;
    for (int idx = tid; idx < kRows * kch; idx += kThreads) {
      const int r = idx / kch, c = idx - r * kch;
      u32x4_t v = u32x4_t{0, 0, 0, 0};
      if (r < nr) v = *reinterpret_cast<const u32x4_t*>(p.x + (size_t)(row0 + rc + r) * p.k + c * 8);
      *reinterpret_cast<u32x4_t*>(xs + (size_t)r * p.k + c * 8) = v;
    }
    __syncthreads();

    float acc[kRows][8];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;

    for (int k0 = 0; k0 < p.k; k0 += KR * kUnroll) {
      u32x4_t w[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int kk = k0 + u * KR + kr;
        w[u] = kk < p.k ? __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(W + (size_t)kk * p.n))
                        : u32x4_t{0, 0, 0, 0};
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int kk = imin(k0 + u * KR + kr, p.k - 1);
        float xv[kRows];
#pragma unroll
        for (int r = 0; r < kRows; ++r) xv[r] = bf16_to_f32(xs[(size_t)r * p.k + kk]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float lo = __builtin_bit_cast(float, w[u][e] << 16);
          const float hi = __builtin_bit_cast(float, w[u][e] & 0xffff0000u);
#pragma unroll
          for (int r = 0; r < kRows; ++r) {
            acc[r][2 * e] = __builtin_fmaf(xv[r], lo, acc[r][2 * e]);
            acc[r][2 * e + 1] = __builtin_fmaf(xv[r], hi, acc[r][2 * e + 1]);
          }
        }
      }
    }

    // reduce over the weight rows: first the KR_WAVE row-slots inside a wave, then the 4 waves through LDS
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float v = acc[r][e];
#pragma unroll
        for (int d = TPR; d < 64; d <<= 1) v += __shfl_xor(v, d, 64);
        acc[r][e] = v;
      }
    if (lane < TPR) {
#pragma unroll
      for (int r = 0; r < kRows; ++r)
#pragma unroll
        for (int e = 0; e < 8; ++e) part[(wave * kRows + r) * NB + lane * 8 + e] = acc[r][e];
    }
    __syncthreads();
    for (int idx = tid; idx < kRows * NB; idx += kThreads) {
      const int r = idx / NB, c = idx - r * NB;
      if (r < nr && c < cols) {
        float v = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < kThreads / 64; ++w2) v += part[(w2 * kRows + r) * NB + c];
        p.y[(size_t)(row0 + rc + r) * p.n + col0 + c] = f32_to_bf16(v);
      }
    }
  }
  (void)col_ok; (void)KR_WAVE;
}

template <int NB>
int launch_nb(hipStream_t s, const DecodeArgs& a) {
  const int n_blocks = (a.n + NB - 1) / NB;
  const size_t lds = (size_t)kRows * a.k * 2 + (size_t)(kThreads / 64) * kRows * NB * sizeof(float);
  auto kern = gmm_decode_kernel<NB>;
  if (lds > 64 * 1024) {
    const int rc = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (rc != hipSuccess) return rc;
  }
  hipLaunchKernelGGL(kern, dim3(a.g * n_blocks), dim3(kThreads), lds, s, a);
  return (int)hipGetLastError();
}

}  // namespace

int launch_gmm_decode(hipStream_t s, const DecodeArgs& a, int nb) {
  if (a.m <= 0 || a.n <= 0 || a.g <= 0) return hipSuccess;
  switch (nb) {
    case 32: return launch_nb<32>(s, a);
    case 64: return launch_nb<64>(s, a);
    case 128: return launch_nb<128>(s, a);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace rd
