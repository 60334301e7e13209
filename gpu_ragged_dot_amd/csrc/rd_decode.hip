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
constexpr int kDepth = 8;   // 16-byte weight loads kept in flight per thread (a ring of registers)
constexpr int kStage = 8;   // activation words a thread stages per round trip

// W is the (work-group uniform) start of the expert's column block; coff the thread's column offset in elements.
// One step = one 16-byte load per thread = KR weight rows per work-group.
template <int KR>
__device__ __forceinline__ u32x4_t load_step(const bf16_bits* W, uint32_t coff, int step, int kr, int k, int n) {
  // Always a load from a valid address (rows past k re-read the last row and are masked out when consumed): a
  // predicated load would make the compiler serialise the ring with a wait per load.
  const int kk = imin(step * KR + kr, k - 1);
  const uint32_t off = (uint32_t)kk * (uint32_t)n + coff;  // k * n < 2^31 is checked on the host
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(W + off));
}

template <int KR, int R>
__device__ __forceinline__ void fma_step(float (&acc)[kRows][8], const u32x4_t w, const u32x2_t* xs, int step, int kr,
                                         int k) {
  const int kk_raw = step * KR + kr;
  const uint32_t live = kk_raw < k ? 0xffffffffu : 0u;  // rows past k contribute nothing
  const u32x2_t xp = xs[imin(kk_raw, k - 1)];          // the kRows activations for contraction index kk, as bf16
  float xv[kRows];
  xv[0] = __builtin_bit_cast(float, (xp[0] << 16) & live);
  xv[1] = __builtin_bit_cast(float, xp[0] & 0xffff0000u & live);
  xv[2] = __builtin_bit_cast(float, (xp[1] << 16) & live);
  xv[3] = __builtin_bit_cast(float, xp[1] & 0xffff0000u & live);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = __builtin_bit_cast(float, w[e] << 16);
    const float hi = __builtin_bit_cast(float, w[e] & 0xffff0000u);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r][2 * e] = __builtin_fmaf(xv[r], lo, acc[r][2 * e]);
      acc[r][2 * e + 1] = __builtin_fmaf(xv[r], hi, acc[r][2 * e + 1]);
    }
  }
}

// The streaming loop for R live rows: a ring of kDepth loads per thread, each refilled with the load kDepth steps
// ahead as soon as it is consumed.
template <int KR, int R>
__device__ __forceinline__ void stream_weights(float (&acc)[kRows][8], u32x4_t (&w)[kDepth], const bf16_bits* W,
                                               uint32_t coff, const u32x2_t* xs, int kr, int k, int n) {
  const int nsteps = (k + KR - 1) / KR;
  for (int base = 0; base < nsteps; base += kDepth) {
#pragma unroll
    for (int u = 0; u < kDepth; ++u) {
      fma_step<KR, R>(acc, w[u], xs, base + u, kr, k);
      w[u] = load_step<KR>(W, coff, base + kDepth + u, kr, k, n);
    }
  }
}

template <int NB>
__global__ __launch_bounds__(kThreads, 3) void gmm_decode_kernel(DecodeArgs p) {
  static_assert(kRows == 4, "activations are staged as one 8-byte word per contraction index");
  constexpr int TPR = NB / 8;          // threads across one weight row segment
  constexpr int KR = kThreads / TPR;   // weight rows fetched per step by the work-group
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __shared__ int red[2][kThreads / 64];
  u32x2_t* xs = reinterpret_cast<u32x2_t*>(smem_raw);                   // [k] x {4 rows as bf16}
  float* part = reinterpret_cast<float*>(smem_raw + (size_t)p.k * 8);   // [waves][kRows][NB]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_blocks = (p.n + NB - 1) / NB;
  const int gi = blockIdx.x / n_blocks, jb = blockIdx.x - gi * n_blocks;
  const int my_rows = __builtin_amdgcn_readfirstlane(p.group_sizes[gi]);
  if (my_rows <= 0 && gi != p.g - 1) return;  // most experts are idle: leave before doing anything else

  const int tc = tid % TPR, kr = tid / TPR;
  const int col0 = jb * NB;
  const int cols = imin(NB, p.n - col0);            // multiple of 8
  const uint32_t coff = (uint32_t)imin(tc * 8, cols - 8);  // clamped: always a valid 16-byte chunk
  const bf16_bits* W = p.A + (size_t)gi * p.k * p.n + col0;

  // The weight stream does not depend on where the group's rows are: start it before the row range is known.
  u32x4_t w[kDepth];
  if (my_rows > 0) {
#pragma unroll
    for (int u = 0; u < kDepth; ++u) w[u] = load_step<KR>(W, coff, u, kr, p.k, p.n);
  }

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

  if (gi == p.g - 1) {  // rows past sum(group_sizes) are zero
    const int t0 = imax(imin(all, p.m), 0);
    const int cpr = cols >> 3;
    for (int idx = tid; idx < (p.m - t0) * cpr; idx += kThreads) {
      const int r = idx / cpr, c = idx - r * cpr;
      *reinterpret_cast<u32x4_t*>(p.y + (size_t)(t0 + r) * p.n + col0 + c * 8) = u32x4_t{0, 0, 0, 0};
    }
  }

  const int row0 = before;
  const int rows = imin(my_rows, p.m - row0);
  if (rows <= 0 || row0 < 0) return;

  for (int rc = 0; rc < rows; rc += kRows) {
    const int nr = imin(kRows, rows - rc);
    __syncthreads();  // previous pass done with xs / part
    // stage the activations transposed: one 8-byte word per contraction index holding the (up to) 4 rows, zero
    // for rows past nr so the FMA loop needs no row predicate.  All loads of a round go out before any is consumed.
    for (int base = 0; base < p.k; base += kThreads * kStage) {
      uint32_t v[kStage][kRows];
#pragma unroll
      for (int s2 = 0; s2 < kStage; ++s2) {
        const int kk = imin(base + s2 * kThreads + tid, p.k - 1);
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          // unconditional loads from clamped (valid) addresses, masked afterwards: keeps them all in flight at once
          const uint32_t x = p.x[(size_t)(row0 + rc + imin(r, nr - 1)) * p.k + kk];
          v[s2][r] = r < nr ? x : 0u;
        }
      }
#pragma unroll
      for (int s2 = 0; s2 < kStage; ++s2) {
        const int kk = base + s2 * kThreads + tid;
        if (kk < p.k) xs[kk] = u32x2_t{v[s2][0] | (v[s2][1] << 16), v[s2][2] | (v[s2][3] << 16)};
      }
    }
    __syncthreads();

    float acc[kRows][8];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;

    if (rc > 0) {
#pragma unroll
      for (int u = 0; u < kDepth; ++u) w[u] = load_step<KR>(W, coff, u, kr, p.k, p.n);
    }
    // a group rarely has more than one or two rows here: only the live ones cost vector-ALU work
    switch (nr) {
      case 1: stream_weights<KR, 1>(acc, w, W, coff, xs, kr, p.k, p.n); break;
      case 2: stream_weights<KR, 2>(acc, w, W, coff, xs, kr, p.k, p.n); break;
      case 3: stream_weights<KR, 3>(acc, w, W, coff, xs, kr, p.k, p.n); break;
      default: stream_weights<KR, 4>(acc, w, W, coff, xs, kr, p.k, p.n); break;
    }

    // reduce over the weight rows: first the row-slots inside a wave, then the 4 waves through LDS
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
}

template <int NB>
int launch_nb(hipStream_t s, const DecodeArgs& a) {
  const int n_blocks = (a.n + NB - 1) / NB;
  const size_t lds = (size_t)a.k * 8 + (size_t)(kThreads / 64) * kRows * NB * sizeof(float);
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
