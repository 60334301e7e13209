// Forward ragged_dot for a handful of rows per group (token-by-token decoding through a mixture of experts).
// The op is then a stream over the weights of the non-empty experts: each weight element is used by <= a few
// rows, so the matrix cores are pointless and HBM bandwidth is everything.  No scheduling-map kernel runs first:
// every work-group finds its group's row range itself from the group sizes.
//
// Three ways of cutting the stream into work-groups:
//  * gmm_decode_kernel<NB>: work-group (group gi, column block jb) streams A[gi][:, jb*NB .. +NB) over the whole
//    contraction range and writes y itself - one launch, no workspace;
//  * gmm_rows_kernel: work-group (non-empty group, slice of the contraction range) streams whole rows of A[gi] - equal
//    contiguous blocks - and leaves fp32 partial sums for gmm_rows_finish_kernel;
//  * gmm_rows_t_kernel, for weights stored [g, n, k] (trans_rhs): work-group (non-empty group, block of weight rows =
//    output columns) - equal contiguous blocks again, but with complete sums: one launch, no workspace.
// Both hold a few rows of x at a time in LDS (4; the whole-row kernel also has a form with 8), accumulate in fp32 on the
// vector ALU and reduce across lanes at the end.
#include "rd_common.h"
#include "rd_decode.h"

namespace rd {

namespace {

constexpr int kThreads = 256;
constexpr int kRows = 4;    // rows of x handled per pass over the weights
constexpr int kDepth = 8;   // 16-byte weight loads kept in flight per thread (a ring of registers)
constexpr int kStage = 8;   // activation words a thread stages per round trip

// The kernels work on 16-bit elements: bf16, or float16 when HALF is set.  Same loads, same staging, same sums in fp32;
// what differs is how the lower / upper half of a 32-bit word becomes an fp32 value, which v_dot2 instruction multiplies
// two pairs, and how a sum is rounded to an output element.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <bool HALF>
__device__ __forceinline__ float lo_f32(uint32_t w) {
  if constexpr (HALF) return (float)__builtin_bit_cast(f16_t, (uint16_t)(w & 0xffffu));
  else return __builtin_bit_cast(float, w << 16);
}
template <bool HALF>
__device__ __forceinline__ float hi_f32(uint32_t w) {
  if constexpr (HALF) return (float)__builtin_bit_cast(f16_t, (uint16_t)(w >> 16));
  else return __builtin_bit_cast(float, w & 0xffff0000u);
}
template <bool HALF>
__device__ __forceinline__ float dot2_f32(uint32_t a, uint32_t b, float c) {
  if constexpr (HALF) return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), c, false);
  else return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}
template <bool HALF>
__device__ __forceinline__ uint16_t round_out(float v) {
  if constexpr (HALF) return __builtin_bit_cast(uint16_t, (f16_t)v);
  else return f32_to_bf16(v);
}
template <bool HALF>
__device__ __forceinline__ uint32_t round_out_x2(float lo, float hi) {
  if constexpr (HALF) return pack_f16x2(lo, hi);
  else return pack_bf16x2(lo, hi);
}

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

template <int KR, int R, bool HALF>
__device__ __forceinline__ void fma_step(float (&acc)[kRows][8], const u32x4_t w, const u32x2_t* xs, int step, int kr,
                                         int k) {
  const int kk_raw = step * KR + kr;
  const uint32_t live = kk_raw < k ? 0xffffffffu : 0u;  // rows past k contribute nothing
  const u32x2_t xp = xs[imin(kk_raw, k - 1)];          // the kRows activations for contraction index kk, as bf16
  float xv[kRows];
  if constexpr (HALF) {
    const uint32_t x0 = xp[0] & live, x1 = xp[1] & live;
    xv[0] = lo_f32<true>(x0); xv[1] = hi_f32<true>(x0); xv[2] = lo_f32<true>(x1); xv[3] = hi_f32<true>(x1);
  } else {
    xv[0] = __builtin_bit_cast(float, (xp[0] << 16) & live);
    xv[1] = __builtin_bit_cast(float, xp[0] & 0xffff0000u & live);
    xv[2] = __builtin_bit_cast(float, (xp[1] << 16) & live);
    xv[3] = __builtin_bit_cast(float, xp[1] & 0xffff0000u & live);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = lo_f32<HALF>(w[e]);
    const float hi = hi_f32<HALF>(w[e]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r][2 * e] = __builtin_fmaf(xv[r], lo, acc[r][2 * e]);
      acc[r][2 * e + 1] = __builtin_fmaf(xv[r], hi, acc[r][2 * e + 1]);
    }
  }
}

// The streaming loop for R live rows: a ring of kDepth loads per thread, each refilled with the load kDepth steps
// ahead as soon as it is consumed.
template <int KR, int R, bool HALF>
__device__ __forceinline__ void stream_weights(float (&acc)[kRows][8], u32x4_t (&w)[kDepth], const bf16_bits* W,
                                               uint32_t coff, const u32x2_t* xs, int kr, int k, int n) {
  const int nsteps = (k + KR - 1) / KR;
  for (int base = 0; base < nsteps; base += kDepth) {
#pragma unroll
    for (int u = 0; u < kDepth; ++u) {
      fma_step<KR, R, HALF>(acc, w[u], xs, base + u, kr, k);
      w[u] = load_step<KR>(W, coff, base + kDepth + u, kr, k, n);
    }
  }
}

template <int NB, bool HALF>
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
      case 1: stream_weights<KR, 1, HALF>(acc, w, W, coff, xs, kr, p.k, p.n); break;
      case 2: stream_weights<KR, 2, HALF>(acc, w, W, coff, xs, kr, p.k, p.n); break;
      case 3: stream_weights<KR, 3, HALF>(acc, w, W, coff, xs, kr, p.k, p.n); break;
      default: stream_weights<KR, 4, HALF>(acc, w, W, coff, xs, kr, p.k, p.n); break;
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
        p.y[(size_t)(row0 + rc + r) * p.n + col0 + c] = round_out<HALF>(v);
      }
    }
  }
}

template <int NB, bool HALF>
int launch_nb(hipStream_t s, const DecodeArgs& a) {
  const int n_blocks = (a.n + NB - 1) / NB;
  const size_t lds = (size_t)a.k * 8 + (size_t)(kThreads / 64) * kRows * NB * sizeof(float);
  auto kern = gmm_decode_kernel<NB, HALF>;
  if (lds > 64 * 1024) {
    const int rc = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (rc != hipSuccess) return rc;
  }
  hipLaunchKernelGGL(kern, dim3(a.g * n_blocks), dim3(kThreads), lds, s, a);
  return (int)hipGetLastError();
}


// ---- whole-row slices ----------------------------------------------------------------------------------------------
// The strip kernel above reads 64- to 256-byte pieces of every weight row and has as many work-groups as there are
// (non-empty expert, column strip) pairs; on the decode shape that is 636 unequal-looking jobs for 256 compute units,
// and bare load kernels show that this access pattern tops out ~25 % below what contiguous, evenly spread blocks
// reach.  The kernel below cuts the stream the other way: every non-empty expert gets the same number C of
// work-groups, each taking whole rows of the weight matrix for a C-th of the contraction range - one contiguous block
// of memory, all blocks the same size.  A piece only yields partial sums: they go to the workspace as fp32
// [row][C][n] and a second, tiny kernel adds the C pieces in order, rounds, and zeroes the rows past sum(group_sizes).
// Which expert a work-group serves depends on which experts are non-empty, so every work-group first scans the group
// sizes (from L2) - the one dependent step before its weight stream starts.

constexpr int kRowsDepth = 6;  // 16-byte weight loads in flight per thread (measured: 3 -> 39 us, 4 -> 34.4, 6 -> 33.2, 8 -> 34.3, 16 -> 36.6)
constexpr int kMaxSeg = 2048;  // contraction indices staged in LDS at a time

struct RowsGeom {
  int wgs;       // work-groups launched
  int lpr;       // threads across one weight row = n / 8 (<= 256)
  int rps;       // weight rows fetched per step = 256 / lpr
  int max_c;     // most pieces per expert the workspace has room for
  int min_rows;  // fewest contraction indices a piece may get
};

struct RowsHeader { int32_t pieces, total_rows; };  // written by work-group 0 for the finishing kernel

__device__ __forceinline__ u32x4_t load_row_step(const bf16_bits* W, uint32_t coff, int step, int rps, int kr, int klen, int n) {
  const int kk = imin(step * rps + kr, klen - 1);  // clamped, masked when consumed
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(W + (uint32_t)kk * (uint32_t)n + coff));
}

template <int R, bool HALF>
__device__ __forceinline__ void fma_row_step(float (&acc)[kRows][8], const u32x4_t w, const u32x2_t* xs, int step, int rps,
                                             int kr, int klen) {
  const int kk_raw = step * rps + kr;
  const uint32_t live = kk_raw < klen ? 0xffffffffu : 0u;
  const u32x2_t xp = xs[imin(kk_raw, klen - 1)];
  float xv[kRows];
  if constexpr (HALF) {
    const uint32_t x0 = xp[0] & live, x1 = xp[1] & live;
    xv[0] = lo_f32<true>(x0); xv[1] = hi_f32<true>(x0); xv[2] = lo_f32<true>(x1); xv[3] = hi_f32<true>(x1);
  } else {
    xv[0] = __builtin_bit_cast(float, (xp[0] << 16) & live);
    xv[1] = __builtin_bit_cast(float, xp[0] & 0xffff0000u & live);
    xv[2] = __builtin_bit_cast(float, (xp[1] << 16) & live);
    xv[3] = __builtin_bit_cast(float, xp[1] & 0xffff0000u & live);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = lo_f32<HALF>(w[e]);
    const float hi = hi_f32<HALF>(w[e]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r][2 * e] = __builtin_fmaf(xv[r], lo, acc[r][2 * e]);
      acc[r][2 * e + 1] = __builtin_fmaf(xv[r], hi, acc[r][2 * e + 1]);
    }
  }
}

template <int R, bool HALF>
__device__ __forceinline__ void stream_rows(float (&acc)[kRows][8], u32x4_t (&w)[kRowsDepth], const bf16_bits* W, uint32_t coff,
                                            const u32x2_t* xs, int rps, int kr, int klen, int n) {
  const int nsteps = (klen + rps - 1) / rps;
  for (int base = 0; base < nsteps; base += kRowsDepth) {
#pragma unroll
    for (int u = 0; u < kRowsDepth; ++u) {
      fma_row_step<R, HALF>(acc, w[u], xs, base + u, rps, kr, klen);
      w[u] = load_row_step(W, coff, base + kRowsDepth + u, rps, kr, klen, n);
    }
  }
}

// ---- passes of up to 8 rows (gmm_rows_kernel<true>) -----------------------------------------------------------------
// Twice the rows on the vector ALU for the same instruction count: a thread takes two adjacent weight rows at a time,
// pairs up the two rows' bf16 values of each column with one byte permute, and one v_dot2_f32_bf16 multiplies the pair
// with a token row's pair of activations (staged in LDS as one 32-bit word per token row and pair of contraction
// indices).  For groups of at most 4 rows the routine above is the faster one by 1 % (32.9 against 33.2 us on 53
// experts of 2048 x 768 with at most 3 rows each), so the launcher picks by the average rows per group.
constexpr int kWideRows = 8;     // rows per pass
constexpr int kPairDepth = 3;    // pairs of 16-byte weight loads in flight per thread
constexpr int kWideSeg = 1024;   // contraction indices staged at a time: (kWideSeg / 2 + 1) entries of 32 bytes
constexpr int kWideStage = 4;    // activation words a thread stages per round trip
constexpr int kXsBytes = ((kWideSeg >> 1) + 1) * kWideRows * 4;

// Weight rows 2 * (step * rps + kr) and the one after it, clamped to the segment (rows past klen, which is even,
// re-read its last two rows; their activations are read from the all-zero entry).
__device__ __forceinline__ void load_row_pair(u32x4_t& even, u32x4_t& odd, const bf16_bits* W, uint32_t coff, int step, int rps,
                                              int kr, int klen, int n) {
  const int kk = 2 * (step * rps + kr);
  const uint32_t off = (uint32_t)imin(kk, klen - 2) * (uint32_t)n + coff;
  even = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(W + off));
  odd = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(W + off + (uint32_t)n));
}

template <int R, bool HALF>
__device__ __forceinline__ void fma_row_pair(float (&acc)[kWideRows][8], const u32x4_t even, const u32x4_t odd,
                                             const u32x4_t* xs, int step, int rps, int kr, int pairs) {
  const int pj = step * rps + kr;
  const int pair = pj < pairs ? pj : (kWideSeg >> 1);  // past the segment: the all-zero entry behind the staged pairs
  uint32_t xv[kWideRows];
  const u32x4_t a = xs[pair * 2];
  xv[0] = a[0]; xv[1] = a[1]; xv[2] = a[2]; xv[3] = a[3];
  if (R > 4) {
    const u32x4_t b = xs[pair * 2 + 1];
    xv[4] = b[0]; xv[5] = b[1]; xv[6] = b[2]; xv[7] = b[3];
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t lo = __builtin_amdgcn_perm(odd[e], even[e], 0x05040100u);  // (W[kk][2e],     W[kk + 1][2e])
    const uint32_t hi = __builtin_amdgcn_perm(odd[e], even[e], 0x07060302u);  // (W[kk][2e + 1], W[kk + 1][2e + 1])
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r][2 * e] = dot2_f32<HALF>(lo, xv[r], acc[r][2 * e]);
      acc[r][2 * e + 1] = dot2_f32<HALF>(hi, xv[r], acc[r][2 * e + 1]);
    }
  }
}

template <int R, bool HALF>
__device__ __forceinline__ void stream_row_pairs(float (&acc)[kWideRows][8], u32x4_t (&w)[2 * kPairDepth], const bf16_bits* W,
                                                 uint32_t coff, const u32x4_t* xs, int rps, int kr, int klen, int n) {
  const int nsteps = (klen + 2 * rps - 1) / (2 * rps);
  const int pairs = klen >> 1;
  for (int base = 0; base < nsteps; base += kPairDepth) {
#pragma unroll
    for (int u = 0; u < kPairDepth; ++u) {
      fma_row_pair<R, HALF>(acc, w[2 * u], w[2 * u + 1], xs, base + u, rps, kr, pairs);
      // Keep every refill where it is written: sunk to the end of the iteration, the loads would all wait for the last
      // pair and the ring would run empty once per iteration.
      __builtin_amdgcn_sched_barrier(0);
      load_row_pair(w[2 * u], w[2 * u + 1], W, coff, base + kPairDepth + u, rps, kr, klen, n);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// One pass of nr = 1 .. 8 rows (rows row_first ..) of a piece: its sums into part[kr][r][n] of the loader threads.
template <bool HALF>
__device__ __forceinline__ void wide_pass(const DecodeArgs& p, int rps, int unit, int gi, int row_first, int nr, int k0,
                                          int klen_all, int tid, int tc, int kr, bool loader, unsigned char* smem_raw,
                                          float* part) {
  const u32x4_t* xs = reinterpret_cast<const u32x4_t*>(smem_raw);
  uint32_t* xs_words = reinterpret_cast<uint32_t*>(smem_raw);
  const uint32_t coff = (uint32_t)(tc * 8);
  float acc[kWideRows][8];
#pragma unroll
  for (int r = 0; r < kWideRows; ++r)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;
  const int seg = kWideSeg / unit * unit;  // whole steps: only a piece's last segment ends inside one
  for (int s0 = 0; s0 < klen_all; s0 += seg) {
    const int klen = imin(seg, klen_all - s0);  // even: k0, seg and the contraction length are
    const bf16_bits* W = p.A + (size_t)gi * p.k * p.n + (size_t)(k0 + s0) * p.n;
    u32x4_t w[2 * kPairDepth];
    if (loader) {
#pragma unroll
      for (int u = 0; u < kPairDepth; ++u) load_row_pair(w[2 * u], w[2 * u + 1], W, coff, u, rps, kr, klen, p.n);
    }
    __syncthreads();  // previous segment / pass done with xs and part
    // stage the activations: word [pair j][row r] = (x[r][2j], x[r][2j + 1]), zero for rows past nr.  Unconditional
    // loads from clamped (valid) addresses, all of a round in flight before any is consumed.
    const int pairs = klen >> 1;
    for (int base = 0; base < pairs * kWideRows; base += kThreads * kWideStage) {
      uint32_t v[kWideStage];
#pragma unroll
      for (int s2 = 0; s2 < kWideStage; ++s2) {
        const int idx = base + s2 * kThreads + tid;
        const int j = imin(idx >> 3, pairs - 1), r = imin(idx & 7, nr - 1);
        v[s2] = *reinterpret_cast<const uint32_t*>(p.x + (size_t)(row_first + r) * p.k + k0 + s0 + 2 * j);
      }
#pragma unroll
      for (int s2 = 0; s2 < kWideStage; ++s2) {
        const int idx = base + s2 * kThreads + tid;
        if (idx < pairs * kWideRows) xs_words[idx] = (idx & 7) < nr ? v[s2] : 0u;
      }
    }
    if (tid < kWideRows) xs_words[(kWideSeg >> 1) * kWideRows + tid] = 0u;
    __syncthreads();
    if (loader) {
      switch (nr) {
        case 1: stream_row_pairs<1, HALF>(acc, w, W, coff, xs, rps, kr, klen, p.n); break;
        case 2: stream_row_pairs<2, HALF>(acc, w, W, coff, xs, rps, kr, klen, p.n); break;
        case 3: stream_row_pairs<3, HALF>(acc, w, W, coff, xs, rps, kr, klen, p.n); break;
        case 4: stream_row_pairs<4, HALF>(acc, w, W, coff, xs, rps, kr, klen, p.n); break;
        case 5: stream_row_pairs<5, HALF>(acc, w, W, coff, xs, rps, kr, klen, p.n); break;
        case 6: stream_row_pairs<6, HALF>(acc, w, W, coff, xs, rps, kr, klen, p.n); break;
        case 7: stream_row_pairs<7, HALF>(acc, w, W, coff, xs, rps, kr, klen, p.n); break;
        default: stream_row_pairs<8, HALF>(acc, w, W, coff, xs, rps, kr, klen, p.n); break;
      }
    }
  }
  __syncthreads();
  if (loader) {
#pragma unroll
    for (int r = 0; r < kWideRows; ++r) {
      if (r < nr) {
        float* dst = part + ((size_t)(kr * kWideRows + r) * p.n + tc * 8);
        *reinterpret_cast<f32x4_t*>(dst) = f32x4_t{acc[r][0], acc[r][1], acc[r][2], acc[r][3]};
        *reinterpret_cast<f32x4_t*>(dst + 4) = f32x4_t{acc[r][4], acc[r][5], acc[r][6], acc[r][7]};
      }
    }
  }
}


template <bool WIDE, bool HALF>
__global__ __launch_bounds__(kThreads, 2) void gmm_rows_kernel(DecodeArgs p, RowsGeom q, RowsHeader* __restrict__ header,
                                                               float* __restrict__ partials) {
  __shared__ int32_t wave_cnt[3][kThreads / 64];
  __shared__ int32_t job[3];                // expert, first row and row count of the pass this work-group serves
  constexpr int RPP = WIDE ? kWideRows : kRows;  // rows per pass
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x2_t* xs = reinterpret_cast<u32x2_t*>(smem_raw);                   // [kMaxSeg] x {4 rows as bf16}
  float* part = reinterpret_cast<float*>(smem_raw + (WIDE ? kXsBytes : kMaxSeg * 8));  // [rps][rows per pass][n]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // ---- which experts are non-empty, and where their rows start: a scan over the group sizes --------------------------
  // One slab of kThreads experts at a time: every thread learns how many jobs and rows precede its own expert's.  A job
  // is one pass over an expert's weights with up to RPP of its rows: an expert with more rows than a pass holds is
  // several jobs, served by different work-groups at the same time - if all rows of a call pile up in one group, its
  // weights are streamed by all work-groups together (out of L2 after the first pass) instead of pass after pass by a
  // few.  With g <= kThreads (the usual case) the group sizes are read once and the result stays in registers.
  auto scan_slab = [&](int base, int seen, int rows_seen, int& sz, int& rank, int& first_row, int& slab_act, int& slab_rows) {
    const int e = base + tid;
    sz = e < p.g ? imin(imax(p.group_sizes[e], 0), p.m) : 0;  // (no group has more than m rows that exist)
    const int units = (sz + RPP - 1) / RPP;  // passes over this expert's weights, each a job of its own
    const unsigned long long m_act = __ballot(sz > 0);
    const bool wave_big = __ballot(sz > RPP) != 0;  // some expert of this wave takes more than one pass
    int incl = sz;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) { const int up = __shfl_up(incl, d, 64); if (lane >= d) incl += up; }
    __syncthreads();  // wave_cnt free again
    if (lane == 63) { wave_cnt[0][wave] = __popcll(m_act); wave_cnt[1][wave] = incl; wave_cnt[2][wave] = wave_big; }
    __syncthreads();
    // One pass per non-empty expert (the usual case): the jobs before this expert are the non-empty experts before it.
    rank = seen + __popcll(m_act & ((1ull << lane) - 1ull));
    first_row = rows_seen + incl - sz;
    slab_act = 0; slab_rows = 0;
    bool any_big = false;
    for (int w2 = 0; w2 < kThreads / 64; ++w2) {
      if (w2 < wave) { rank += wave_cnt[0][w2]; first_row += wave_cnt[1][w2]; }
      slab_act += wave_cnt[0][w2]; slab_rows += wave_cnt[1][w2];
      any_big |= wave_cnt[2][w2] != 0;
    }
    if (any_big) {  // (the same in every thread) experts with several passes: count passes instead of experts
      int incl_u = units;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) { const int up = __shfl_up(incl_u, d, 64); if (lane >= d) incl_u += up; }
      __syncthreads();
      if (lane == 63) wave_cnt[0][wave] = incl_u;
      __syncthreads();
      rank = seen + incl_u - units;
      slab_act = 0;
      for (int w2 = 0; w2 < kThreads / 64; ++w2) {
        if (w2 < wave) rank += wave_cnt[0][w2];
        slab_act += wave_cnt[0][w2];
      }
    }
  };
  const bool one_slab = p.g <= kThreads;
  int sz0 = 0, rank0 = 0, first0 = 0;
  int n_jobs = 0, total = 0;
  for (int base = 0; base < p.g; base += kThreads) {
    int sz, rank, first_row, sa, sr;
    scan_slab(base, n_jobs, total, sz, rank, first_row, sa, sr);
    if (base == 0) { sz0 = sz; rank0 = rank; first0 = first_row; }
    n_jobs += sa; total += sr;
  }
  int C = n_jobs > 0 ? q.wgs / n_jobs : 1;
  C = imax(1, imin(imin(C, q.max_c), p.k / q.min_rows));
  if (blockIdx.x == 0 && tid == 0) { header->pieces = C; header->total_rows = imin(total, p.m); }
  if (n_jobs == 0 || (int)blockIdx.x >= (q.wgs / C) * C) return;  // nothing to do / left-over work-groups

  const int c = blockIdx.x % C;
  for (int want = blockIdx.x / C; want < n_jobs; want += q.wgs / C) {
    // the `want`-th non-empty expert and the rows before it
    __syncthreads();  // job free again
    if (one_slab) {
      if (sz0 > 0 && rank0 <= want && want < rank0 + (sz0 + RPP - 1) / RPP) {
        const int done = (want - rank0) * RPP;  // rows of the expert that earlier passes take
        job[0] = tid; job[1] = first0 + done; job[2] = imin(RPP, sz0 - done);
      }
    } else {
      int seen = 0, rows_seen = 0;
      for (int base = 0; base < p.g; base += kThreads) {
        int sz, rank, first_row, sa, sr;
        scan_slab(base, seen, rows_seen, sz, rank, first_row, sa, sr);
        if (sz > 0 && rank <= want && want < rank + (sz + RPP - 1) / RPP) {
          const int done = (want - rank) * RPP;
          job[0] = base + tid; job[1] = first_row + done; job[2] = imin(RPP, sz - done);
        }
        seen += sa; rows_seen += sr;
      }
    }
    __syncthreads();
    const int gi = job[0], row0 = job[1];
    const int rows = imin(job[2], p.m - row0);
    if (rows <= 0) continue;

    // ---- this piece: contraction indices [k0, k0 + klen_all) of expert gi, whole rows ---------------------------------
    const int unit = q.rps * 2;
    const int per = ((p.k + C - 1) / C + unit - 1) / unit * unit;
    const int k0 = c * per;
    const int klen_all = imin(per, p.k - k0);
    const int tc = tid % q.lpr, kr = tid / q.lpr;
    const bool loader = kr < q.rps;
    const uint32_t coff = (uint32_t)(tc * 8);
    if constexpr (WIDE) {
      for (int rc = 0; rc < rows; rc += kWideRows) {
        const int nr = imin(kWideRows, rows - rc);
        wide_pass<HALF>(p, q.rps, unit, gi, row0 + rc, nr, k0, klen_all, tid, tc, kr, loader, smem_raw, part);
        __syncthreads();
        for (int idx = tid; idx < nr * p.n; idx += kThreads) {
          const int r = idx / p.n, col = idx - r * p.n;
          float v = 0.f;
          for (int s2 = 0; s2 < q.rps; ++s2) v += part[(size_t)(s2 * kWideRows + r) * p.n + col];
          partials[((size_t)(row0 + rc + r) * C + c) * p.n + col] = v;
        }
      }
      continue;
    }
    for (int rc = 0; rc < rows; rc += kRows) {
      const int nr = imin(kRows, rows - rc);
      float acc[kRows][8];
#pragma unroll
      for (int r = 0; r < kRows; ++r)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;
      for (int s0 = 0; s0 < klen_all; s0 += kMaxSeg) {
        const int klen = imin(kMaxSeg, klen_all - s0);
        const bf16_bits* W = p.A + (size_t)gi * p.k * p.n + (size_t)(k0 + s0) * p.n;
        u32x4_t w[kRowsDepth];
        if (loader) {
#pragma unroll
          for (int u = 0; u < kRowsDepth; ++u) w[u] = load_row_step(W, coff, u, q.rps, kr, klen, p.n);
        }
        __syncthreads();  // previous segment / pass done with xs and part
        for (int j = tid; j < klen; j += kThreads) {
          uint32_t v[kRows];
#pragma unroll
          for (int r = 0; r < kRows; ++r) {
            const uint32_t x = p.x[(size_t)(row0 + rc + imin(r, nr - 1)) * p.k + k0 + s0 + j];
            v[r] = r < nr ? x : 0u;
          }
          xs[j] = u32x2_t{v[0] | (v[1] << 16), v[2] | (v[3] << 16)};
        }
        __syncthreads();
        if (loader) {
          switch (nr) {
            case 1: stream_rows<1, HALF>(acc, w, W, coff, xs, q.rps, kr, klen, p.n); break;
            case 2: stream_rows<2, HALF>(acc, w, W, coff, xs, q.rps, kr, klen, p.n); break;
            case 3: stream_rows<3, HALF>(acc, w, W, coff, xs, q.rps, kr, klen, p.n); break;
            default: stream_rows<4, HALF>(acc, w, W, coff, xs, q.rps, kr, klen, p.n); break;
          }
        }
      }
      // reduce over the rps row slots through LDS, then hand the piece's sums over
      __syncthreads();
      if (loader) {
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          float* dst = part + ((size_t)(kr * kRows + r) * p.n + tc * 8);
          *reinterpret_cast<f32x4_t*>(dst) = f32x4_t{acc[r][0], acc[r][1], acc[r][2], acc[r][3]};
          *reinterpret_cast<f32x4_t*>(dst + 4) = f32x4_t{acc[r][4], acc[r][5], acc[r][6], acc[r][7]};
        }
      }
      __syncthreads();
      for (int idx = tid; idx < nr * p.n; idx += kThreads) {
        const int r = idx / p.n, col = idx - r * p.n;
        float v = 0.f;
        for (int s2 = 0; s2 < q.rps; ++s2) v += part[(size_t)(s2 * kRows + r) * p.n + col];
        partials[((size_t)(row0 + rc + r) * C + c) * p.n + col] = v;
      }
    }
  }
}

// ---- trans_rhs: weights stored [g, n, k] --------------------------------------------------------------------------
// Every weight row A[gi][j][:] is one contiguous run along the contraction index and yields one output column, so the
// stream is cut along n: every non-empty expert gets the same number C of work-groups, each taking a contiguous block
// of whole weight rows - and with them complete sums.  No partial sums, no workspace, one launch that writes y itself.
// A wave takes one weight row at a time (64 lanes x 16 bytes = 1 KB per load, the four waves of a work-group four
// consecutive rows); a lane multiplies its 8 contraction indices of the row with the same 8 of up to RMAX token rows
// (both operands run along k, so pairs of bf16 meet in v_dot2_f32_bf16 as they are loaded), sums over its positions
// along the row, and the 64 lanes' sums are added at the end of the row.
constexpr int kTBlock = 4;        // weight rows a wave works on at a time: one read of the activations serves them all
constexpr int kTDepth = 2;        // steps (of kTBlock 16-byte loads per lane) in flight
constexpr int kTMaxLds = 64 * 1024;  // staged activations: RMAX rows x k (padded to 512) x 2 bytes

// Sums of V values per lane over the 64 lanes of a wave.  Butterfly steps that halve the values as they go: in the step
// with lane distance d a lane keeps one half of what it still holds, hands the other half to lane ^ d and adds what it
// gets for its own half, so V - 1 exchanges (plus one per remaining step once a single value is left) replace the 6 V of
// reducing every value by itself.  Returns the complete sum of value (lane >> (6 - log2 V)) & (V - 1).
template <int V, int COUNT, int D>
__device__ __forceinline__ float wave_sums_step(float (&v)[V], int lane) {
  if constexpr (COUNT > 1) {
    constexpr int HALF = COUNT / 2;
    const bool upper = (lane & D) != 0;
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
      const float send = upper ? v[i] : v[i + HALF];
      const float keep = upper ? v[i + HALF] : v[i];
      v[i] = keep + __shfl_xor(send, D, 64);
    }
    return wave_sums_step<V, HALF, D / 2>(v, lane);
  } else if constexpr (D >= 1) {
    v[0] += __shfl_xor(v[0], D, 64);
    return wave_sums_step<V, 1, D / 2>(v, lane);
  } else {
    return v[0];
  }
}
template <int V>
__device__ __forceinline__ float wave_sums(float (&v)[V], int lane) {
  static_assert(V >= 1 && V <= 64 && (V & (V - 1)) == 0, "a power of two");
  return wave_sums_step<V, V, 32>(v, lane);
}

// F8: x and A hold float8 e4m3fn bytes (y is bf16 all the same).  A 16-byte chunk is then 16 contraction indices; the
// activations are widened to bf16 as they are staged (two 16-byte entries per chunk, the chunk's lower and upper eight),
// the weights as they are used (one v_cvt_scalef32_pk_bf16_fp8 per pair, once per block of weight rows and shared
// by the token rows), and the same v_dot2_f32_bf16 multiplies them - exactly, every e4m3 value being a bf16 value.
template <int RMAX, bool F8, bool HALF>
__global__ __launch_bounds__(kThreads, 2) void gmm_rows_t_kernel(DecodeArgs p, int wgs) {
  static_assert(!(F8 && HALF), "float8 operands are widened to bf16");
  constexpr int EB = F8 ? 1 : 2;     // bytes per element of x and A
  constexpr int EPC = 16 / EB;       // elements per 16-byte chunk
  constexpr int XE = F8 ? 2 : 1;     // staged 16-byte entries per chunk and token row
  __shared__ int32_t wave_cnt[3][kThreads / 64];
  __shared__ int32_t job[3];
  constexpr int RPP = RMAX;          // rows per pass
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4_t* xs = reinterpret_cast<u32x4_t*>(smem_raw);  // [RMAX rows][XE][chunk] x 16 bytes (8 bf16)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // which experts are non-empty and where their rows start (as in gmm_rows_kernel)
  auto scan_slab = [&](int base, int seen, int rows_seen, int& sz, int& rank, int& first_row, int& slab_act, int& slab_rows) {
    const int e = base + tid;
    sz = e < p.g ? imin(imax(p.group_sizes[e], 0), p.m) : 0;  // (no group has more than m rows that exist)
    const int units = (sz + RPP - 1) / RPP;  // passes over this expert's weights, each a job of its own
    const unsigned long long m_act = __ballot(sz > 0);
    const bool wave_big = __ballot(sz > RPP) != 0;  // some expert of this wave takes more than one pass
    int incl = sz;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) { const int up = __shfl_up(incl, d, 64); if (lane >= d) incl += up; }
    __syncthreads();
    if (lane == 63) { wave_cnt[0][wave] = __popcll(m_act); wave_cnt[1][wave] = incl; wave_cnt[2][wave] = wave_big; }
    __syncthreads();
    // One pass per non-empty expert (the usual case): the jobs before this expert are the non-empty experts before it.
    rank = seen + __popcll(m_act & ((1ull << lane) - 1ull));
    first_row = rows_seen + incl - sz;
    slab_act = 0; slab_rows = 0;
    bool any_big = false;
    for (int w2 = 0; w2 < kThreads / 64; ++w2) {
      if (w2 < wave) { rank += wave_cnt[0][w2]; first_row += wave_cnt[1][w2]; }
      slab_act += wave_cnt[0][w2]; slab_rows += wave_cnt[1][w2];
      any_big |= wave_cnt[2][w2] != 0;
    }
    if (any_big) {  // (the same in every thread) experts with several passes: count passes instead of experts
      int incl_u = units;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) { const int up = __shfl_up(incl_u, d, 64); if (lane >= d) incl_u += up; }
      __syncthreads();
      if (lane == 63) wave_cnt[0][wave] = incl_u;
      __syncthreads();
      rank = seen + incl_u - units;
      slab_act = 0;
      for (int w2 = 0; w2 < kThreads / 64; ++w2) {
        if (w2 < wave) rank += wave_cnt[0][w2];
        slab_act += wave_cnt[0][w2];
      }
    }
  };
  const bool one_slab = p.g <= kThreads;
  int sz0 = 0, rank0 = 0, first0 = 0;
  int n_jobs = 0, total = 0;
  for (int base = 0; base < p.g; base += kThreads) {
    int sz, rank, first_row, sa, sr;
    scan_slab(base, n_jobs, total, sz, rank, first_row, sa, sr);
    if (base == 0) { sz0 = sz; rank0 = rank; first0 = first_row; }
    n_jobs += sa; total += sr;
  }

  // rows past sum(group_sizes) are zero: every work-group clears its share of them
  {
    const int t0 = imax(imin(total, p.m), 0);
    const size_t words = (size_t)(p.m - t0) * p.n / 8;  // n % 8 == 0
    u32x4_t* tail = reinterpret_cast<u32x4_t*>(p.y + (size_t)t0 * p.n);
    for (size_t i = (size_t)blockIdx.x * kThreads + tid; i < words; i += (size_t)wgs * kThreads) tail[i] = u32x4_t{0, 0, 0, 0};
  }
  if (n_jobs == 0) return;
  int C = imax(1, imin(wgs / n_jobs, p.n / kTBlock));  // a piece holds at least one block of weight rows
  const int per = ((p.n + C - 1) / C + kTBlock - 1) / kTBlock * kTBlock;  // weight rows per piece (n % 8 == 0: whole blocks)
  C = (p.n + per - 1) / per;                          // pieces that hold any
  const int jobs_at_a_time = wgs / C;
  if ((int)blockIdx.x >= jobs_at_a_time * C) return;
  const int c = blockIdx.x % C;
  const int j_begin = c * per, j_end = imin(p.n, j_begin + per);
  const int chunks = p.k / EPC;                       // 16-byte chunks per weight row (k % EPC == 0)
  const int npos = (chunks + 63) >> 6;                // loads per lane and weight row
  const int r_stride = npos * 64;                     // staged chunks per token row
  const unsigned char* xb = reinterpret_cast<const unsigned char*>(p.x);

  for (int want = blockIdx.x / C; want < n_jobs; want += jobs_at_a_time) {
    __syncthreads();  // job free again
    if (one_slab) {
      if (sz0 > 0 && rank0 <= want && want < rank0 + (sz0 + RPP - 1) / RPP) {
        const int done = (want - rank0) * RPP;  // rows of the expert that earlier passes take
        job[0] = tid; job[1] = first0 + done; job[2] = imin(RPP, sz0 - done);
      }
    } else {
      int seen = 0, rows_seen = 0;
      for (int base = 0; base < p.g; base += kThreads) {
        int sz, rank, first_row, sa, sr;
        scan_slab(base, seen, rows_seen, sz, rank, first_row, sa, sr);
        if (sz > 0 && rank <= want && want < rank + (sz + RPP - 1) / RPP) {
          const int done = (want - rank) * RPP;
          job[0] = base + tid; job[1] = first_row + done; job[2] = imin(RPP, sz - done);
        }
        seen += sa; rows_seen += sr;
      }
    }
    __syncthreads();
    const int gi = job[0], row0 = job[1];
    const int rows = imin(job[2], p.m - row0);
    if (rows <= 0) continue;
    const unsigned char* W = reinterpret_cast<const unsigned char*>(p.A) + (size_t)gi * p.n * p.k * EB;
    // this wave's weight rows: blocks of kTBlock consecutive rows, block wave, wave + 4, ... of the piece (a piece is a
    // whole number of blocks); its loads as one sequence of (block, position) steps of kTBlock loads each
    const int blocks = (j_end - j_begin) / kTBlock;
    const int my_blocks = wave < blocks ? (blocks - wave + 3) >> 2 : 0;
    const int nsteps = my_blocks * npos;
    // step s: position s % npos of block s / npos; the chunk is clamped to the row (the activations past k are zero)
    auto load_step = [&](u32x4_t (&dst)[kTBlock], int s) {
      const int sc = imin(s, nsteps - 1);
      const int i = sc / npos, q = sc - i * npos;
      const int ch = imin(q * 64 + lane, chunks - 1);
      // byte offsets: n * k < 2^31 elements
      const uint32_t off = ((uint32_t)(j_begin + kTBlock * (wave + 4 * i)) * (uint32_t)p.k) * EB + (uint32_t)ch * 16u;
#pragma unroll
      for (int b = 0; b < kTBlock; ++b)
        dst[b] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(W + off + (uint32_t)b * (uint32_t)p.k * EB));
    };

    for (int rc = 0; rc < rows; rc += RMAX) {
      const int nr = imin(RMAX, rows - rc);
      u32x4_t w[kTDepth][kTBlock];
      if (nsteps > 0) {
#pragma unroll
        for (int u = 0; u < kTDepth; ++u) load_step(w[u], u);
      }
      __syncthreads();  // previous pass done with xs
      // stage the activations: entry [row][chunk] = the chunk's 8 (float8: [row][0 / 1][chunk] = its lower / upper 8)
      // contraction indices of x[row] as bf16; zero for rows past nr and for the chunks that pad the row to a whole
      // number of positions (unconditional loads from clamped, valid addresses, four in flight per thread; masked
      // afterwards)
      for (int base = 0; base < r_stride * RMAX; base += kThreads * 4) {
        u32x4_t v[4];
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2) {
          const int idx = base + s2 * kThreads + tid;
          const int r = imin(idx / r_stride, nr - 1), ch = imin(idx % r_stride, chunks - 1);
          v[s2] = *reinterpret_cast<const u32x4_t*>(xb + ((size_t)(row0 + rc + r) * p.k) * EB + (size_t)ch * 16);
        }
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2) {
          const int idx = base + s2 * kThreads + tid;
          const int r = idx / r_stride, ch = idx - r * r_stride;
          const bool live = r < nr && ch < chunks;
          if (idx < r_stride * RMAX) {
            if constexpr (F8) {
              const uint32_t c0 = v[s2][0], c1 = v[s2][1], c2 = v[s2][2], c3 = v[s2][3];
              const u32x4_t lo = {fp8e4m3x2_to_bf16x2<false>(c0), fp8e4m3x2_to_bf16x2<true>(c0),
                                  fp8e4m3x2_to_bf16x2<false>(c1), fp8e4m3x2_to_bf16x2<true>(c1)};
              const u32x4_t hi = {fp8e4m3x2_to_bf16x2<false>(c2), fp8e4m3x2_to_bf16x2<true>(c2),
                                  fp8e4m3x2_to_bf16x2<false>(c3), fp8e4m3x2_to_bf16x2<true>(c3)};
              xs[(2 * r) * r_stride + ch] = live ? lo : u32x4_t{0, 0, 0, 0};
              xs[(2 * r + 1) * r_stride + ch] = live ? hi : u32x4_t{0, 0, 0, 0};
            } else {
              xs[idx] = live ? v[s2] : u32x4_t{0, 0, 0, 0};
            }
          }
        }
      }
      __syncthreads();
      if (nsteps <= 0) continue;

      float acc[kTBlock][RMAX];
#pragma unroll
      for (int b = 0; b < kTBlock; ++b)
#pragma unroll
        for (int r = 0; r < RMAX; ++r) acc[b][r] = 0.f;
      int q = 0, i = 0;  // position in the rows, block of this wave
      for (int base = 0; base < nsteps; base += kTDepth) {
#pragma unroll
        for (int u = 0; u < kTDepth; ++u) {
          if (base + u < nsteps) {  // uniform over the wave
            const u32x4_t* xe = xs + (q * 64 + lane);
            // the block's weights as pairs of bf16 (float8: widened here, once for all token rows).
            // Scalars first: a bit cast applied to one element of a vector reads element 0 whatever the index.
            uint32_t wp[kTBlock][4 * XE];
#pragma unroll
            for (int b = 0; b < kTBlock; ++b) {
              const uint32_t w0 = w[u][b][0], w1 = w[u][b][1], w2 = w[u][b][2], w3 = w[u][b][3];
              if constexpr (F8) {
                wp[b][0] = fp8e4m3x2_to_bf16x2<false>(w0); wp[b][1] = fp8e4m3x2_to_bf16x2<true>(w0);
                wp[b][2] = fp8e4m3x2_to_bf16x2<false>(w1); wp[b][3] = fp8e4m3x2_to_bf16x2<true>(w1);
                wp[b][4] = fp8e4m3x2_to_bf16x2<false>(w2); wp[b][5] = fp8e4m3x2_to_bf16x2<true>(w2);
                wp[b][6] = fp8e4m3x2_to_bf16x2<false>(w3); wp[b][7] = fp8e4m3x2_to_bf16x2<true>(w3);
              } else {
                wp[b][0] = w0; wp[b][1] = w1; wp[b][2] = w2; wp[b][3] = w3;
              }
            }
#pragma unroll
            for (int r = 0; r < RMAX; ++r) {
              // one read of the token row's activations serves the block's kTBlock weight rows
#pragma unroll
              for (int h = 0; h < XE; ++h) {
                const u32x4_t xv = xe[(size_t)(XE * r + h) * r_stride];
                const uint32_t x0 = xv[0], x1 = xv[1], x2 = xv[2], x3 = xv[3];
#pragma unroll
                for (int b = 0; b < kTBlock; ++b) {
                  float a = acc[b][r];
                  a = dot2_f32<HALF>(wp[b][4 * h + 0], x0, a);
                  a = dot2_f32<HALF>(wp[b][4 * h + 1], x1, a);
                  a = dot2_f32<HALF>(wp[b][4 * h + 2], x2, a);
                  a = dot2_f32<HALF>(wp[b][4 * h + 3], x3, a);
                  acc[b][r] = a;
                }
              }
            }
            if (++q == npos) {
              // end of the block's rows: the 64 lanes' sums of all kTBlock x RMAX values; every lane ends up with one of
              // them, the first lane of each run of 64 / (kTBlock * RMAX) stores it
              constexpr int V = kTBlock * RMAX, RUN = 64 / V;
              float vals[V];
#pragma unroll
              for (int b = 0; b < kTBlock; ++b)
#pragma unroll
                for (int r = 0; r < RMAX; ++r) { vals[b * RMAX + r] = acc[b][r]; acc[b][r] = 0.f; }
              const float mine = wave_sums<V>(vals, lane);
              const int idx = lane / RUN;
              const int b = idx / RMAX, r = idx - b * RMAX;
              if (lane % RUN == 0 && r < nr)
                p.y[(size_t)(row0 + rc + r) * p.n + (j_begin + kTBlock * (wave + 4 * i) + b)] = round_out<HALF>(mine);
              q = 0; ++i;
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          load_step(w[u], base + kTDepth + u);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }
}

// y[row, :] = sum over the pieces of partials[row, piece, :] for rows below sum(group_sizes), zero above.
// Work-group = (row, block of 256 columns); thread = (8 columns, one of 8 piece lanes).
template <bool HALF>
__global__ __launch_bounds__(kThreads) void gmm_rows_finish_kernel(DecodeArgs p, const RowsHeader* __restrict__ header,
                                                                   const float* __restrict__ partials) {
  __shared__ float sums[8][32][8];
  const int tid = threadIdx.x;
  const int col_blocks = (p.n + 255) / 256;
  const int row = blockIdx.x / col_blocks, cb = blockIdx.x - row * col_blocks;
  const int C = header->pieces, total = header->total_rows;
  const int chunk = tid & 31, lane_s = tid >> 5;
  const int col = cb * 256 + chunk * 8;
  float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (row < total && col < p.n) {
    for (int s = lane_s; s < C; s += 8) {
      const f32x4_t* src = reinterpret_cast<const f32x4_t*>(partials + ((size_t)row * C + s) * p.n + col);
      const f32x4_t a = src[0], b = src[1];
      v[0] += a[0]; v[1] += a[1]; v[2] += a[2]; v[3] += a[3];
      v[4] += b[0]; v[5] += b[1]; v[6] += b[2]; v[7] += b[3];
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) sums[lane_s][chunk][e] = v[e];
  __syncthreads();
  if (lane_s == 0 && col < p.n) {
    float t[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      t[e] = 0.f;
#pragma unroll
      for (int s = 0; s < 8; ++s) t[e] += sums[s][chunk][e];
    }
    u32x4_t out;
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = round_out_x2<HALF>(t[2 * e], t[2 * e + 1]);
    *reinterpret_cast<u32x4_t*>(p.y + (size_t)row * p.n + col) = out;
  }
}

}  // namespace

int launch_gmm_decode(hipStream_t s, const DecodeArgs& a, int nb) {
  if (a.m <= 0 || a.n <= 0 || a.g <= 0) return hipSuccess;
  switch (nb) {
    case 32: return a.half ? launch_nb<32, true>(s, a) : launch_nb<32, false>(s, a);
    case 64: return a.half ? launch_nb<64, true>(s, a) : launch_nb<64, false>(s, a);
    case 128: return a.half ? launch_nb<128, true>(s, a) : launch_nb<128, false>(s, a);
    default: return hipErrorInvalidValue;
  }
}


size_t gmm_rows_workspace_bytes(int m, int n, int pieces) {
  return 256 + (size_t)m * n * sizeof(float) * (pieces > 0 ? pieces : 1);
}

namespace {

template <bool WIDE, bool HALF>
int launch_rows(hipStream_t s, const DecodeArgs& a, RowsGeom q, RowsHeader* header, float* partials) {
  q.min_rows = WIDE ? q.rps * 2 * kPairDepth * 2 : q.rps * kRowsDepth * 2;
  const size_t lds = WIDE ? (size_t)kXsBytes + (size_t)q.rps * kWideRows * a.n * sizeof(float)
                          : (size_t)kMaxSeg * 8 + (size_t)q.rps * kRows * a.n * sizeof(float);
  if (lds > 64 * 1024) {
    const int rc = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(gmm_rows_kernel<WIDE, HALF>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (rc != hipSuccess) return rc;
  }
  hipLaunchKernelGGL((gmm_rows_kernel<WIDE, HALF>), dim3(q.wgs), dim3(kThreads), lds, s, a, q, header, partials);
  return (int)hipGetLastError();
}

}  // namespace

int launch_gmm_rows(hipStream_t s, const DecodeArgs& a, int num_cus, void* workspace, size_t workspace_bytes) {
  if (a.m <= 0 || a.n <= 0 || a.g <= 0) return hipSuccess;
  if (a.n % 8 != 0 || a.n > 2048 || !workspace || (reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return hipErrorInvalidValue;
  const size_t per_piece = (size_t)a.m * a.n * sizeof(float);
  if (workspace_bytes < 256 + per_piece) return hipErrorInvalidValue;
  RowsGeom q;
  q.wgs = 2 * (num_cus > 0 ? num_cus : 256);  // measured best on the decode shape: more pieces cost more in partial sums than they gain in balance
  q.lpr = a.n / 8;
  q.rps = kThreads / q.lpr;
  q.max_c = (int)((workspace_bytes - 256) / per_piece < 1024 ? (workspace_bytes - 256) / per_piece : 1024);
  q.min_rows = 0;
  RowsHeader* header = static_cast<RowsHeader*>(workspace);
  float* partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + 256);
  // More than one row per group on average: some group has more than the four rows a narrow pass takes, and the
  // wide passes stream its weights once where the narrow ones would twice.
  const int rc = a.m > a.g ? (a.half ? launch_rows<true, true>(s, a, q, header, partials) : launch_rows<true, false>(s, a, q, header, partials))
                           : (a.half ? launch_rows<false, true>(s, a, q, header, partials) : launch_rows<false, false>(s, a, q, header, partials));
  if (rc != hipSuccess) return rc;
  const int col_blocks = (a.n + 255) / 256;
  if (a.half) hipLaunchKernelGGL(gmm_rows_finish_kernel<true>, dim3(a.m * col_blocks), dim3(kThreads), 0, s, a, header, partials);
  else hipLaunchKernelGGL(gmm_rows_finish_kernel<false>, dim3(a.m * col_blocks), dim3(kThreads), 0, s, a, header, partials);
  return (int)hipGetLastError();
}

// trans_rhs: A is [g, n, k].  Needs k % 8 == 0 (float8: 16), n % 8 == 0, n * k < 2^31 and rows-per-pass x k (padded to
// 64 chunks of 16 bytes) x 2 bytes of LDS within kTMaxLds.  No workspace.
bool gmm_rows_t_fits(int m, int k, int n, int g, bool f8) {
  (void)m; (void)n; (void)g;  // only the contraction length decides: 4 token rows of it must fit in LDS
  const long long pad = f8 ? 1023 : 511;
  const long long kpad = ((long long)k + pad) & ~pad;
  return k > 0 && 4 * kpad * 2 <= kTMaxLds;
}

int launch_gmm_rows_t(hipStream_t s, const DecodeArgs& a, int num_cus, bool f8) {
  if (a.m <= 0 || a.n <= 0 || a.g <= 0) return hipSuccess;
  if (a.n % 8 != 0 || a.k % (f8 ? 16 : 8) != 0 || a.k <= 0) return hipErrorInvalidValue;
  const int pad = f8 ? 1023 : 511;
  const int kpad = (a.k + pad) & ~pad;
  const int wgs = 2 * (num_cus > 0 ? num_cus : 256);
  // more than one row per group on average and room for them: 8 token rows per pass over the weights, else 4
  const bool wide = a.m > a.g && (size_t)8 * kpad * 2 <= (size_t)kTMaxLds;
  const size_t lds = (size_t)(wide ? 8 : 4) * kpad * 2;
  if (lds > (size_t)kTMaxLds) return hipErrorInvalidValue;
  if (f8) {
    if (a.half) return hipErrorInvalidValue;
    if (wide) hipLaunchKernelGGL((gmm_rows_t_kernel<8, true, false>), dim3(wgs), dim3(kThreads), lds, s, a, wgs);
    else hipLaunchKernelGGL((gmm_rows_t_kernel<4, true, false>), dim3(wgs), dim3(kThreads), lds, s, a, wgs);
  } else if (a.half) {
    if (wide) hipLaunchKernelGGL((gmm_rows_t_kernel<8, false, true>), dim3(wgs), dim3(kThreads), lds, s, a, wgs);
    else hipLaunchKernelGGL((gmm_rows_t_kernel<4, false, true>), dim3(wgs), dim3(kThreads), lds, s, a, wgs);
  } else {
    if (wide) hipLaunchKernelGGL((gmm_rows_t_kernel<8, false, false>), dim3(wgs), dim3(kThreads), lds, s, a, wgs);
    else hipLaunchKernelGGL((gmm_rows_t_kernel<4, false, false>), dim3(wgs), dim3(kThreads), lds, s, a, wgs);
  }
  return (int)hipGetLastError();
}

}  // namespace rd
