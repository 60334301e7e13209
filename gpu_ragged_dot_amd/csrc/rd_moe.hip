// Token routing around ragged_dot: the rows ragged_dot takes must be sorted by group, and its output rows go back
// to their tokens.  The reference leaves both steps to its caller (its tests build sorted rows directly,
// tests.py:51-71); these kernels are that caller's side, kept on the device so that group_sizes never visits the host.
//
//   route    : expert id per (token, slot)  ->  group_sizes, row_of_slot, slot_of_row     (stable counting sort)
//   dispatch : x[row] = h[token of the row's slot]  (optionally scaled per slot)          (row gather)
//   combine  : out[token] = sum over its slots of weight * y[row of slot]                 (row gather + sum)
//   combine_wgrad : dw[token, slot] = <y[row of slot], dout[token]>
//
// All of it is integer / byte work bound by HBM: rows move as 16-byte pieces, one work-group per row or token.
#include "rd_common.h"
#include "rd_moe.h"

namespace rd {

namespace {

constexpr int kScanThreads = 1024;

// ---- route -----------------------------------------------------------------------------------------------------------

// hist[b][e] = number of kept slots of chunk b that go to expert e.
__global__ __launch_bounds__(64) void moe_hist_kernel(const int32_t* __restrict__ ids, int S, int g, int chunk,
                                                      int32_t* __restrict__ hist) {
  extern __shared__ int32_t cnt[];
  const int lane = threadIdx.x, b = blockIdx.x;
  for (int e = lane; e < g; e += 64) cnt[e] = 0;
  __syncthreads();
  const int end = (int)(((long long)(b + 1) * chunk < S) ? (long long)(b + 1) * chunk : S);
  for (int s = b * chunk + lane; s < end; s += 64) {
    const int e = ids[s];
    if (e >= 0 && e < g) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  for (int e = lane; e < g; e += 64) hist[(size_t)b * g + e] = cnt[e];
}

// Per expert: exclusive running sum of hist over the chunks (in place) and the total = group_sizes[e]; then the
// exclusive sum of the totals over the experts = first row of each group; rows past the last group get slot -1.
__global__ __launch_bounds__(kScanThreads) void moe_scan_kernel(int32_t* __restrict__ hist, int nb, int g, int S,
                                                                int32_t* __restrict__ group_sizes,
                                                                int32_t* __restrict__ group_first,
                                                                int32_t* __restrict__ slot_of_row) {
  __shared__ int32_t wave_sum[kScanThreads / 64];
  __shared__ int32_t carry_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int base = 0; base < g; base += kScanThreads) {
    const int e = base + tid;
    int total = 0;
    if (e < g) {
      for (int b0 = 0; b0 < nb; b0 += 8) {  // eight independent loads at a time, then their running sums
        int32_t c[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) c[u] = b0 + u < nb ? hist[(size_t)(b0 + u) * g + e] : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (b0 + u < nb) hist[(size_t)(b0 + u) * g + e] = total;
          total += c[u];
        }
      }
      group_sizes[e] = total;
    }
    // exclusive scan of `total` over this slab of experts
    int incl = total;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = carry_s;
    for (int w = 0; w < wave; ++w) before += wave_sum[w];
    if (e < g) group_first[e] = before + incl - total;
    __syncthreads();
    if (tid == kScanThreads - 1) carry_s = before + incl;
    __syncthreads();
  }
  const int total_rows = carry_s;
  for (int r = total_rows + tid; r < S; r += kScanThreads) slot_of_row[r] = -1;
}

// Stable rank of every slot inside its chunk, chunk by 64 slots at a time: lanes of one expert find each other with
// one ballot per id bit; the expert's running position lives in LDS.
__global__ __launch_bounds__(64) void moe_rank_kernel(const int32_t* __restrict__ ids, int S, int g, int chunk, int id_bits,
                                                      const int32_t* __restrict__ hist,
                                                      const int32_t* __restrict__ group_first,
                                                      int32_t* __restrict__ row_of_slot,
                                                      int32_t* __restrict__ slot_of_row) {
  extern __shared__ int32_t pos[];
  const int lane = threadIdx.x, b = blockIdx.x;
  for (int e = lane; e < g; e += 64) pos[e] = group_first[e] + hist[(size_t)b * g + e];
  __syncthreads();
  const int end = (int)(((long long)(b + 1) * chunk < S) ? (long long)(b + 1) * chunk : S);
  const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int s0 = b * chunk; s0 < end; s0 += 64) {
    const int s = s0 + lane;
    const int e = s < end ? ids[s] : -1;
    const bool keep = e >= 0 && e < g;
    unsigned long long same = __ballot(keep);
    for (int bit = 0; bit < id_bits; ++bit) {
      const bool one = (e >> bit) & 1;
      const unsigned long long ones = __ballot(keep && one);
      same &= one ? ones : ~ones;
    }
    int row = -1;
    if (keep) row = pos[e] + __popcll(same & below);
    __builtin_amdgcn_wave_barrier();  // every lane has read its expert's position before any leader moves it
    if (keep && (same & below) == 0) pos[e] = row + __popcll(same);
    __builtin_amdgcn_wave_barrier();
    if (s < end) row_of_slot[s] = row;
    if (keep) slot_of_row[row] = s;
  }
}

// ---- rows ------------------------------------------------------------------------------------------------------------

template <class T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<bf16_bits>(bf16_bits v) { return bf16_to_f32(v); }
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<f16_t>(f16_t v) { return (float)v; }
template <class T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ bf16_bits from_f32<bf16_bits>(float v) { return f32_to_bf16(v); }
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float v) { return (f16_t)v; }

constexpr int kRowThreads = 256;

// x[row_of_slot[t, s]] = h[t] * scale[t, s] for every kept slot of token t: the token's row is read once and written
// top_k times.  The rows past sum(group_sizes) (slot_of_row = -1) are zeroed by the work-group that owns their index
// (row r belongs to work-group r / top_k for this purpose only).  VEC: rows are whole 16-byte pieces at 16-byte
// aligned addresses.
template <class T, bool VEC>
__global__ __launch_bounds__(kRowThreads) void moe_dispatch_kernel(const T* __restrict__ h,
                                                                   const int32_t* __restrict__ row_of_slot,
                                                                   const int32_t* __restrict__ slot_of_row,
                                                                   const float* __restrict__ row_scale, T* __restrict__ x,
                                                                   int top_k, int d) {
  __shared__ int32_t rows[kMoeMaxTopK];
  __shared__ int32_t zero_row[kMoeMaxTopK];
  __shared__ float sc[kMoeMaxTopK];
  const int t = blockIdx.x, tid = threadIdx.x;
  if (tid < top_k) {
    const size_t slot = (size_t)t * top_k + tid;
    rows[tid] = row_of_slot[slot];
    sc[tid] = row_scale ? row_scale[slot] : 1.f;
    zero_row[tid] = slot_of_row[slot] < 0 ? (int32_t)slot : -1;
  }
  __syncthreads();
  constexpr int PER = 16 / sizeof(T);
  const T* src = h + (size_t)t * d;
  if (VEC) {
    const int pieces = d / PER;
    for (int c0 = tid; c0 < pieces; c0 += 4 * kRowThreads) {
      u32x4_t v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)  // clamped: always a valid piece, stored only if in range
        v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src) + imin(c0 + u * kRowThreads, pieces - 1));
      for (int s = 0; s < top_k; ++s) {
        if (rows[s] < 0) continue;
        u32x4_t* dst = reinterpret_cast<u32x4_t*>(x + (size_t)rows[s] * d);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (c0 + u * kRowThreads >= pieces) continue;
          u32x4_t o = v[u];
          if (row_scale) {
            alignas(16) T e[PER];
            *reinterpret_cast<u32x4_t*>(e) = o;
#pragma unroll
            for (int i = 0; i < PER; ++i) e[i] = from_f32<T>(to_f32<T>(e[i]) * sc[s]);
            o = *reinterpret_cast<u32x4_t*>(e);
          }
          dst[c0 + u * kRowThreads] = o;
        }
      }
    }
    for (int s = 0; s < top_k; ++s)
      if (zero_row[s] >= 0)
        for (int c = tid; c < pieces; c += kRowThreads)
          reinterpret_cast<u32x4_t*>(x + (size_t)zero_row[s] * d)[c] = u32x4_t{0, 0, 0, 0};
  } else {
    for (int c = tid; c < d; c += kRowThreads) {
      const float v = to_f32<T>(src[c]);
      for (int s = 0; s < top_k; ++s)
        if (rows[s] >= 0) x[(size_t)rows[s] * d + c] = row_scale ? from_f32<T>(v * sc[s]) : src[c];
    }
    for (int s = 0; s < top_k; ++s)
      if (zero_row[s] >= 0)
        for (int c = tid; c < d; c += kRowThreads) x[(size_t)zero_row[s] * d + c] = from_f32<T>(0.f);
  }
}

// out[t] = sum_s weights[t, s] * y[row_of_slot[t, s]], fp32, slots in order.
template <class T, bool VEC>
__global__ __launch_bounds__(kRowThreads) void moe_combine_kernel(const T* __restrict__ y,
                                                                  const int32_t* __restrict__ row_of_slot,
                                                                  const float* __restrict__ weights, T* __restrict__ out,
                                                                  int top_k, int d) {
  __shared__ int32_t rows[kMoeMaxTopK];
  __shared__ float ws[kMoeMaxTopK];
  const int t = blockIdx.x, tid = threadIdx.x;
  if (tid < top_k) {
    rows[tid] = row_of_slot[(size_t)t * top_k + tid];
    ws[tid] = weights ? weights[(size_t)t * top_k + tid] : 1.f;
  }
  __syncthreads();
  constexpr int PER = 16 / sizeof(T);
  T* dst = out + (size_t)t * d;
  if (VEC) {
    for (int c = tid; c < d / PER; c += kRowThreads) {
      float acc[PER];
#pragma unroll
      for (int e = 0; e < PER; ++e) acc[e] = 0.f;
      for (int s = 0; s < top_k; ++s) {
        if (rows[s] < 0) continue;
        alignas(16) T v[PER];
        *reinterpret_cast<u32x4_t*>(v) = reinterpret_cast<const u32x4_t*>(y + (size_t)rows[s] * d)[c];
#pragma unroll
        for (int e = 0; e < PER; ++e) acc[e] = __builtin_fmaf(ws[s], to_f32<T>(v[e]), acc[e]);
      }
      alignas(16) T o[PER];
#pragma unroll
      for (int e = 0; e < PER; ++e) o[e] = from_f32<T>(acc[e]);
      reinterpret_cast<u32x4_t*>(dst)[c] = *reinterpret_cast<u32x4_t*>(o);
    }
  } else {
    for (int c = tid; c < d; c += kRowThreads) {
      float acc = 0.f;
      for (int s = 0; s < top_k; ++s)
        if (rows[s] >= 0) acc = __builtin_fmaf(ws[s], to_f32<T>(y[(size_t)rows[s] * d + c]), acc);
      dst[c] = from_f32<T>(acc);
    }
  }
}

// dw[t, s] = <y[row_of_slot[t, s]], dout[t]>, fp32.
template <class T>
__global__ __launch_bounds__(kRowThreads) void moe_combine_wgrad_kernel(const T* __restrict__ y,
                                                                        const T* __restrict__ dout,
                                                                        const int32_t* __restrict__ row_of_slot,
                                                                        float* __restrict__ dw, int top_k, int d) {
  __shared__ float part[kRowThreads / 64];
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* g = dout + (size_t)t * d;
  for (int s = 0; s < top_k; ++s) {
    const int row = __builtin_amdgcn_readfirstlane(row_of_slot[(size_t)t * top_k + s]);
    float acc = 0.f;
    if (row >= 0) {
      const T* yr = y + (size_t)row * d;
      for (int c = tid; c < d; c += kRowThreads) acc = __builtin_fmaf(to_f32<T>(yr[c]), to_f32<T>(g[c]), acc);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) acc += __shfl_xor(acc, o, 64);
    __syncthreads();  // previous slot's partials consumed
    if (lane == 0) part[wave] = acc;
    __syncthreads();
    if (tid == 0) dw[(size_t)t * top_k + s] = part[0] + part[1] + part[2] + part[3];
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

// Slots per single-wave work-group of the histogram and ranking kernels: short chunks for parallelism, longer ones
// when the per-chunk histograms ([chunks][g] int32 in the workspace) would get large.
static int route_chunk(long long slots, int g) {
  int chunk = 512;
  while (((slots + chunk - 1) / chunk) * g > (4ll << 20) && chunk < (1 << 20)) chunk *= 2;
  return chunk;
}

size_t moe_route_workspace_bytes(long long slots, int g) {
  const int chunk = route_chunk(slots, g);
  const long long nb = (slots + chunk - 1) / chunk;
  return (size_t)(nb * g + g) * sizeof(int32_t);
}

int launch_moe_route(hipStream_t s, const int32_t* ids, int slots, int g, int32_t* group_sizes, int32_t* row_of_slot,
                     int32_t* slot_of_row, int32_t* workspace) {
  const int chunk = route_chunk(slots, g);
  const int nb = (slots + chunk - 1) / chunk;
  int32_t* hist = workspace;
  int32_t* group_first = workspace + (size_t)nb * g;
  int id_bits = 0;
  while ((1 << id_bits) < g) ++id_bits;
  const size_t lds = (size_t)g * sizeof(int32_t);
  if (nb > 0) hipLaunchKernelGGL(moe_hist_kernel, dim3(nb), dim3(64), lds, s, ids, slots, g, chunk, hist);
  hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(kScanThreads), 0, s, hist, nb, g, slots, group_sizes, group_first,
                     slot_of_row);
  if (nb > 0)
    hipLaunchKernelGGL(moe_rank_kernel, dim3(nb), dim3(64), lds, s, ids, slots, g, chunk, id_bits, hist, group_first,
                       row_of_slot, slot_of_row);
  return (int)hipGetLastError();
}

template <class T>
static int dispatch_t(hipStream_t s, const void* h, const int32_t* row_of_slot, const int32_t* slot_of_row,
                      const float* row_scale, void* x, int tokens, int top_k, int d) {
  const bool vec = (d * sizeof(T)) % 16 == 0 && aligned16(h) && aligned16(x);
  if (vec) hipLaunchKernelGGL((moe_dispatch_kernel<T, true>), dim3(tokens), dim3(kRowThreads), 0, s, (const T*)h, row_of_slot, slot_of_row, row_scale, (T*)x, top_k, d);
  else hipLaunchKernelGGL((moe_dispatch_kernel<T, false>), dim3(tokens), dim3(kRowThreads), 0, s, (const T*)h, row_of_slot, slot_of_row, row_scale, (T*)x, top_k, d);
  return (int)hipGetLastError();
}

int launch_moe_dispatch(hipStream_t s, const void* h, const int32_t* row_of_slot, const int32_t* slot_of_row,
                        const float* row_scale, void* x, int tokens, int top_k, int d, int elem) {
  if (tokens <= 0 || d <= 0) return hipSuccess;
  return elem == 1 ? dispatch_t<float>(s, h, row_of_slot, slot_of_row, row_scale, x, tokens, top_k, d)
       : elem == 2 ? dispatch_t<f16_t>(s, h, row_of_slot, slot_of_row, row_scale, x, tokens, top_k, d)
                   : dispatch_t<bf16_bits>(s, h, row_of_slot, slot_of_row, row_scale, x, tokens, top_k, d);
}

template <class T>
static int combine_t(hipStream_t s, const void* y, const int32_t* row_of_slot, const float* weights, void* out,
                     int tokens, int top_k, int d) {
  const bool vec = (d * sizeof(T)) % 16 == 0 && aligned16(y) && aligned16(out);
  if (vec) hipLaunchKernelGGL((moe_combine_kernel<T, true>), dim3(tokens), dim3(kRowThreads), 0, s, (const T*)y, row_of_slot, weights, (T*)out, top_k, d);
  else hipLaunchKernelGGL((moe_combine_kernel<T, false>), dim3(tokens), dim3(kRowThreads), 0, s, (const T*)y, row_of_slot, weights, (T*)out, top_k, d);
  return (int)hipGetLastError();
}

int launch_moe_combine(hipStream_t s, const void* y, const int32_t* row_of_slot, const float* weights, void* out,
                       int tokens, int top_k, int d, int elem) {
  if (tokens <= 0 || d <= 0) return hipSuccess;
  return elem == 1 ? combine_t<float>(s, y, row_of_slot, weights, out, tokens, top_k, d)
       : elem == 2 ? combine_t<f16_t>(s, y, row_of_slot, weights, out, tokens, top_k, d)
                   : combine_t<bf16_bits>(s, y, row_of_slot, weights, out, tokens, top_k, d);
}

int launch_moe_combine_wgrad(hipStream_t s, const void* y, const void* dout, const int32_t* row_of_slot, float* dw,
                             int tokens, int top_k, int d, int elem) {
  if (tokens <= 0 || top_k <= 0) return hipSuccess;
  if (elem == 2) hipLaunchKernelGGL(moe_combine_wgrad_kernel<f16_t>, dim3(tokens), dim3(kRowThreads), 0, s, (const f16_t*)y, (const f16_t*)dout, row_of_slot, dw, top_k, d);
  else if (elem == 1) hipLaunchKernelGGL(moe_combine_wgrad_kernel<float>, dim3(tokens), dim3(kRowThreads), 0, s, (const float*)y, (const float*)dout, row_of_slot, dw, top_k, d);
  else hipLaunchKernelGGL(moe_combine_wgrad_kernel<bf16_bits>, dim3(tokens), dim3(kRowThreads), 0, s, (const bf16_bits*)y, (const bf16_bits*)dout, row_of_slot, dw, top_k, d);
  return (int)hipGetLastError();
}

}  // namespace rd
