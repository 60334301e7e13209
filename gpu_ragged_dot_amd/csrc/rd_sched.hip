// group_sizes -> (tile -> group, tile -> index inside group, row offsets) scheduling map, as one prefix-sum
// kernel.  Produces exactly the five arrays of the reference's GMMGroupLookupMetadata
// (gpu_ragged_dot.py:60-90) in int32, every output element written once.
#include "rd_common.h"
#include "rd_sched.h"

namespace rd {

namespace {

constexpr int kSchedThreads = 1024;
constexpr int kSchedWaves = kSchedThreads / 64;

// floor(a / b) for b > 0, as numpy's // on int32.
__device__ __forceinline__ int32_t floor_div(int32_t a, int32_t b) {
  int32_t q = a / b;
  return (a % b != 0 && a < 0) ? q - 1 : q;
}

// Inclusive scan across the work-group of two values at once; every thread gets its inclusive sums and the
// work-group totals.  Sums wrap like int32 cumsum does.
__device__ __forceinline__ void block_scan2(uint32_t& a, uint32_t& b, uint32_t& total_a, uint32_t& total_b,
                                            uint32_t* wave_a, uint32_t* wave_b) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t ua = __shfl_up(a, d, 64), ub = __shfl_up(b, d, 64);
    if (lane >= d) { a += ua; b += ub; }
  }
  if (lane == 63) { wave_a[wave] = a; wave_b[wave] = b; }
  __syncthreads();
  uint32_t pa = 0, pb = 0, ta = 0, tb = 0;
#pragma unroll
  for (int w = 0; w < kSchedWaves; ++w) {
    const uint32_t xa = wave_a[w], xb = wave_b[w];
    if (w < wave) { pa += xa; pb += xb; }
    ta += xa; tb += xb;
  }
  a += pa; b += pb;
  total_a = ta; total_b = tb;
  __syncthreads();
}

constexpr int kSizeClasses = 33;
__device__ __forceinline__ int size_class(int32_t rows) { return rows <= 0 ? 0 : 32 - __clz(rows); }

__global__ __launch_bounds__(kSchedThreads) void sched_map_kernel(const int32_t* __restrict__ gs, int g, int U,
                                                                  int chunk, int32_t* __restrict__ group_offsets,
                                                                  int32_t* __restrict__ tile2group,
                                                                  int32_t* __restrict__ tile2it,
                                                                  int32_t* __restrict__ total_tiles,
                                                                  int32_t* __restrict__ counters, int n_counters,
                                                                  int32_t* __restrict__ tile2band, int band_rows,
                                                                  int32_t* __restrict__ block_order, int n_blocks,
                                                                  int per_block, int n_tiles, int long_rows,
                                                                  int32_t* __restrict__ group_order, int order_first,
                                                                  int order_count, int defer_rows, int defer_cus,
                                                                  int defer_slots) {
  // arrival counters of the K-split tiles of the launch that follows start at zero
  for (int i = threadIdx.x; i < n_counters; i += kSchedThreads) counters[i] = 0;
  __shared__ uint32_t wave_a[kSchedWaves], wave_b[kSchedWaves];
  __shared__ int32_t incl[kSchedThreads];  // inclusive tile-count scan of the current slab of groups
  __shared__ int32_t incl_d[kSchedThreads], tiles_of[kSchedThreads];  // deferred tiles: their scan, and every group's tile count
  const int tid = threadIdx.x;
  uint32_t carry_rows = 0, carry_tiles = 0, carry_def = 0;

  // defer_rows > 0 (gmm launches of the cores that have the streaming routines, when the last round of tiles is cut along
  // K; never the map rd_sched_map returns): the last row tile of a group of several row tiles, when it holds at most
  // defer_rows rows, may be taken out of its group's run of tiles and listed behind all other tiles, as a band of its
  // own with the kBandDeferred mark.  That is done when all such tiles then fall into the partly filled last round of
  // the launch (defer_cus tiles run at a time) and that round is cut along K (at most defer_slots / 2 tiles in it): the
  // rounds before it then hold whole tiles of full height only - the layout of a dense product - and the pieces of the
  // last round, which run alone at the end of the launch either way, go through the streaming routines instead of the
  // tall one.  Anywhere else a tile moved out of its group's run would cost a pass of its own over the group's weights.
  bool defer_on = false;
  auto deferred = [&](int32_t sz, int32_t bpg) {
    return defer_on && bpg >= 2 && sz - (bpg - 1) * chunk <= defer_rows ? 1 : 0;
  };
  uint32_t total_regular = 0;
  if (defer_rows > 0 && defer_cus > 0) {  // count the candidates and all tiles, then decide
    uint32_t all = 0, cand = 0;
    defer_on = true;
    for (int base = 0; base < g; base += kSchedThreads) {
      const int gi = base + tid;
      const int32_t sz = gi < g ? gs[gi] : 0;
      const int32_t bpg = gi < g ? floor_div(sz + chunk - 1, chunk) : 0;
      uint32_t a = (uint32_t)imax(bpg, 0), b = (uint32_t)deferred(sz, bpg), ta, tb;
      block_scan2(a, b, ta, tb, wave_a, wave_b);
      all += ta; cand += tb;
    }
    const long long live = (long long)imin((int32_t)all, U) * n_tiles;
    const long long first = live / defer_cus * defer_cus;  // where the last round starts
    defer_on = cand > 0 && (long long)(all - cand) * n_tiles >= first && (live - first) * 2 <= defer_slots && all <= (uint32_t)U;
    total_regular = all - cand;
  }

  for (int base = 0; base < g; base += kSchedThreads) {
    const int gi = base + tid;
    const int32_t sz = gi < g ? gs[gi] : 0;
    const int32_t bpg_all = gi < g ? floor_div(sz + chunk - 1, chunk) : 0;  // gpu_ragged_dot.py:73
    const int32_t dfr = deferred(sz, bpg_all);
    const int32_t bpg = bpg_all - dfr;  // tiles in the group's own run
    uint32_t a = (uint32_t)sz, b = (uint32_t)bpg, ta, tb;
    block_scan2(a, b, ta, tb, wave_a, wave_b);
    if (gi < g) group_offsets[gi] = (int32_t)(carry_rows + a - (uint32_t)sz);  // :86
    incl[tid] = (int32_t)(carry_tiles + b);
    uint32_t td = 0;
    if (defer_on) {
      uint32_t c = (uint32_t)dfr, z = 0, tz;
      block_scan2(c, z, td, tz, wave_a, wave_b);
      incl_d[tid] = (int32_t)(carry_def + c);
      tiles_of[tid] = bpg_all;
    }
    __syncthreads();

    // Tiles [carry_tiles, carry_tiles + tb) belong to this slab of groups (:76-82).
    const int32_t lo = (int32_t)carry_tiles, hi = (int32_t)(carry_tiles + tb);
    const int cnt = imin(kSchedThreads, g - base);
    for (int32_t t = imax(lo, 0) + tid; t < hi && t < U; t += kSchedThreads) {
      int l = 0, r = cnt;  // first j with incl[j] > t; empty groups repeat their predecessor and are skipped
      while (l < r) {
        const int mid = (l + r) >> 1;
        if (incl[mid] > t) r = mid; else l = mid + 1;
      }
      const int32_t start = l == 0 ? lo : incl[l - 1];
      tile2group[t] = base + l;
      tile2it[t] = t - start;
      if (tile2band) {
        // The group's R row tiles are cut into ceil(R / band_rows) bands of nearly equal height (the first R % bands of
        // them one taller), so that no band spans two groups; the entry says where this tile's band starts and how tall
        // it is.
        const int32_t R = incl[l] - start, it = t - start;
        const int32_t nb = (R + band_rows - 1) / band_rows, r = R / nb, rem = R - r * nb;
        int32_t row0, rb;
        if (it < rem * (r + 1)) { rb = r + 1; row0 = (it / rb) * rb; }
        else { rb = r; row0 = rem * (r + 1) + ((it - rem * (r + 1)) / rb) * rb; }
        tile2band[t] = ((start + row0) << kBandShift) | rb;
      }
    }
    // The deferred tiles of this slab of groups: slots total_regular + [carry_def, carry_def + td), each a band of its own.
    if (defer_on) {
      const int cnt_d = imin(kSchedThreads, g - base);
      for (int32_t j = (int32_t)carry_def + tid; j < (int32_t)(carry_def + td); j += kSchedThreads) {
        int l = 0, r = cnt_d;  // first group of the slab with incl_d > j
        while (l < r) {
          const int mid = (l + r) >> 1;
          if (incl_d[mid] > j) r = mid; else l = mid + 1;
        }
        const int32_t slot = (int32_t)total_regular + j;
        if (slot >= 0 && slot < U) {
          tile2group[slot] = base + l;
          tile2it[slot] = tiles_of[l] - 1;
          if (tile2band) tile2band[slot] = kBandDeferred | (slot << kBandShift) | 1;
        }
      }
    }
    carry_rows += ta;
    carry_tiles += tb;
    carry_def += td;
    __syncthreads();
  }
  carry_tiles += carry_def;  // all tiles
  // Unused slots read as zero (the masked sums of :81-82 are empty there).
  for (int32_t t = imax((int32_t)carry_tiles, 0) + tid; t < U; t += kSchedThreads) {
    tile2group[t] = 0;
    tile2it[t] = 0;
    if (tile2band) tile2band[t] = (t << kBandShift) | 1;  // the slots that zero the rows past sum(group_sizes): one-tile bands
  }
  if (tid == 0) *total_tiles = (int32_t)carry_tiles;  // :89

  if (block_order) {
    // The blocks of the gmm tile walk, sorted into those of long groups (from the front) and the others (from the back);
    // a block is judged by its first position.
    __threadfence_block();
    __syncthreads();  // the map above is complete
    const int total = imax(imin((int32_t)carry_tiles, U), 0);
    const int live_blocks = imin((int)(((long long)total * n_tiles + per_block - 1) / per_block), n_blocks);
    int32_t* order = block_order + 2;
    uint32_t carry_l = 0, carry_s = 0;
    for (int base = 0; base < live_blocks; base += kSchedThreads) {
      const int b = base + tid;
      bool is_long = false, is_short = false;
      if (b < live_blocks) {
        // (a long group's short last tile that was moved behind the others counts as short: it streams)
        const int slot = imin((int)(((long long)b * per_block) / n_tiles), total - 1);
        is_long = gs[tile2group[slot]] > long_rows && !(tile2band && (tile2band[slot] & kBandDeferred));
        is_short = !is_long;
      }
      uint32_t a = is_long, c = is_short, ta, tc;
      block_scan2(a, c, ta, tc, wave_a, wave_b);
      if (is_long) order[carry_l + a - 1] = b;
      if (is_short) order[n_blocks - 1 - (int)(carry_s + c - 1)] = b;
      carry_l += ta;
      carry_s += tc;
    }
    if (tid == 0) { block_order[0] = (int32_t)carry_l; block_order[1] = (int32_t)(carry_l + carry_s); }
  }
  if (group_order) {
    __threadfence_block();  // group_offsets, written above by other threads of this work-group, are read below
    // tgmm: groups [order_first, order_first + order_count) listed by falling size class (bit length of the row count:
    // 0, 1, 2-3, 4-7, ...), groups of one class in index order - a stable counting sort over 33 classes.
    __shared__ int32_t cls_base[kSizeClasses], cls_wave[kSchedWaves][kSizeClasses];
    __syncthreads();
    if (tid < kSizeClasses) cls_base[tid] = 0;
    __syncthreads();
    for (int i = tid; i < order_count; i += kSchedThreads) atomicAdd(&cls_base[size_class(gs[order_first + i])], 1);
    __syncthreads();
    if (tid == 0) {
      int32_t run = 0;
      for (int c = kSizeClasses - 1; c >= 0; --c) { const int32_t cnt = cls_base[c]; cls_base[c] = run; run += cnt; }
    }
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6;
    for (int base = 0; base < order_count; base += kSchedThreads) {
      const int i = base + tid;
      const int c = i < order_count ? size_class(gs[order_first + i]) : -1;
      int rank = 0;
      for (int cc = 0; cc < kSizeClasses; ++cc) {
        const unsigned long long mask = __ballot(c == cc);
        if (c == cc) rank = __popcll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) cls_wave[wave][cc] = __popcll(mask);
      }
      __syncthreads();
      if (c >= 0) {
        int32_t before = cls_base[c];
        for (int w = 0; w < wave; ++w) before += cls_wave[w][c];
        // one record per position: the group, its first row and its row count, so that a tile of the launch finds all
        // three with a single load
        int32_t* rec = group_order + 4 * (before + rank);
        rec[0] = i; rec[1] = group_offsets[order_first + i]; rec[2] = gs[order_first + i]; rec[3] = 0;
      }
      __syncthreads();
      if (tid < kSizeClasses) {
        int32_t tot = 0;
        for (int w = 0; w < kSchedWaves; ++w) tot += cls_wave[w][tid];
        cls_base[tid] += tot;
      }
      __syncthreads();
    }
  }
}

template <typename T>
__global__ void fill_kernel(T* p, size_t n, T v) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

// Load-only kernel: work-group b reads block b (block_bytes contiguous bytes, the last one shorter) with streaming
// 16-byte loads and folds what it read into one word that is stored only if it equals a value the caller never expects,
// which keeps the loads alive without a store stream.
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4_t* __restrict__ src, size_t n16, size_t block16,
                                                          uint32_t* __restrict__ sink, uint32_t never) {
  const size_t lo = (size_t)blockIdx.x * block16, hi = lo + block16 < n16 ? lo + block16 : n16;
  u32x4_t acc = {0, 0, 0, 0};
  size_t i = lo + threadIdx.x;
  for (; i + 3 * 256 < hi; i += 4 * 256) {  // four independent loads in flight per thread
    const u32x4_t a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + 256);
    const u32x4_t c = __builtin_nontemporal_load(src + i + 512), d = __builtin_nontemporal_load(src + i + 768);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < hi; i += 256) acc ^= __builtin_nontemporal_load(src + i);
  const uint32_t w = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (w == never && sink) *sink = w;
}

}  // namespace

int launch_stream_read(hipStream_t s, const void* src, size_t bytes, size_t block_bytes, void* sink) {
  const size_t n16 = bytes / 16, block16 = block_bytes / 16;
  if (n16 == 0 || block16 == 0) return hipSuccess;
  const size_t blocks = (n16 + block16 - 1) / block16;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const u32x4_t*>(src), n16, block16,
                     static_cast<uint32_t*>(sink), 0x9e3779b9u);
  return (int)hipGetLastError();
}

int launch_sched_map(hipStream_t s, const int32_t* gs, int g, int m, int chunk, int32_t* group_offsets,
                     int32_t* tile2group, int32_t* tile2it, int32_t* total_tiles, int32_t* counters, int n_counters,
                     int32_t* tile2band, int band_rows, int32_t* block_order, int n_blocks, int per_block, int n_tiles,
                     int long_rows, int32_t* group_order, int order_first, int order_count, int defer_rows,
                     int defer_cus, int defer_slots) {
  const int U = (m + chunk - 1) / chunk + g;  // gpu_ragged_dot.py:77
  if (band_rows < 1) band_rows = 1;
  if (band_rows > kBandMaxRows) band_rows = kBandMaxRows;
  hipLaunchKernelGGL(sched_map_kernel, dim3(1), dim3(kSchedThreads), 0, s, gs, g, U, chunk, group_offsets,
                     tile2group, tile2it, total_tiles, counters, counters ? n_counters : 0, tile2band, band_rows,
                     n_blocks > 0 ? block_order : nullptr, n_blocks, per_block > 0 ? per_block : 1, n_tiles > 0 ? n_tiles : 1,
                     long_rows, order_count > 0 ? group_order : nullptr, order_first, order_count, tile2band ? defer_rows : 0, defer_cus,
                     defer_slots);
  return (int)hipGetLastError();
}

int launch_zero_bytes(hipStream_t s, void* p, size_t bytes) {
  if (bytes == 0) return hipSuccess;
  // Callers may be under graph capture, where memset nodes are unreliable: clear with a plain kernel.
  if (bytes % 4 == 0 && (reinterpret_cast<uintptr_t>(p) % 4) == 0) {
    const size_t n = bytes / 4;
    const int grid = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    hipLaunchKernelGGL(fill_kernel<uint32_t>, dim3(grid), dim3(256), 0, s, (uint32_t*)p, n, 0u);
  } else {
    const int grid = (int)((bytes + 255) / 256 < 4096 ? (bytes + 255) / 256 : 4096);
    hipLaunchKernelGGL(fill_kernel<uint8_t>, dim3(grid), dim3(256), 0, s, (uint8_t*)p, bytes, (uint8_t)0);
  }
  return (int)hipGetLastError();
}

}  // namespace rd
