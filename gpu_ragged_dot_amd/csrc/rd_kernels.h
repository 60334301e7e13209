// Grouped-GEMM kernels built on gemm_tile(): launch-index -> tile mapping, group lookup through the scheduling
// map, tail / empty-group zeroing.
#pragma once
#include "rd_gemm_dlds.h"
#include "rd_gemm_f32.h"
#include "rd_gemm_f8.h"
#include "rd_gemm_w4.h"
#include "rd_gemm_w4r.h"
#include "rd_gemm_pp.h"
#include "rd_gemm_tile.h"
#include "rd_sched.h"

namespace rd {

// y[m, n] = ragged x[m, k] . A[g]  (A is [g, k, n], or [g, n, k] when trans_rhs).
struct GmmArgs {
  const void* x;  // element type is the kernel configuration's Elem (bf16 bits or float)
  const void* A;
  void* y;
  const int32_t* group_sizes;    // [g]
  const int32_t* group_offsets;  // [g]   exclusive prefix sum of group_sizes
  const int32_t* tile2group;     // [U]   scheduling map built with chunk = tile height
  const int32_t* tile2it;        // [U]
  const int32_t* tile2band;      // [U]   band of row tiles each row tile belongs to (see rd_sched.h)
  const int32_t* total_tiles;    // [1]
  int m, k, n, g;  // g: all groups of group_sizes
  int g_first, g_local;  // A holds the g_local groups [g_first, g_first + g_local); rows of the others are zero
  int U;        // static bound on row tiles: ceil(m / BM) + g
  int n_tiles;  // ceil(n / BN)
  int group_m, group_n;  // tile walk: most row tiles per band; positions per block = group_m x group_n
  // K-split of the last, partly filled round of tiles (kernels whose configuration has SPLITK; 0 slots = off)
  float* partials;     // [split_slots][BM * BN] fp32
  int32_t* counters;   // [split_slots], zero at launch
  int split_slots;     // work-groups appended to the launch for the split pieces
  int max_parts;       // > 0: most pieces a tile is cut into, as the caller asked; 0: chosen from k
  int num_cus;         // tiles the device runs at a time (one work-group per compute unit)
  int main_grid;       // launch indices below this walk whole tiles (set by the launcher)
  // order in which the blocks of the walk are dealt (see launch_sched_map; null: walk order)
  const int32_t* block_order;
  int n_blocks;
};

// dA[g, k, n] = x[rows of g, k]^T . dy[rows of g, n]
struct TgmmArgs {
  const void* x;
  const void* dy;
  void* dA;
  const int32_t* group_sizes;
  const int32_t* group_offsets;
  int m, k, n, g;  // g: groups of dA (the slices computed)
  int g_first;     // dA[i] belongs to group g_first + i of group_sizes / group_offsets
  int k_tiles, n_tiles;  // ceil(k / BM), ceil(n / BN)
  int group_m;
  const int32_t* group_order;  // null, or the records of the order in which the launch visits the groups (launch_sched_map)
};

// A value every lane holds identically, moved to a scalar register.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

template <class C, class = void>
struct IsW4 { static constexpr bool value = false; };
template <class C>
struct IsW4<C, decltype((void)C::W4)> { static constexpr bool value = true; };
template <class C, class = void>
struct IsW4R { static constexpr bool value = false; };
template <class C>
struct IsW4R<C, decltype((void)C::W4R)> { static constexpr bool value = true; };

// Element type of a configuration's output: its Out when it names one (float8 operands give bf16), else that of its operands.
template <class C, class = void>
struct OutOf { typedef typename C::Elem type; };
template <class C>
struct OutOf<C, decltype((void)sizeof(typename C::Out))> { typedef typename C::Out type; };

constexpr int kW4RMinK = 1792;  // measured: level at 1536, 7 % ahead at 2048, 13 % at 8192 (eight groups of 2048 rows)

template <class C>
__device__ __forceinline__ void run_tile(const typename C::Elem* Ap, int lda, int a_lim, const typename C::Elem* Bp,
                                         int ldb, int b_lim, int klen, typename OutOf<C>::type* Op, int ldo,
                                         typename C::Elem* smem, const SplitK& sk = SplitK()) {
  if constexpr (C::F32) gemm_tile_f32<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem);
  else if constexpr (IsF8Direct<C>::value) {
    if constexpr (C::PINGPONG) gemm_tile_f8_pingpong<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem, sk);
    else gemm_tile_f8<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem, sk);
  }
  else if constexpr (IsW4R<C>::value) {
    // The register-staged form has four 64-wide slabs to fill before it runs and pays for that on a short contraction:
    // below kW4RMinK the 32-wide direct-to-LDS form of the same core takes the tile.
    if (klen >= kW4RMinK) gemm_tile_w4r<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem, sk);
    else gemm_tile_w4<W4Cfg<C::BM, C::BN, true, true, 5, C::HALF>>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem, sk);
  }
  else if constexpr (IsW4<C>::value) gemm_tile_w4<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem, sk);
  else if constexpr (C::MIXED) gemm_tile_pingpong_mixed<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem, sk);
  else if constexpr (C::DLDS && C::PINGPONG) gemm_tile_pingpong<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem, sk);
  else if constexpr (C::DLDS) gemm_tile_dlds<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, smem, sk);
  else gemm_tile<C>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, Op, ldo, reinterpret_cast<bf16_bits*>(smem));
}

// Row tiles of a group with at most kShortRows rows (most tiles of a launch when the groups are much shorter than the
// tile: a mixture of experts with a few dozen tokens per expert).  Such a tile is a stream over its 256 columns of the
// group's weights with next to no matrix-core work, so what counts is how many bytes each compute unit keeps in flight
// and that every load covers whole 128-byte lines: the same 256 threads run a 64-row tile routine instead, whose LDS
// ring holds only 4-8 KB of activations per slab - 8 slabs of 32 deep for weights read across rows (7 x 20 KB requested
// ahead of use against 3.5 x 32 KB in the tall routine), 4 slabs of 64 deep for weights read along rows.  The weights
// of such a group are read by this one row tile only: they are streamed past L2 (nt), which keeps L2 for what the
// tall tiles of long groups share.
// A 128-row routine of the same kind (6 slabs of 32, or 3 of 64) serves the tiles with 65 to 128 rows.
constexpr int kShortRows = 64, kMidRows = 128;
template <class C, int ROWS>
struct ShortTileCfg {
  static constexpr int BK = C::B_KMAJOR ? 64 : 32;
  static constexpr int STAGES = (160 * 1024) / ((ROWS + C::BN) * BK * 2);
  typedef DldsCfg<ROWS, C::BN, BK, 1, 4, true, C::B_KMAJOR, STAGES, false, kCachePolicyStream, C::HALF> type;
};

// How the last round of a gmm launch is cut along K.  The device runs num_cus tiles at a time; when the live tiles do
// not fill the last round, the tiles from position `first_tile` of the walk on (the ones that round would hold) are each
// computed by `parts` work-groups over a `parts`-th of the contraction range instead, so the round takes about
// 1 / parts as long.
struct SplitPlan {
  int first_tile;  // walk positions >= first_tile (and < live) are split; == live when nothing is
  int parts;
  int tiles;       // live - first_tile
};
constexpr int kMaxSplitParts = 8;
constexpr int kMinSplitK = 512;  // contraction elements a piece must keep

// k_cost: the contraction length in units of what a bf16 K loop spends per element (float8 operands: k / 2).
__device__ __forceinline__ SplitPlan split_plan(int live, int k, int k_cost, int slots, int num_cus, int max_parts) {
  SplitPlan sp{live, 1, 0};
  if (slots <= 0 || live <= 0) return sp;
  const int first = (live / num_cus) * num_cus;
  const int tiles = live - first;
  if (tiles <= 0) return sp;
  // The piece that arrives last reads every piece's 256 KB of partial sums at what one compute unit can pull (about
  // 25 GB/s: ~10 us per piece), so the gain of a finer cut, T/parts for a K loop of T us, is soon eaten: parts ~
  // sqrt(T / 10 us), with T ~ k / 32 x 0.77 us, i.e. sqrt(k) / 20 - and below k = 6400 (4 pieces) cutting was measured
  // to gain nothing.  max_parts > 0 is the caller's own choice and is taken as it is.
  int parts = imin(imin(slots / tiles, kMaxSplitParts), k / kMinSplitK);
  if (max_parts > 0) {
    parts = imin(parts, max_parts);
  } else {
    int by_k = 1;
    while ((by_k + 1) * (by_k + 1) * 400 <= k_cost) ++by_k;
    if (by_k < 4) return sp;
    parts = imin(parts, by_k);
  }
  if (parts < 2) return sp;
  sp.first_tile = first; sp.parts = parts; sp.tiles = tiles;
  return sp;
}

// Walk tiles in bands of `group_m` rows: consecutive ids share B columns / A rows so that the ~32 tiles one XCD
// has in flight re-use each other's operands out of its L2.
__device__ __forceinline__ void band_walk(int id, int rows, int cols, int group_m, int& ri, int& cj) {
  const int band_sz = group_m * cols;
  const int band = id / band_sz;
  const int within = id - band * band_sz;
  const int gm = imin(group_m, rows - band * group_m);
  cj = within / gm;
  ri = band * group_m + (within - cj * gm);
}

template <class C, bool TRANS_RHS>
__global__ __launch_bounds__(C::NT, C::WAVES_PER_EU) void gmm_kernel(GmmArgs p) {
  typedef typename C::Elem E;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  E* smem = reinterpret_cast<E*>(smem_raw);
  const E* px = static_cast<const E*>(p.x);
  const E* pA = static_cast<const E*>(p.A);
  typedef typename OutOf<C>::type O;
  O* py = static_cast<O*>(p.y);
  // Tile walk.  The scheduling-map kernel has cut every group's row tiles into bands of at most group_m row tiles
  // (tile2band); the walk visits band after band and, inside a band, column after column (all the band's row tiles of
  // one column tile, then the next column).  Position t of the walk therefore lies in the band of row tile t / n_tiles.
  // The walk is cut into blocks of group_m x group_n consecutive positions - a band's rows times a few columns, about
  // what one XCD runs at a time, so the block's operand slabs are fetched into that XCD's L2 once - and the blocks are
  // dealt to the 8 XCDs (launch index mod 8) round-robin.  No block spans two groups' weights except where a band ends.
  // Everything read through the map is the same for the whole work-group: pin it to scalar registers.
  const int total = imin(uniform(*p.total_tiles), p.U);
  const int live = total * p.n_tiles;
  SplitPlan sp{live, 1, 0};
  if constexpr (C::SPLITK) sp = split_plan(live, p.k, sizeof(E) == 1 ? p.k >> 1 : p.k, p.split_slots, p.num_cus, p.max_parts);

  int t;
  SplitK sk;
  int k0 = 0, klen = p.k;
  if ((int)blockIdx.x < p.main_grid) {
    // With only a few rounds of tiles, blocks of the full size would leave some XCDs without work (180 tiles in blocks
    // of 32 occupy 6 of the 8): the blocks shrink so that every round deals one to each XCD.
    int per_block = p.group_m * p.group_n;
    bool whole_blocks = true;
    if (live < 4 * p.num_cus) {
      const int rounds = (live + p.num_cus - 1) / p.num_cus;
      const int fewer = imax(1, imin(per_block, (live + 8 * rounds - 1) / (8 * rounds)));
      whole_blocks = fewer == per_block;
      per_block = fewer;
    }
    const int pos = blockIdx.x >> 3;
    int block = (pos / per_block) * 8 + (blockIdx.x & 7);
    // Groups much longer than a tile (matrix-core-bound tiles) and groups shorter than one (tiles that stream their
    // group's weights) in one launch: their blocks are dealt interleaved instead of in the order the groups come in, so
    // that at any time some of every XCD's compute units multiply while the others stream (DeepSeek-V3 shape, dlhs:
    // 1.63 -> 1.55 ms; all long groups first, or all short ones, is slower than either).  Same tiles, same results.
    if (p.block_order && whole_blocks) {
      const int n_long = uniform(p.block_order[0]), n_live = uniform(p.block_order[1]);
      bool from_long;
      int rank;
      if (interleaved_slot(block, n_long, n_live, &from_long, &rank))
        block = uniform(p.block_order[from_long ? 2 + rank : 2 + p.n_blocks - 1 - rank]);
    }
    t = block * per_block + pos % per_block;
    if (t >= p.U * p.n_tiles) return;
    if (t >= sp.first_tile && t < live) return;  // computed in pieces by the appended work-groups
  } else {
    // Piece `part` of split tile tt.  The pieces are numbered part-major (all tiles of the first K range, then the
    // second ...) and every XCD (launch index mod 8) takes one contiguous stretch of that numbering, so that the pieces
    // an XCD runs together are neighbouring tiles of one K range and share their operand slabs in its L2.
    const int r = blockIdx.x - p.main_grid;
    const int pieces = sp.tiles * sp.parts;
    const int per_xcd = (pieces + 7) >> 3;
    if ((r >> 3) >= per_xcd) return;
    const int id = (r & 7) * per_xcd + (r >> 3);
    if (id >= pieces) return;
    const int part = id / sp.tiles, tt = id - part * sp.tiles;
    t = sp.first_tile + tt;
    const int k64 = (p.k + 63) >> 6;
    k0 = (int)((long long)k64 * part / sp.parts) << 6;
    klen = imin(p.k, (int)((long long)k64 * (part + 1) / sp.parts) << 6) - k0;
    sk.partials = p.partials + (size_t)tt * sp.parts * (C::BM * C::BN);
    sk.counter = p.counters + tt;
    sk.parts = sp.parts;
    sk.part = part;
  }
  const int band = uniform(p.tile2band[t / p.n_tiles]);
  const bool deferred = (band & kBandDeferred) != 0;  // a short last row tile the map has moved behind all other tiles
  const int band_row0 = (band & ~kBandDeferred) >> kBandShift, band_rows = band & kBandMaxRows;
  const int w = t - band_row0 * p.n_tiles;
  const int nj = w / band_rows;
  const int mi = band_row0 + (w - nj * band_rows);
  const int col0 = nj * C::BN;
  const int cols = imin(C::BN, p.n - col0);

  if (mi < total) {
    const int gi = uniform(p.tile2group[mi]);
    const int it = uniform(p.tile2it[mi]);
    const int row0 = uniform(p.group_offsets[gi]) + it * C::BM;
    int rows = imin(C::BM, uniform(p.group_sizes[gi]) - it * C::BM);
    rows = imin(rows, p.m - row0);  // group_sizes summing past m: never touch rows >= m
    if (rows <= 0 || row0 < 0) return;
    O* Op = py + (size_t)row0 * p.n + col0;
    const int gl = gi - p.g_first;  // index of the group's weights in A
    if (gl < 0 || gl >= p.g_local) {
      // a group whose weights live elsewhere (A is a slice of the groups): its rows of y are zero
      if (sk.part == 0) zero_tile<C::NT, C::VEC, O>(Op, p.n, rows, cols);
      return;
    }
    const E* Ap = px + (size_t)row0 * p.k + k0;
    const E* Bp = TRANS_RHS ? pA + (size_t)gl * p.n * p.k + (size_t)col0 * p.k + k0
                            : pA + (size_t)gl * p.k * p.n + (size_t)k0 * p.n + col0;
    if constexpr (IsW4<C>::value && C::A_KMAJOR) {
      // For a group's single row tile, and for the short last tile of a longer group where the scheduling map has moved
      // it behind all other tiles (into the K-split last round).  Left in its group's run such a tile must stay on the tall routine: run
      // through the short one it finishes early, the tiles dealt next start out of step with the rest of their block,
      // and the block's operand slabs are fetched into L2 twice (measured: +1 GB of fetches per launch, no time gained).
      if (rows <= kMidRows && (it == 0 || deferred)) {
        typedef typename ShortTileCfg<C, kShortRows>::type S;
        typedef typename ShortTileCfg<C, kMidRows>::type M;
        static_assert(S::LDS_BYTES <= C::LDS_BYTES && S::NT == C::NT && S::BN == C::BN, "the short routine runs in the tall one's launch");
        static_assert(M::LDS_BYTES <= C::LDS_BYTES && M::NT == C::NT && M::BN == C::BN, "the 128-row routine runs in the tall one's launch");
        const int ldb = TRANS_RHS ? p.k : p.n;
        if (rows <= kShortRows) gemm_tile_dlds<S>(Ap, p.k, rows, Bp, ldb, cols, klen, Op, p.n, smem, sk);
        else gemm_tile_dlds<M>(Ap, p.k, rows, Bp, ldb, cols, klen, Op, p.n, smem, sk);
        return;
      }
    }
    if constexpr (IsF8Direct<C>::value) {
      if constexpr (C::NW == 8 && C::WAVES_M == 2 && C::A_KMAJOR && C::BM > kShortRows) {
        // a group's single row tile of at most kShortRows rows, as above: a 64-row routine on 128-deep slabs (every load
        // covers whole 128-byte lines), the weights streamed past L2 - where the tall routine's LDS has room for its ring
        typedef F8Cfg<kShortRows, C::BN, 2, 4, 3, 128, kCachePolicyStream, true, C::B_KMAJOR, false> S;
        if constexpr (S::LDS_BYTES <= C::LDS_BYTES) {
          static_assert(S::NT == C::NT, "the short routine runs in the tall one's launch");
          if (rows <= kShortRows && it == 0) {
            gemm_tile_f8<S>(Ap, p.k, rows, Bp, TRANS_RHS ? p.k : p.n, cols, klen, Op, p.n, smem, sk);
            return;
          }
        }
      }
    }
    run_tile<C>(Ap, p.k, rows, Bp, TRANS_RHS ? p.k : p.n, cols, klen, Op, p.n, smem, sk);
  } else {
    // Rows past sum(group_sizes) are defined to be zero.  The map never uses more than
    // U - ceil(tail / BM) entries, so the unused tile slots cover the tail.
    long long s = (long long)uniform(p.group_offsets[p.g - 1]) + uniform(p.group_sizes[p.g - 1]);
    if (s < 0) s = 0;
    const long long r0 = s + (long long)(mi - total) * C::BM;
    if (r0 >= p.m) return;
    const int rows = imin(C::BM, p.m - (int)r0);
    zero_tile<C::NT, C::VEC, O>(py + (size_t)r0 * p.n + col0, p.n, rows, cols);
  }
}

template <class C>
__global__ __launch_bounds__(C::NT, C::WAVES_PER_EU) void tgmm_kernel(TgmmArgs p) {
  typedef typename C::Elem E;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  E* smem = reinterpret_cast<E*>(smem_raw);
  // Work per tile is proportional to its group's row count, which only the device knows and which can be wildly
  // skewed.  So every XCD (launch index mod 8) takes one eighth of every group's tiles - a contiguous stretch of the
  // group's banded walk, so its tiles still share operand columns in its L2 - and all XCDs get the same share of every
  // group however the rows are distributed.
  const int per_group = p.k_tiles * p.n_tiles;
  const int quota = (per_group + 7) >> 3;  // tiles of one group per XCD
  const int xcd = blockIdx.x & 7, pos = blockIdx.x >> 3;
  const int slot = pos / quota;
  if (slot >= p.g) return;
  // groups are visited by falling size class, so that tiles of about equal duration run side by side; the record of
  // a position holds the group, its first row and its row count
  int gi = slot, row0, rows;
  if (p.group_order) {
    const int32_t* rec = p.group_order + 4 * (size_t)slot;
    gi = uniform(rec[0]); row0 = uniform(rec[1]); rows = uniform(rec[2]);
  } else {
    row0 = uniform(p.group_offsets[slot + p.g_first]);
    rows = uniform(p.group_sizes[slot + p.g_first]);
  }
  const int t = ((xcd + slot) & 7) * quota + (pos - slot * quota);
  if (gi < 0 || gi >= p.g || t >= per_group) return;
  int ri, cj;
  band_walk(t, p.k_tiles, p.n_tiles, p.group_m, ri, cj);

  const int kk0 = ri * C::BM, col0 = cj * C::BN;
  const int krows = imin(C::BM, p.k - kk0), cols = imin(C::BN, p.n - col0);
  typedef typename OutOf<C>::type O;
  O* Op = static_cast<O*>(p.dA) + (size_t)gi * p.k * p.n + (size_t)kk0 * p.n + col0;

  rows = imin(rows, p.m - row0);
  if (rows <= 0 || row0 < 0) {  // empty group: its slice of dA is zero
    zero_tile<C::NT, C::VEC, O>(Op, p.n, krows, cols);
    return;
  }
  const E* Ap = static_cast<const E*>(p.x) + (size_t)row0 * p.k + kk0;
  const E* Bp = static_cast<const E*>(p.dy) + (size_t)row0 * p.n + col0;
  run_tile<C>(Ap, p.k, krows, Bp, p.n, cols, rows, Op, p.n, smem);
}

// ---- host-side launchers, one set per compiled tile shape -------------------------------------------------------

typedef int (*gmm_launch_fn)(hipStream_t, const GmmArgs&);
typedef int (*tgmm_launch_fn)(hipStream_t, const TgmmArgs&);

struct TileVariant {
  const char* name;
  int bm, bn, bk, waves_m, waves_n;
  int vec;  // 1: needs k % 8 == 0 and n % 8 == 0 (16-byte row pitches); 0: any shape
  int dtype;   // RD_DTYPE_* of the operands and the output this shape is compiled for
  int dlds;    // 1: direct-to-LDS core (byte extents of one tile's operand window must stay below 2 GiB)
  int stages;  // LDS ring depth
  int splitk;  // 1: the gmm kernels can cut the last round of tiles along K (needs partials in the workspace)
  gmm_launch_fn gmm_nn, gmm_nt;  // null: the shape has no kernel for that product
  tgmm_launch_fn tgmm;
};

// Kernels that use more than 64 KB of LDS must opt in, once per device.
static inline int allow_big_lds(const void* kern, int bytes) {
  if (bytes <= 64 * 1024) return hipSuccess;
  return (int)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

template <class C, bool TRANS_RHS>
int launch_gmm(hipStream_t s, const GmmArgs& a) {
  auto kern = gmm_kernel<C, TRANS_RHS>;
  const int attr_rc = allow_big_lds(reinterpret_cast<const void*>(kern), C::LDS_BYTES);
  if (attr_rc != hipSuccess) return attr_rc;
  // positions per XCD: enough for any block size the kernel may shrink to (at most group_m x group_n)
  const int per_block = a.group_m * a.group_n;
  GmmArgs args = a;
  args.main_grid = 8 * ((a.U * a.n_tiles + 7) / 8 + 2 * per_block);
  if (!C::SPLITK) args.split_slots = 0;
  const int grid = args.main_grid + args.split_slots;
  if (args.main_grid <= 0) return hipSuccess;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::NT), C::LDS_BYTES, s, args);
  return (int)hipGetLastError();
}

template <class C>
int launch_tgmm(hipStream_t s, const TgmmArgs& a) {
  auto kern = tgmm_kernel<C>;
  const int attr_rc = allow_big_lds(reinterpret_cast<const void*>(kern), C::LDS_BYTES);
  if (attr_rc != hipSuccess) return attr_rc;
  const int grid = 8 * a.g * ((a.k_tiles * a.n_tiles + 7) / 8);
  if (grid <= 0) return hipSuccess;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::NT), C::LDS_BYTES, s, a);
  return (int)hipGetLastError();
}

}  // namespace rd
