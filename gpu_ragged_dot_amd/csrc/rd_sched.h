// Host-side launchers of the scheduling-map and fill kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace rd {

// tile2band entries: (first row tile of the band << kBandShift) | rows of the band.
constexpr int kBandShift = 7;
constexpr int kBandMaxRows = (1 << kBandShift) - 1;
constexpr int kBandDeferred = 1 << 30;  // mark of a short last row tile listed behind all other tiles (see launch_sched_map)

// Arrays as in the reference's GMMGroupLookupMetadata (gpu_ragged_dot.py:60-90); tile2group / tile2it hold
// ceil(m / chunk) + g entries.  `counters` (may be null) are n_counters int32 cleared by the same launch.
// `tile2band` (may be null; same length) receives, for every row tile, the band of at most band_rows consecutive row
// tiles of its group that the gmm tile walk puts it in.
// `block_order` (may be null; 2 + n_blocks entries): the two lists from which the gmm tile walk deals its blocks of
// per_block consecutive positions (n_tiles column tiles per row tile) when groups of more than long_rows rows - whose
// tiles are bound by the matrix cores - and shorter ones - whose tiles stream their group's weights - share a launch:
//   [0] blocks of long groups L, [1] live blocks L + S, [2 ..] the long groups' blocks in walk order from the front,
//   the others' from the back (last entry first).  interleaved_slot() says which list a position of the launch takes from.
// `group_order` (may be null; order_count records of 4 words): for tgmm, the groups [order_first, order_first +
// order_count) of group_sizes, numbered from 0, listed by falling size class (bit length of the row count: 0, 1, 2-3,
// 4-7, ...) and by index within a class; a record holds the group's number, first row and row count (one load per tile:
// looking the group up first and its rows after costs a short group's tile a second round trip, 2 % of the launch).  A tgmm launch that visits the groups in this order runs tiles of about equal duration side
// by side (DeepSeek-V3 shape, 256 groups of 0 to 7099 rows: 1.97 -> 1.92 ms; with the groups also stored in that order
// 1.90; an exact sort by rows gives the same, classes of 64 or 128 rows half of it or nothing, long groups merely moved
// to the front nothing).  Where two groups' tiles share an XCD the order the groups come in mixes long and short
// tiles and is the better one (128 groups with Zipf lengths, k 2048, n 4096: 0.84 -> 0.88 ms), so the caller of this function decides.
// `defer_rows` > 0 (internal maps of gmm launches only, needs tile2band): the last row tile of a group of two or more
// row tiles, when it holds at most defer_rows rows, is listed behind all other tiles instead of behind its group's - as a
// band of its own, marked kBandDeferred - provided all such tiles then lie in the launch's partly filled last round
// (defer_cus tiles run at a time) and that round holds at most defer_slots / 2 tiles, i.e. is cut along K.
int launch_sched_map(hipStream_t s, const int32_t* group_sizes, int g, int m, int chunk, int32_t* group_offsets,
                     int32_t* tile2group, int32_t* tile2it, int32_t* total_tiles, int32_t* counters = nullptr,
                     int n_counters = 0, int32_t* tile2band = nullptr, int band_rows = 1, int32_t* block_order = nullptr,
                     int n_blocks = 0, int per_block = 1, int n_tiles = 1, int long_rows = 0,
                     int32_t* group_order = nullptr, int order_first = 0, int order_count = 0, int defer_rows = 0,
                     int defer_cus = 0, int defer_slots = 0);

// Which block the i-th block position of a gmm launch takes from the two lists of block_order.  Positions are dealt to
// the 8 XCDs round-robin (position i runs on XCD i mod 8), so the launch is a sequence of rounds of 8.  The long groups'
// blocks are spread so that every round holds floor or ceil of 8 L / (L + S) of them AND every XCD receives floor or
// ceil of L / 8 over the launch: XCD x takes a long block in round r when r L / R + rev(x) / 8 passes an integer (R
// complete rounds, rev = the 3-bit reversal, so the 8 phases are evenly spaced and the per-round sum comes out exact).
// Spreading along the sequence alone is not enough: with L / (L + S) = 3 / 8 every long block lands on the same three
// XCDs (two long groups + 60 short ones, k = n = 4096: 550 us in group order, 585 us so, 535 us with this rule).
// The blocks of an incomplete last round are short ones.  Returns false (walk order stays) when there is nothing to
// mix or too few short blocks for that last round; else *from_long and the rank within that list.
__host__ __device__ inline bool interleaved_slot(int i, int n_long, int n_live, bool* from_long, int* rank) {
  const int rounds = n_live >> 3, mixed = rounds << 3;
  if (n_long <= 0 || n_long >= n_live || n_long > mixed || i >= n_live) return false;
  if (i >= mixed) { *from_long = false; *rank = i - n_long; return true; }
  const int r = i >> 3, x = i & 7;
  const unsigned rl = (unsigned)r * (unsigned)n_long, span = 8u * (unsigned)rounds;
  int longs = (int)(rl / (unsigned)rounds);  // long blocks of the earlier rounds
  const unsigned at = rl % span;
  bool mine = false;
  for (int xx = 0; xx < 8; ++xx) {
    const unsigned phase = (unsigned)(((xx & 1) << 2) | (xx & 2) | ((xx >> 2) & 1)) * (unsigned)rounds;
    const unsigned rem = at + phase >= span ? at + phase - span : at + phase;
    const bool l = rem + (unsigned)n_long >= span;
    if (xx < x) longs += l;
    if (xx == x) mine = l;
  }
  *from_long = mine;
  *rank = mine ? longs : i - longs;
  return true;
}
// r * L must fit 32 bits: block lists of at most this many entries are interleaved
constexpr int kMaxOrderedBlocks = 1 << 15;

// Measurement aid: a bare read of `bytes` (16-byte aligned) cut into contiguous blocks of block_bytes, one work-group each.
int launch_stream_read(hipStream_t s, const void* src, size_t bytes, size_t block_bytes, void* sink);

// Stream-ordered clear that is safe to record into a HIP graph.
int launch_zero_bytes(hipStream_t s, void* p, size_t bytes);

}  // namespace rd
