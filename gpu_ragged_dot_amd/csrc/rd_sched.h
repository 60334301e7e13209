// Host-side launchers of the scheduling-map and fill kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace rd {

// tile2band entries: (first row tile of the band << kBandShift) | rows of the band.
constexpr int kBandShift = 7;
constexpr int kBandMaxRows = (1 << kBandShift) - 1;

// Arrays as in the reference's GMMGroupLookupMetadata (gpu_ragged_dot.py:60-90); tile2group / tile2it hold
// ceil(m / chunk) + g entries.  `counters` (may be null) are n_counters int32 cleared by the same launch.
// `tile2band` (may be null; same length) receives, for every row tile, the band of at most band_rows consecutive row
// tiles of its group that the gmm tile walk puts it in.
// `block_order` (may be null; 2 + n_blocks entries): the order in which the gmm tile walk deals its blocks of
// per_block consecutive positions (n_tiles column tiles per row tile) when groups of more than long_rows rows - whose
// tiles are bound by the matrix cores - and shorter ones - whose tiles stream their group's weights - share a launch:
//   [0] blocks of long groups L, [1] live blocks L + S, [2 ..] the long groups' blocks in walk order from the front,
//   the others' from the back (last entry first).  Block i of the new order is the next long one when
//   floor((i + 1) L / (L + S)) > floor(i L / (L + S)), else the next short one: the two kinds evenly interleaved.
int launch_sched_map(hipStream_t s, const int32_t* group_sizes, int g, int m, int chunk, int32_t* group_offsets,
                     int32_t* tile2group, int32_t* tile2it, int32_t* total_tiles, int32_t* counters = nullptr,
                     int n_counters = 0, int32_t* tile2band = nullptr, int band_rows = 1, int32_t* block_order = nullptr,
                     int n_blocks = 0, int per_block = 1, int n_tiles = 1, int long_rows = 0);

// Measurement aid: a bare read of `bytes` (16-byte aligned) cut into contiguous blocks of block_bytes, one work-group each.
int launch_stream_read(hipStream_t s, const void* src, size_t bytes, size_t block_bytes, void* sink);

// Stream-ordered clear that is safe to record into a HIP graph.
int launch_zero_bytes(hipStream_t s, void* p, size_t bytes);

}  // namespace rd
