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
int launch_sched_map(hipStream_t s, const int32_t* group_sizes, int g, int m, int chunk, int32_t* group_offsets,
                     int32_t* tile2group, int32_t* tile2it, int32_t* total_tiles, int32_t* counters = nullptr,
                     int n_counters = 0, int32_t* tile2band = nullptr, int band_rows = 1);

// Measurement aid: a bare read of `bytes` (16-byte aligned) cut into contiguous blocks of block_bytes, one work-group each.
int launch_stream_read(hipStream_t s, const void* src, size_t bytes, size_t block_bytes, void* sink);

// Stream-ordered clear that is safe to record into a HIP graph.
int launch_zero_bytes(hipStream_t s, void* p, size_t bytes);

}  // namespace rd
