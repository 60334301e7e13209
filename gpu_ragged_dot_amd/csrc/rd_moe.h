// Host-side launchers of the token-routing kernels (rd_moe.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace rd {

constexpr int kMoeMaxTopK = 64;       // slots per token the combine kernels stage in LDS
constexpr int kMoeMaxGroups = 12288;  // one int32 of LDS per expert in the single-wave ranking kernel

// int32 scratch of the route kernels: one histogram row per 2048 slots plus one row of group starts.
size_t moe_route_workspace_bytes(long long slots, int g);
int launch_moe_route(hipStream_t s, const int32_t* ids, int slots, int g, int32_t* group_sizes, int32_t* row_of_slot,
                     int32_t* slot_of_row, int32_t* workspace);
// elem: 0 bfloat16, 1 float32, 2 float16 rows
int launch_moe_dispatch(hipStream_t s, const void* h, const int32_t* row_of_slot, const int32_t* slot_of_row,
                        const float* row_scale, void* x, int tokens, int top_k, int d, int elem);
int launch_moe_combine(hipStream_t s, const void* y, const int32_t* row_of_slot, const float* weights, void* out,
                       int tokens, int top_k, int d, int elem);
int launch_moe_combine_wgrad(hipStream_t s, const void* y, const void* dout, const int32_t* row_of_slot, float* dw,
                             int tokens, int top_k, int d, int elem);

}  // namespace rd
