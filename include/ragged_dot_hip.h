/* C ABI of the MI355X (gfx950) ragged_dot kernels.
 *
 * This is the boundary the reference crosses at its two pl.pallas_call sites
 * (gpu_ragged_dot.py:217-226 for gmm, :331-340 for tgmm): device buffers in, device buffers out, everything
 * enqueued on the caller's stream, no host synchronisation.  Plain C types only.
 *
 * Conventions
 *  - every pointer is a device pointer unless it says "host"; the caller owns all buffers, including the
 *    workspace; the library never allocates or frees device memory and never synchronises;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *  - matrices are dense row-major; element type is selected by `dtype` (RD_DTYPE_*), output type = input type
 *    (gpu_ragged_dot.py:210,324; the float8 type, which the reference does not have, gives bfloat16), accumulation is
 *    always fp32 (acc_dtype, gpu_ragged_dot.py:119,251);
 *  - return value 0 = success; negative = RD_ERR_*; the text of the last error of the calling thread is
 *    available from rd_last_error().  Nothing here aborts the process;
 *  - no host reads of device data: the launch grid is the static bound ceil(m / tile_m) + g of
 *    gpu_ragged_dot.py:212, so every entry point can be recorded into a HIP graph.
 */
#ifndef RAGGED_DOT_HIP_H_
#define RAGGED_DOT_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 3: RD_DTYPE_F16; rd_plan.group_n = 1 / -1 for rd_tgmm; the workspaces hold the orders the scheduling-map kernel builds
 * (all source compatible with 2: same structs, same signatures) */
#define RD_ABI_VERSION 3

/* Element type of the operands and the output (the same, gpu_ragged_dot.py:210,324, but for float8) and what the matrix
 * cores multiply.  RD_DTYPE_F32_BF16 is compute_dtype = bfloat16 on float32 arrays (gpu_ragged_dot.py:116-119, 145, 149): the
 * float32 elements are rounded to bfloat16 (nearest even) as they are loaded, multiplied on the bf16 matrix cores with
 * fp32 accumulation, and stored as float32.  (compute_dtype = float32 on bfloat16 arrays is RD_DTYPE_BF16 itself: a
 * product of two bfloat16 values is exact in fp32, and the accumulation is fp32 either way.)
 * RD_DTYPE_F8E4M3_BF16: both operands (x and A of rd_gmm, x and dy of rd_tgmm) are float8 e4m3fn bytes (the OCP format:
 * bias 7, no infinities, 0x7f / 0xff are NaN), the output is bfloat16 - jax.lax.ragged_dot on float8 operands with
 * preferred_element_type = bfloat16; the reference itself has no float8 path.  With 16-byte row pitches (k % 16 == 0,
 * and n % 16 == 0 unless trans_rhs) the bytes go to the float8 matrix-core instruction as they are (fp32
 * accumulation); otherwise they are widened to bfloat16 as
 * they are loaded (exact: every e4m3 value is a bfloat16 value) and multiplied on the bf16 matrix cores.  Either way the
 * result is that of an exact-product fp32-accumulating float8 multiply; the first path has half the bytes to read and
 * twice the matrix-core rate of bfloat16, the second only the former.  Of the streaming kernels for a few rows per group
 * float8 has the one for weights stored [g, n, k] (trans_rhs, decode_nb = RD_DECODE_ROWS, k % 16 == 0; rd_default_plan
 * picks it up to one row per group on average); the K-split of rd_plan.split_k on the first path only.
 * RD_DTYPE_F16: float16 (IEEE half) arrays - the reference takes whatever element type its arrays have - multiplied on
 * the float16 matrix-core instruction with fp32 accumulation, float16 out (nearest even).  Everything bfloat16 has
 * except the smaller direct-to-LDS tile shapes: the four-wave 256 x 256 core with the K-split, register-staged tiles for
 * any shape, the streaming kernels for a few rows per group, the routing kernels. */
enum rd_dtype { RD_DTYPE_BF16 = 0, RD_DTYPE_F32 = 1, RD_DTYPE_F32_BF16 = 2, RD_DTYPE_F8E4M3_BF16 = 3, RD_DTYPE_F16 = 4 };

#define RD_DECODE_ROWS (-1) /* rd_plan.decode_nb: the streaming kernel that cuts each expert's weights into whole-row slices */

enum rd_status {
  RD_OK = 0,
  RD_ERR_INVALID_ARGUMENT = -1, /* bad shape / null pointer / unknown enum */
  RD_ERR_UNSUPPORTED = -2,      /* valid request that this build has no kernel for */
  RD_ERR_WORKSPACE = -3,        /* workspace too small or misaligned */
  RD_ERR_HIP = -4               /* a HIP runtime call failed; see rd_last_error() */
};

/* One compiled tile shape.  `id` indexes the table rd_num_variants()/rd_get_variant() expose. */
typedef struct rd_variant_info {
  int id;
  int tile_m, tile_n, tile_k; /* macro-tile: rows x columns x contraction slab */
  int waves_m, waves_n;       /* wavefront grid inside a work-group (64 lanes each) */
  int vec;                    /* 1: needs 16-byte row pitches (k % 8 == 0 and n % 8 == 0 for bf16) */
  int dtype;                  /* RD_DTYPE_* of operands and output this variant is compiled for */
  int direct_to_lds;          /* 1: HBM -> LDS loads bypass registers; max(m,k)*max(k,n) must stay below 2^30 */
  int stages;                 /* depth of the K-slab ring in LDS */
  char name[48];
} rd_variant_info;

/* Launch plan for one call; the host planner (or the caller) fills it.  variant = -1 with every other field 0 = library defaults. */
typedef struct rd_plan {
  int variant; /* index into the variant table, or -1: let the library choose by shape */
  int group_m; /* tile walk.  rd_gmm: a group's row tiles are cut into bands of at most group_m (1..127) row tiles and the
                  walk goes band by band, column by column inside a band.  rd_tgmm: row tiles per band.  0 = default */
  int group_n; /* rd_gmm: the walk is dealt to the 8 XCDs in blocks of group_m x group_n (<= 4096) consecutive tiles;
                  the product should equal what one XCD runs at a time (32 for the 256 x 256 tiles).  0 = default.
                  rd_tgmm: 1 = visit the groups by falling row count class (tiles of about equal duration then run side
                  by side, and the longest groups' tiles do not end the launch alone), -1 = as they come, 0 = by size
                  class when the groups average 512 rows or more and the launch has more than a round of tiles */
  int decode_nb; /* rd_gmm only, for a few rows per group: > 0 selects the streaming kernel that gives each work-group
                    this many columns (32, 64 or 128) of one expert; RD_DECODE_ROWS the one that gives it whole rows
                    for a slice of the contraction range (fp32 partial sums in the workspace, n <= 2048) or, with
                    trans_rhs, whole weight rows of a slice of the columns (no partial sums, k <= 8192) */
  int split_k; /* rd_gmm only: 0 = when the tiles do not fill the device's last round and k >= 6400 (float8: 12800), cut
                  those tiles' contraction range over up to sqrt(k)/20 work-groups (fp32 partial sums in the workspace); n > 0 =
                  cut them over up to n (at most 8) whatever k is; -1 = never */
} rd_plan;

int rd_abi_version(void);
const char* rd_last_error(void); /* host pointer, valid until the thread's next failing call */

int rd_num_variants(void);
int rd_get_variant(int id, rd_variant_info* out /* host */);

/* The library's own shape-based choice (what variant = -1 resolves to); op: 0 gmm, 1 gmm trans_rhs, 2 tgmm.
 * For op 0 with m <= 4 g (and m <= 1024, n <= 2048, min(g, m) * ceil(n / 256) <= 512) it selects the streaming kernel, which holds 4 rows of a group at a
 * time (8 when m > g) and streams the group's weights once per pass.  The shape cannot tell how the rows are spread: a
 * group with more rows than a pass holds is served by several work-groups at once, one pass each, so that rows piling
 * up in ONE group cost no more than a tile kernel would (128 groups of 2048 x 768, all 256 rows in one group: 33 us,
 * weights stored [g, n, k] 19 us; best tile kernel 35 us; rows spread evenly: 69 us).  Op 1 (weights stored [g, n, k])
 * has a streaming kernel of its own under the same conditions and k <= 8192; it needs no workspace beyond the map's. */
int rd_default_plan(int op, int m, int k, int n, int g, int dtype, rd_plan* out /* host */);

/* ---- scheduling map --------------------------------------------------------------------------------------
 * Replaces _make_gmm_group_metadata (gpu_ragged_dot.py:70-90).  Bit-exact int32 outputs:
 *   group_offsets[g]                = exclusive prefix sum of group_sizes                         (:86)
 *   row_it2group[U], row_it2it_in_group[U],  U = ceil(m / chunk_m) + g                            (:77-82)
 *   total_row_its[1]                = sum(ceil(group_sizes / chunk_m))                            (:89)
 * Requires g >= 1, m >= 0, chunk_m >= 1. */
int rd_sched_map(void* stream, const int32_t* group_sizes, int g, int m, int chunk_m, int32_t* group_offsets,
                 int32_t* row_it2group, int32_t* row_it2it_in_group, int32_t* total_row_its);

/* Number of entries U of the two per-tile arrays (gpu_ragged_dot.py:77, :212). */
int rd_sched_map_len(int m, int g, int chunk_m);

/* ---- gmm: y[m, n] = ragged x[m, k] . A ----------------------------------------------------------------------
 * Replaces the "gpu_gmm" pallas_call (gpu_ragged_dot.py:93-165, 217-226).
 *   A is [g, k, n] (trans_rhs = 0) or [g, n, k] (trans_rhs = 1, gpu_ragged_dot.py:139-144, :190).
 *   Rows of group i are [offset_i, offset_i + group_sizes[i]); rows >= sum(group_sizes) of y are set to zero
 *   (:155-165) -- also when every group is empty.  Groups that would run past m are clipped to m.
 * Workspace: rd_gmm_workspace_bytes() bytes, 256-byte aligned; holds the scheduling map, 64 KiB for the order in which
 * the tile walk's blocks are dealt (long groups' among short groups') and, unless the plan says split_k = -1, fp32
 * partial sums (64 MiB for the 256 x 256 tiles).  A smaller workspace that has room for the map is accepted: the call
 * then runs without the K-split and, if the order does not fit either, in plain walk order - same results. */
size_t rd_gmm_workspace_bytes(int m, int g, const rd_plan* plan /* host, may be NULL */);
int rd_gmm(void* stream, const void* x, const void* A, const int32_t* group_sizes, void* y, int m, int k, int n,
           int g, int trans_rhs, int dtype, const rd_plan* plan /* host, may be NULL */, void* workspace,
           size_t workspace_bytes);

/* ---- a slice of the groups (expert-parallel sharding) ----------------------------------------------------------
 * The `group_offset` of jax.lax.ragged_dot (named by its documentation; the reference gpu_ragged_dot.py has no such
 * parameter).  group_sizes still describes all g_total groups and x / y all m rows, but A (dA) holds only the
 * g_local groups [group_offset, group_offset + g_local): a rank that owns a slice of the experts calls with its
 * slice and the global group_sizes.
 *   rd_gmm_sharded : rows of the groups in the slice as rd_gmm; rows of every other group and past sum(group_sizes) zero.
 *   rd_tgmm_sharded: dA[i] = slice of group group_offset + i, i < g_local.
 * Workspace: rd_gmm_workspace_bytes / rd_tgmm_workspace_bytes with g = g_total.  The streaming kernels
 * (plan.decode_nb != 0) serve all groups only.  group_offset = 0 and g_local = g_total is rd_gmm / rd_tgmm. */
int rd_gmm_sharded(void* stream, const void* x, const void* A, const int32_t* group_sizes, void* y, int m, int k, int n,
                   int g_total, int group_offset, int g_local, int trans_rhs, int dtype,
                   const rd_plan* plan /* host, may be NULL */, void* workspace, size_t workspace_bytes);
int rd_tgmm_sharded(void* stream, const void* x, const void* dy, const int32_t* group_sizes, void* dA, int m, int k, int n,
                    int g_total, int group_offset, int g_local, int dtype, const rd_plan* plan /* host, may be NULL */,
                    void* workspace, size_t workspace_bytes);

/* ---- rd_gmm without a workspace -------------------------------------------------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  Same product as rd_gmm, same kernels; what rd_gmm keeps in the
 * caller's workspace (the scheduling map, the streaming kernel's partial sums) lives in a buffer of
 * rd_gmm_noalloc_scratch_bytes() = 4 MiB built into the library, one copy per device, held until the process ends.
 * The call allocates and frees nothing.  Limits: the scheduling map must fit (rd_gmm_workspace_bytes(m, g, plan with
 * split_k = -1) <= 4 MiB, i.e. roughly 12 (m / 16) + 16 g bytes <= 4 MiB - 64 KiB: 5.5 M rows with a few hundred groups),
 * otherwise RD_ERR_WORKSPACE; the K-split is never used.
 * All calls on one device share that device's buffer: calls that overlap on one device (different streams, or
 * different threads without stream ordering between them) race; calls ordered on one stream do not. */
size_t rd_gmm_noalloc_scratch_bytes(void);
int rd_gmm_noalloc(void* stream, const void* x, const void* A, const int32_t* group_sizes, void* y, int m, int k, int n,
                   int g, int trans_rhs, int dtype, const rd_plan* plan /* host, may be NULL */);

/* ---- tgmm: dA[g, k, n] = x[rows of g, :]^T . dy[rows of g, :] -----------------------------------------------
 * Replaces the "gpu_tgmm" pallas_call (gpu_ragged_dot.py:231-281, 331-340).  Slices of empty groups are zero
 * (:277-281).  x is [m, k], dy is [m, n].
 * Workspace: rd_tgmm_workspace_bytes() bytes, 256-byte aligned: the groups' row offsets and 16 bytes per group for the
 * order in which the launch visits the groups when they go by size class (group_n of the plan).  A workspace with room for the
 * offsets only is accepted: the groups are then visited as they come - same results. */
size_t rd_tgmm_workspace_bytes(int m, int g, const rd_plan* plan /* host, may be NULL */);
int rd_tgmm(void* stream, const void* x, const void* dy, const int32_t* group_sizes, void* dA, int m, int k,
            int n, int g, int dtype, const rd_plan* plan /* host, may be NULL */, void* workspace,
            size_t workspace_bytes);

/* ---- measurement aid ----------------------------------------------------------------------------------------------
 * No counterpart in the reference and not part of the surface that replaces it: nothing a caller of ragged_dot needs,
 * only what the benchmark uses to time a bare read on the same device in the same process.  A load-only kernel: reads `bytes` (src 16-byte aligned) cut into contiguous blocks
 * of block_bytes, one work-group per block, and stores nothing (`sink`, 4 bytes of device memory or NULL, is written
 * only if the folded data equals one fixed word).  It is what a bare stream over the same bytes takes on this device -
 * the floor the benchmark prints next to the memory-bound kernels. */
int rd_probe_stream_read(void* stream, const void* src, size_t bytes, size_t block_bytes, void* sink);

/* ---- token routing around ragged_dot --------------------------------------------------------------------------
 * The reference takes rows that are already sorted by group and leaves the sorting to its caller (its tests and
 * tuner build sorted rows directly: tests.py:51-71, tuning.py:41-47).  These entry points are that caller's side for a
 * mixture of experts, on the device, so that group_sizes is produced where rd_gmm consumes it.
 *   A "slot" is one (token, choice) pair, numbered token * top_k + choice; a "row" is a row of the sorted matrix.
 *   expert_ids[tokens * top_k]: expert of every slot; ids outside [0, g) mark dropped slots.
 *   rd_moe_route: stable counting sort of the kept slots by expert id (ties keep slot order):
 *     group_sizes[g]; row_of_slot[slots] (-1 for dropped slots); slot_of_row[slots] (-1 for rows past
 *     sum(group_sizes)).  Bit-exact integer outputs.  1 <= g <= 12288, 1 <= top_k <= 64.
 *   rd_moe_dispatch: x[row, :] = h[slot_of_row[row] / top_k, :] (times row_scale[slot] when row_scale is not NULL,
 *     product rounded once to the element type); rows with slot -1 are zero.  h is [tokens, d], x is [slots, d].
 *     Takes both index arrays of rd_moe_route: each token's row is read once and written to its top_k rows.
 *     With row_scale it is also the adjoint of rd_moe_combine with respect to y.
 *   rd_moe_combine: out[token, :] = sum over its kept slots, in slot order, of weights[slot] * y[row_of_slot[slot], :]
 *     (weights NULL = 1), fp32 accumulation, rounded once.  y is [slots, d], out is [tokens, d].  With weights NULL it
 *     is the adjoint of rd_moe_dispatch.
 *   rd_moe_combine_wgrad: dw[slot] = <y[row_of_slot[slot], :], dout[token, :]> in fp32 (0 for dropped slots).
 * weights, row_scale and dw are float32 [tokens * top_k]; the rows (h, x, y, out, dout) are RD_DTYPE_BF16, RD_DTYPE_F32
 * or RD_DTYPE_F16. */
size_t rd_moe_route_workspace_bytes(int tokens, int top_k, int g);
int rd_moe_route(void* stream, const int32_t* expert_ids, int tokens, int top_k, int g, int32_t* group_sizes,
                 int32_t* row_of_slot, int32_t* slot_of_row, void* workspace, size_t workspace_bytes);
int rd_moe_dispatch(void* stream, const void* h, const int32_t* row_of_slot, const int32_t* slot_of_row,
                    const float* row_scale, void* x, int tokens, int top_k, int d, int dtype);
int rd_moe_combine(void* stream, const void* y, const int32_t* row_of_slot, const float* weights, void* out,
                   int tokens, int top_k, int d, int dtype);
int rd_moe_combine_wgrad(void* stream, const void* y, const void* dout, const int32_t* row_of_slot, float* dw,
                         int tokens, int top_k, int d, int dtype);

#ifdef __cplusplus
}
#endif
#endif /* RAGGED_DOT_HIP_H_ */
