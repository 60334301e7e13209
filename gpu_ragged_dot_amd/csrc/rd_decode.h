// Launcher of the skinny-m ("decode") forward kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rd {

struct DecodeArgs {
  const uint16_t* x;   // [m, k] bf16 (or float16, see half)
  const uint16_t* A;   // [g, k, n]
  uint16_t* y;         // [m, n]
  const int32_t* group_sizes;
  int m, k, n, g;
  int half;  // 0: the 16-bit elements are bf16; 1: float16 (same layouts, another conversion and dot instruction)
};

// nb: columns per work-group (32, 64 or 128).  Needs k % 8 == 0, n % 8 == 0 and k <= kDecodeMaxK.
constexpr int kDecodeMaxK = 16384;
int launch_gmm_decode(hipStream_t s, const DecodeArgs& a, int nb);

// Whole-row slices: every non-empty expert's weights are cut into equally many contiguous pieces along k, one per
// work-group; fp32 partial sums [m][pieces][n] in the workspace, a second kernel adds them.  Needs n % 8 == 0,
// n <= 2048, k * n < 2^31 and a 16-byte aligned workspace of at least gmm_rows_workspace_bytes(m, n, 1) bytes (more
// room = more pieces, up to what keeps ~3 work-groups per compute unit busy).
size_t gmm_rows_workspace_bytes(int m, int n, int pieces);
int launch_gmm_rows(hipStream_t s, const DecodeArgs& a, int num_cus, void* workspace, size_t workspace_bytes);

// The same for weights stored [g, n, k] (trans_rhs): the stream is cut along n, every piece yields complete sums, one
// launch and no workspace.  DecodeArgs::A is then [g, n, k].  gmm_rows_t_fits: the shape can be served (k up to 8192).
// f8: x and A hold float8 e4m3fn bytes behind the same pointers (k % 16 == 0); y is bf16 either way.
bool gmm_rows_t_fits(int m, int k, int n, int g, bool f8 = false);
int launch_gmm_rows_t(hipStream_t s, const DecodeArgs& a, int num_cus, bool f8 = false);

}  // namespace rd
