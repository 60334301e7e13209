// Host-side check of rd::interleaved_slot() (gpu_ragged_dot_amd/csrc/rd_sched.h), the rule by which a gmm launch deals
// the blocks of long groups among those of short groups.  For every pair (long blocks L, live blocks N) tried:
//   - every entry of both lists is dealt exactly once (the launch computes the same tiles as in walk order);
//   - both lists are consumed in order (the walk's locality between consecutive blocks of a kind is kept);
//   - every XCD (position mod 8) receives floor or ceil of L / 8 long blocks;
//   - every complete round of 8 positions holds floor or ceil of 8 L / (8 floor(N / 8)) long blocks;
//   - where the function declines (nothing to mix, or too few short blocks for the incomplete last round) it
//     declines for every position.
// Built without GPU code by the library's Makefile; run by tests/test_host_checks.py.
#include <stdio.h>
#include <stdlib.h>
#include <vector>
#include "rd_sched.h"

static long long g_checked = 0;

static bool check(int L, int N) {
  std::vector<int> seen_long(L > 0 ? L : 0, 0), seen_short(N - L > 0 ? N - L : 0, 0);
  int per_xcd[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int last_long = -1, last_short = -1, declined = 0;
  const int rounds = N >> 3;
  std::vector<int> per_round(rounds > 0 ? rounds : 0, 0);
  for (int i = 0; i < N; ++i) {
    bool from_long = false;
    int rank = -1;
    if (!rd::interleaved_slot(i, L, N, &from_long, &rank)) { ++declined; continue; }
    if (declined) { fprintf(stderr, "L=%d N=%d: declined only for some positions\n", L, N); return false; }
    if (rank < 0 || rank >= (from_long ? L : N - L)) { fprintf(stderr, "L=%d N=%d i=%d: rank %d out of range\n", L, N, i, rank); return false; }
    int& seen = from_long ? seen_long[rank] : seen_short[rank];
    int& last = from_long ? last_long : last_short;
    if (seen++ || rank != last + 1) { fprintf(stderr, "L=%d N=%d i=%d: rank %d out of order or dealt twice\n", L, N, i, rank); return false; }
    last = rank;
    if (from_long) {
      ++per_xcd[i & 7];
      if ((i >> 3) >= rounds) { fprintf(stderr, "L=%d N=%d i=%d: long block in the incomplete last round\n", L, N, i); return false; }
      ++per_round[i >> 3];
    }
    ++g_checked;
  }
  if (declined) {
    const bool expected = L <= 0 || L >= N || L > (rounds << 3);
    if (!expected) { fprintf(stderr, "L=%d N=%d: declined without cause\n", L, N); return false; }
    return true;
  }
  if (last_long != L - 1 || last_short != N - L - 1) { fprintf(stderr, "L=%d N=%d: lists not exhausted\n", L, N); return false; }
  for (int x = 0; x < 8; ++x)
    if (per_xcd[x] < L / 8 || per_xcd[x] > (L + 7) / 8) { fprintf(stderr, "L=%d N=%d: XCD %d takes %d long blocks\n", L, N, x, per_xcd[x]); return false; }
  for (int r = 0; r < rounds; ++r)
    if (per_round[r] < L / rounds || per_round[r] > (L + rounds - 1) / rounds) {
      fprintf(stderr, "L=%d N=%d: round %d holds %d long blocks\n", L, N, r, per_round[r]);
      return false;
    }
  return true;
}

int main() {
  for (int N = 0; N <= 300; ++N)
    for (int L = 0; L <= N; ++L)
      if (!check(L, N)) return 1;
  // the ratios that put every long block on a few XCDs when only the sequence is spread (3/8, 1/2, 1/4, 1/8), larger
  // launches, and the largest list the library builds
  const int big[][2] = {{72, 192}, {81, 268}, {512, 1024}, {256, 1024}, {128, 1024}, {3000, 8000}, {1, 4097}, {4096, 4104},
                        {16381, 16382}, {1, rd::kMaxOrderedBlocks}, {rd::kMaxOrderedBlocks - 8, rd::kMaxOrderedBlocks}, {12345, rd::kMaxOrderedBlocks}};
  for (const auto& c : big)
    if (!check(c[0], c[1])) return 1;
  srand(7);
  for (int it = 0; it < 300; ++it) {
    const int N = 1 + rand() % rd::kMaxOrderedBlocks, L = rand() % (N + 1);
    if (!check(L, N)) return 1;
  }
  printf("block_order ok %lld\n", g_checked);
  return 0;
}
