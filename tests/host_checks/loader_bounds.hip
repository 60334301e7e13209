// Host-side check of the direct-to-LDS operand loaders (DldsLoader in gpu_ragged_dot_amd/csrc/rd_gemm_dlds.h), which
// every large-tile core shares - with direct-to-LDS loads and, in the register-staged core, with plain buffer loads.
// No GPU is used: DldsLoader::init / advance are integer arithmetic and run here as they do on the device.
//
// Every K loop in the tree keeps one invariant: the loads of slab s are issued when the loader has been advanced s
// times (resource() then describes the bytes from slab s to the end of the operand window), with the per-lane offsets
// voff[], and - for a K-major operand whose slab runs past the contraction length - the chunks at or past it replaced
// by an offset beyond the buffer.  Under that invariant this program walks every load of every slab of every wave and
// lane for the loader shapes compiled into the library, on operand windows with ragged edges (row / column limits,
// contraction tails, the DeepSeek-V3 and Mixtral pitches), and checks that
//   * the byte count handed to the buffer resource is positive whenever a load is issued (a count that has gone to zero
//     or below would switch the hardware's range check off);
//   * a load the range check lets through (offset + 16 <= count) reads only elements of the window: row / column below
//     the tile's limit, contraction index below the contraction length and inside the slab being loaded;
//   * every element of the window that belongs to the slab is read exactly once (nothing missing, nothing twice);
//   * every offset is 16-byte aligned and non-negative.
// Prints "loader_bounds ok <loads checked>" and returns 0, or the first violation and 1.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "rd_gemm_dlds.h"

using namespace rd;

static long long g_loads = 0;

template <int T, int BK, int NW, bool KMAJOR>
static bool check_window(int lim, int ld, int klen, const char* what) {
  typedef DldsLoader<T, BK, NW, KMAJOR> Ld;
  const int nk = (klen + BK - 1) / BK;
  // all (wave, lane) loaders, advanced in lock step
  std::vector<Ld> ld_all((size_t)NW * 64);
  for (int w = 0; w < NW; ++w)
    for (int l = 0; l < 64; ++l) ld_all[(size_t)w * 64 + l].init(nullptr, ld, lim, klen, w, l);
  const long long window = KMAJOR ? ((long long)(lim - 1) * ld + klen) * 2 : ((long long)(klen - 1) * ld + lim) * 2;
  std::vector<unsigned char> seen;
  for (int s = 0; s < nk; ++s) {
    const int k0 = s * BK, kend = k0 + BK < klen ? k0 + BK : klen;
    const int rows = KMAJOR ? lim : kend - k0, cols = KMAJOR ? kend - k0 : lim;  // the slab's valid elements, [rows][cols]
    seen.assign((size_t)rows * cols, 0);
    for (int w = 0; w < NW; ++w)
      for (int l = 0; l < 64; ++l) {
        const Ld& L = ld_all[(size_t)w * 64 + l];
        const long long base_bytes = reinterpret_cast<const unsigned char*>(L.base) - static_cast<const unsigned char*>(nullptr);
        if (L.records <= 0) {
          std::printf("%s: T=%d BK=%d NW=%d kmajor=%d lim=%d ld=%d klen=%d slab %d: byte count %d not positive\n", what, T, BK, NW,
                      (int)KMAJOR, lim, ld, klen, s, L.records);
          return false;
        }
        if (base_bytes + L.records != window) {
          std::printf("%s: lim=%d ld=%d klen=%d slab %d: base + count = %lld, window %lld\n", what, lim, ld, klen, s,
                      base_bytes + L.records, window);
          return false;
        }
        const bool tail = k0 + BK > klen;
        for (int j = 0; j < Ld::PER; ++j) {
          int off = L.voff[j];
          if (KMAJOR && tail && k0 + L.kcol >= klen) off = kOobOffset;  // DldsLoader::issue<true>, w4r's fetch_one
          ++g_loads;
          if (off < 0 || (off & 15) != 0) {
            std::printf("%s: lim=%d ld=%d klen=%d slab %d wave %d lane %d load %d: offset %d\n", what, lim, ld, klen, s, w, l, j, off);
            return false;
          }
          if ((long long)off + 16 > L.records) continue;  // out of range: the hardware returns zeros and touches nothing
          const long long e0 = (base_bytes + off) / 2;    // first of 8 elements, from the window's origin
          for (int e = 0; e < 8; ++e) {
            const long long el = e0 + e;
            const long long major = el / ld, minor = el % ld;  // K-major: (row, k); MN-major: (k, column)
            const long long r = KMAJOR ? major : major - k0, c = KMAJOR ? minor - k0 : minor;
            if (r < 0 || r >= rows || c < 0 || c >= cols) {
              std::printf("%s: T=%d BK=%d NW=%d kmajor=%d lim=%d ld=%d klen=%d slab %d wave %d lane %d load %d: element (%lld, %lld) "
                          "outside the slab's %d x %d valid elements\n", what, T, BK, NW, (int)KMAJOR, lim, ld, klen, s, w, l, j, r, c, rows, cols);
              return false;
            }
            if (seen[(size_t)r * cols + c]++) {
              std::printf("%s: lim=%d ld=%d klen=%d slab %d: element (%lld, %lld) read twice\n", what, lim, ld, klen, s, r, c);
              return false;
            }
          }
        }
      }
    for (size_t i = 0; i < seen.size(); ++i)
      if (!seen[i]) {
        std::printf("%s: T=%d BK=%d NW=%d kmajor=%d lim=%d ld=%d klen=%d slab %d: element (%zu, %zu) never read\n", what, T, BK, NW,
                    (int)KMAJOR, lim, ld, klen, s, i / cols, i % cols);
        return false;
      }
    for (auto& L : ld_all) L.advance();
  }
  return true;
}

template <int T, int BK, int NW, bool KMAJOR>
static bool check_loader(const char* what) {
  // row pitches: DeepSeek-V3 (2048, 7168), Mixtral (4096, 14336), and small ones; limits and contraction lengths with
  // ragged ends (multiples of 8 where they are row pitches of 16-byte loads: the contraction length of a K-major
  // operand, the column limit of an MN-major one; the rows of a group - tgmm's contraction - are arbitrary)
  const int pitches[] = {2048, 7168, 4096, 14336, 264, T > 256 ? T : 256};
  const int lims_k[] = {1, 4, 7, 21, 33, 64, 100, 128, 129, 255, 256};
  const int lims_mn[] = {8, 24, 64, 120, 128, 136, 248, 256};
  const int klens_k[] = {8, 16, 24, 32, 40, 64, 72, 200, 2040, 2048};
  const int klens_mn[] = {1, 2, 7, 31, 32, 33, 63, 64, 65, 100, 257, 1219};
  for (int ld : pitches)
    for (int lim : (KMAJOR ? std::vector<int>(lims_k, lims_k + 11) : std::vector<int>(lims_mn, lims_mn + 8)))
      for (int klen : (KMAJOR ? std::vector<int>(klens_k, klens_k + 10) : std::vector<int>(klens_mn, klens_mn + 12))) {
        if (lim > T) continue;
        if (KMAJOR ? klen > ld : lim > ld) continue;
        if (!check_window<T, BK, NW, KMAJOR>(lim, ld, klen, what)) return false;
      }
  return true;
}

int main() {
  bool ok = true;
  // (tile extent, slab depth, waves, K-major): the loader shapes of the compiled cores
  ok = ok && check_loader<256, 32, 4, true>("four-wave core, K-major operand");
  ok = ok && check_loader<256, 32, 4, false>("four-wave core, MN-major operand");
  ok = ok && check_loader<256, 64, 4, true>("four-wave register-staged core (64-wide slabs through plain buffer loads)");
  ok = ok && check_loader<256, 32, 8, true>("eight-wave cores, K-major operand");
  ok = ok && check_loader<256, 32, 8, false>("eight-wave cores, MN-major operand");
  ok = ok && check_loader<256, 64, 8, true>("per-operand rings, 64-wide K-major slabs");
  ok = ok && check_loader<128, 32, 8, true>("128 x 256 ping-pong core, rows");
  ok = ok && check_loader<128, 32, 8, false>("128 x 256 ping-pong core, MN-major rows (tgmm)");
  ok = ok && check_loader<128, 32, 4, true>("128 x 128 core, K-major");
  ok = ok && check_loader<128, 32, 4, false>("128 x 128 core, MN-major");
  ok = ok && check_loader<64, 32, 4, true>("64-row streaming routine, activations (32-wide slabs)");
  ok = ok && check_loader<64, 64, 4, true>("64-row streaming routine, activations (64-wide slabs)");
  ok = ok && check_loader<128, 64, 4, true>("128-row streaming routine, activations (64-wide slabs)");
  if (!ok) return 1;
  std::printf("loader_bounds ok %lld\n", g_loads);
  return 0;
}
