// Four-wave GEMM core: a 256 x 256 tile held by a 2 x 2 grid of waves, 128 x 128 per wave (one wave per SIMD, all
// 512 registers).  Per 32-wide K-slab the four waves read 64 KB of fragments from LDS where the eight-wave cores read
// 96 KB - the LDS pipe is what paces those - at the price of having no second wave on the SIMD to hide latency: the
// wave itself keeps the matrix core fed, so every MFMA is followed in program order by at most one LDS read and the
// occasional direct load, and fragments are fetched half a slab ahead of their use.
//
// Pipeline (S = ring slots, one barrier per slab, in the middle of it):
//   first half of slab t : MFMAs on the fragments of (t, k 0..15) | read the fragments of (t, k 16..31) | request the
//                          second operand's part of slab t+S-1
//   wait: own share of slab t+1 landed, own LDS reads returned; barrier - slab t+1 is complete, slab t's slot is free
//   second half of slab t: MFMAs on (t, k 16..31) | read the fragments of (t+1, k 0..15) | request the first operand's
//                          part of slab t+S into the slot slab t just left
#pragma once
#include "rd_gemm_dlds.h"

namespace rd {

template <int BM_, int BN_, bool A_KMAJOR_, bool B_KMAJOR_, int STAGES_, bool HALF_ = false>
struct W4Cfg {
  typedef bf16_bits Elem;  // 16 bits per element: bf16, or float16 with HALF
  static constexpr bool F32 = false, W4 = true, HALF = HALF_;
  static constexpr int BM = BM_, BN = BN_, BK = 32, WAVES_M = 2, WAVES_N = 2, STAGES = STAGES_;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, VEC = true, DLDS = true, PINGPONG = false, MIXED = false,
                        SPLITK = true;
  static constexpr int NW = 4, NT = 256;
  static constexpr int WM = BM / 2, WN = BN / 2;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int KSTEPS = 2;
  static constexpr int WAVES_PER_EU = 1;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int EPI_PITCH = WN * 2 + 16;
  static constexpr int EPI_BYTES = NW * WM * EPI_PITCH;
  static constexpr int RING_BYTES = STAGES * STAGE_BYTES;
  static constexpr int LDS_BYTES = RING_BYTES > EPI_BYTES ? RING_BYTES : EPI_BYTES;
  static_assert(BM % 128 == 0 && BN % 128 == 0, "tile shape");
  static_assert(STAGES >= 3, "ring depth");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

namespace w4_detail {
template <bool V>
struct Flag { static constexpr bool value = V; };
}  // namespace w4_detail

// The K loop for a wave that has matrix-core work (LIVE) or only fetches its share of the slabs (!LIVE).
template <class C, bool LIVE>
__device__ __forceinline__ void w4_kloop(const bf16_bits* __restrict__ Ap, int lda, int a_lim,
                                         const bf16_bits* __restrict__ Bp, int ldb, int b_lim, int klen,
                                         unsigned char* smem, int wave, int lane, f32x16_t (&acc)[C::TM][C::TN]) {
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int S = C::STAGES;
  typedef DldsLoader<C::BM, C::BK, C::NW, C::A_KMAJOR> LdA;
  typedef DldsLoader<C::BN, C::BK, C::NW, C::B_KMAJOR> LdB;
  LdA la; LdB lb;
  la.init(Ap, lda, a_lim, klen, wave, lane);
  lb.init(Bp, ldb, b_lim, klen, wave, lane);
  DldsFragReader<C::BM, C::BK, C::TM, C::A_KMAJOR> fra;
  DldsFragReader<C::BN, C::BK, C::TN, C::B_KMAJOR> frb;
  fra.init(wm * C::WM, lane);
  frb.init(wn * C::WN, lane);

  const int nk = (klen + C::BK - 1) / C::BK;
  constexpr int L = LdA::PER + LdB::PER;
  constexpr int MF = C::TM * C::TN;  // MFMAs per half slab
  static_assert(MF >= 2 * LdA::PER && MF >= 2 * LdB::PER && MF >= C::TM + C::TN, "a half slab has room for its loads and reads");

  // one load of slab `step`; FULL: the slab lies wholly inside the contraction range
  auto issue_one_a = [&](int step, int slot_off, int q, auto full_tag) {
    unsigned char* st = smem + slot_off;
    const int k0 = step * C::BK;
    __amdgpu_buffer_rsrc_t r = la.resource();
    if (decltype(full_tag)::value || k0 + C::BK <= klen) la.template issue<false>(r, st, wave, q, k0, klen);
    else la.template issue<true>(r, st, wave, q, k0, klen);
  };
  auto issue_one_b = [&](int step, int slot_off, int q, auto full_tag) {
    unsigned char* st = smem + slot_off + C::A_BYTES;
    const int k0 = step * C::BK;
    __amdgpu_buffer_rsrc_t r = lb.resource();
    if (decltype(full_tag)::value || k0 + C::BK <= klen) lb.template issue<false>(r, st, wave, q, k0, klen);
    else lb.template issue<true>(r, st, wave, q, k0, klen);
  };

  // prologue: slabs 0 .. S-2 whole, and A's part of slab S-1 (B's part follows in the first half of slab 0)
#pragma unroll
  for (int s = 0; s < S; ++s) {
    if (s < nk) {
#pragma unroll
      for (int q = 0; q < LdA::PER; ++q) issue_one_a(s, s * C::STAGE_BYTES, q, w4_detail::Flag<false>{});
      la.advance();
      if (s < S - 1) {
#pragma unroll
        for (int q = 0; q < LdB::PER; ++q) issue_one_b(s, s * C::STAGE_BYTES, q, w4_detail::Flag<false>{});
        lb.advance();
      }
    }
  }
  // slab 0 landed (in the steady case S-2 whole slabs and one A part were requested after it)
  if (S <= nk) wait_vmcnt<(S - 2) * L + LdA::PER>(); else wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();

  bf16x8_t fa[2][C::TM], fb[2][C::TN];
  if (LIVE) {
    const unsigned char* ra = smem;
#pragma unroll
    for (int i = 0; i < C::TM; ++i) fa[0][i] = fra.read(ra, i, 0);
#pragma unroll
    for (int j = 0; j < C::TN; ++j) fb[0][j] = frb.read(ra + C::A_BYTES, j, 0);
  }

  // One slab.  STEADY: slabs kt+S-1 and kt+S exist and are whole, so nothing in here is conditional.
  // `cur`: byte offset of slab kt's ring slot, carried along instead of computing kt % S.
  int cur = 0;
  auto slab = [&](int kt, auto steady_tag) {
    constexpr bool STEADY = decltype(steady_tag)::value;
    const int prev_off = cur == 0 ? (S - 1) * C::STAGE_BYTES : cur - C::STAGE_BYTES;  // slot of slab kt-1 = of slab kt+S-1
    const int next_off = cur == (S - 1) * C::STAGE_BYTES ? 0 : cur + C::STAGE_BYTES;
    const unsigned char* ra = smem + cur;
    const unsigned char* rb = ra + C::A_BYTES;
    // ---- first half: MFMAs on k 0..15, fragments of k 16..31, B's part of slab kt+S-1 ---------------------------------
    const bool more_b = STEADY || kt + S - 1 < nk;
#pragma unroll
    for (int t = 0; t < MF; ++t) {
      const int i = t / C::TN, j = t % C::TN;
      if (LIVE) {
        if (t < C::TM) fa[1][t] = fra.read(ra, t, 1);
        else if (t < C::TM + C::TN) fb[1][t - C::TM] = frb.read(rb, t - C::TM, 1);
      }
      constexpr int T0 = MF - 2 * LdB::PER;
      if (t >= T0 && ((t - T0) & 1) == 0 && more_b) issue_one_b(kt + S - 1, prev_off, (t - T0) >> 1, steady_tag);
      if (LIVE) acc[i][j] = mfma_32x32x16<C::HALF>(fb[0][j], fa[0][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more_b) lb.advance();
    // ---- own share of slab kt+1 landed, own reads of slab kt returned ------------------------------------------------
    if (STEADY || kt + S - 1 < nk) wait_vmcnt<(S - 2) * L>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // ---- second half: MFMAs on k 16..31, fragments of (kt+1, k 0..15), A's part of slab kt+S into slab kt's slot ------
    const bool next = STEADY || kt + 1 < nk;
    const bool more_a = STEADY || kt + S < nk;
    const unsigned char* na = smem + next_off;
    const unsigned char* nb = na + C::A_BYTES;
#pragma unroll
    for (int t = 0; t < MF; ++t) {
      const int i = t / C::TN, j = t % C::TN;
      if (LIVE && next) {
        if (t < C::TM) fa[0][t] = fra.read(na, t, 0);
        else if (t < C::TM + C::TN) fb[0][t - C::TM] = frb.read(nb, t - C::TM, 0);
      }
      constexpr int T0 = MF - 2 * LdA::PER;
      if (t >= T0 && ((t - T0) & 1) == 0 && more_a) issue_one_a(kt + S, cur, (t - T0) >> 1, steady_tag);
      if (LIVE) acc[i][j] = mfma_32x32x16<C::HALF>(fb[1][j], fa[1][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more_a) la.advance();
    cur = next_off;
  };

  const int n_steady = klen / C::BK - S;  // slabs kt with (kt + S + 1) * BK <= klen
  int kt = 0;
  for (; kt < n_steady; ++kt) slab(kt, w4_detail::Flag<true>{});
  for (; kt < nk; ++kt) slab(kt, w4_detail::Flag<false>{});

  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_s_barrier();  // the ring is no longer read by any wave
}

template <class C>
__device__ __forceinline__ void gemm_tile_w4(const bf16_bits* __restrict__ Ap, int lda, int a_lim,
                                             const bf16_bits* __restrict__ Bp, int ldb, int b_lim, int klen,
                                             bf16_bits* __restrict__ Op, int ldo, bf16_bits* smem_,
                                             const SplitK& sk = SplitK()) {
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  // A wave whose whole patch lies past the tile's limits only fetches its share of the slabs.
  const bool patch_live = wm * C::WM < a_lim && wn * C::WN < b_lim;

  f32x16_t acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  if (patch_live) w4_kloop<C, true>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, smem, wave, lane, acc);
  else w4_kloop<C, false>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, smem, wave, lane, acc);

  if (!splitk_combine<C>(acc, sk, tid, smem)) return;
  store_accumulators<C>(acc, wm, wn, wave, lane, a_lim, b_lim, Op, ldo, smem);
}

}  // namespace rd
