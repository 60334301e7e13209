// Four-wave GEMM core for two K-major operands (gmm with trans_rhs: dout[m, n] and A[g, k, n] both run along the
// contraction index).  Same 2 x 2 grid of waves with 128 x 128 per wave as rd_gemm_w4.h, other data path:
//
//  * 64-wide slabs.  A wave-wide load then covers 8 rows x 128 bytes - whole cache lines - instead of 16 rows x 64
//    bytes.  With 32-wide slabs of two K-major operands the texture addresser is busy twice as long as in the forward
//    product and its address queue is full ten times as often, and a wave that cannot issue a load cannot issue the
//    MFMAs behind it either.
//  * HBM -> registers -> LDS.  A 64-wide slab of both operands is 64 KB, so LDS holds two of them; filled by
//    direct-to-LDS loads, the second slot would be in flight for at most the time one slab takes to multiply, which
//    is less than a load takes.  So the loads land in registers (two sets of 16 x 16 bytes per lane: two more slabs in
//    flight) and are written to LDS when a slot comes free, to the very place a direct load would have put them.
//
// Slab t lives in LDS slot t & 1 and, before that, in register set t & 1.  In every substep (16 MFMAs, fragments read
// one substep ahead) the wave moves four of its 16 pieces per slab from registers to LDS: during substeps 0 .. 2 of
// slab t the last twelve pieces of slab t + 1, into the slot slab t - 1 has left; during substep 3, after the barrier,
// the first four of slab t + 2, into the slot slab t has just left.  Each write is followed by the load of the same
// piece two slabs further on into the registers it freed.  So every load has two slabs' worth of time before it is
// needed, and the LDS writes are spread evenly among the fragment reads - written in a burst (all sixteen in two
// substeps) they saturate LDS together with the reads and cost a fifth of the rate.
#pragma once
#include "rd_gemm_dlds.h"

namespace rd {

template <int BM_, int BN_, bool HALF_ = false>
struct W4RCfg {
  typedef bf16_bits Elem;  // 16 bits per element: bf16, or float16 with HALF
  static constexpr bool F32 = false, W4 = true, W4R = true, HALF = HALF_;
  static constexpr int BM = BM_, BN = BN_, BK = 64, WAVES_M = 2, WAVES_N = 2, STAGES = 2;
  static constexpr bool A_KMAJOR = true, B_KMAJOR = true, VEC = true, DLDS = true, PINGPONG = false, MIXED = false, SPLITK = true;
  static constexpr int NW = 4, NT = 256;
  static constexpr int WM = BM / 2, WN = BN / 2;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int KSTEPS = 4;
  static constexpr int WAVES_PER_EU = 1;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  static constexpr int SLOT_BYTES = A_BYTES + B_BYTES;
  static constexpr int EPI_PITCH = WN * 2 + 16;
  static constexpr int EPI_BYTES = NW * WM * EPI_PITCH;
  static constexpr int RING_BYTES = 2 * SLOT_BYTES;
  // the whole of LDS: the streaming routines for short groups that run in the same launch use it all
  static constexpr int LDS_BYTES = 160 * 1024;
  static_assert(BM % 128 == 0 && BN % 128 == 0, "tile shape");
  static_assert(RING_BYTES <= LDS_BYTES && EPI_BYTES <= LDS_BYTES, "LDS budget");
};

namespace w4r_detail {
template <int V>
struct Int { static constexpr int value = V; };
}  // namespace w4r_detail

template <class C, bool LIVE>
__device__ __forceinline__ void w4r_kloop(const bf16_bits* __restrict__ Ap, int lda, int a_lim,
                                          const bf16_bits* __restrict__ Bp, int ldb, int b_lim, int klen,
                                          unsigned char* smem, int wave, int lane, f32x16_t (&acc)[C::TM][C::TN]) {
  const int wm = wave >> 1, wn = wave & 1;
  typedef DldsLoader<C::BM, C::BK, C::NW, true> LdA;
  typedef DldsLoader<C::BN, C::BK, C::NW, true> LdB;
  LdA la; LdB lb;
  la.init(Ap, lda, a_lim, klen, wave, lane);
  lb.init(Bp, ldb, b_lim, klen, wave, lane);
  DldsFragReader<C::BM, C::BK, C::TM, true> fra;
  DldsFragReader<C::BN, C::BK, C::TN, true> frb;
  fra.init(wm * C::WM, lane);
  frb.init(wn * C::WN, lane);

  const int nk = (klen + C::BK - 1) / C::BK;
  constexpr int PA = LdA::PER, PB = LdB::PER, P = PA + PB;  // pieces per lane per slab
  constexpr int MF = C::TM * C::TN;                        // MFMAs per substep
  constexpr int R0 = C::TM + C::TN;  // gaps between MFMAs that the fragment reads of a substep take
  constexpr int HEAD = P / 4;  // pieces moved in substep 3 (of the slab after next); the rest go four per substep 0 .. 2
  static_assert(P % 4 == 0 && 2 * HEAD <= MF - R0, "every substep has a slot for its pieces");

  u32x4_t regs[2][P];  // register set s & 1: slab s between its loads and its write to LDS
  // piece q of slab `step` -> regs[SET][q].  The loaders' bases stand at slab `step` (they advance once per slab).
  auto fetch_one = [&](auto set_tag, int step, int q, auto full_tag) {
    constexpr int SET = decltype(set_tag)::value;
    const int k0 = step * C::BK;
    const bool tail = !decltype(full_tag)::value && k0 + C::BK > klen;
    if (q < PA) {
      int off = la.voff[q];
      if (tail && k0 + la.kcol >= klen) off = kOobOffset;
      regs[SET][q] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(la.resource(), off, 0, 0));
    } else {
      int off = lb.voff[q - PA];
      if (tail && k0 + lb.kcol >= klen) off = kOobOffset;
      regs[SET][q] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(lb.resource(), off, 0, 0));
    }
  };
  // regs[SET][q] -> where a direct-to-LDS load of the same piece would have landed in the slot
  auto commit_one = [&](auto set_tag, int slot_off, int q) {
    constexpr int SET = decltype(set_tag)::value;
    unsigned char* st = smem + slot_off + (q < PA ? (wave + C::NW * q) * 1024 : C::A_BYTES + (wave + C::NW * (q - PA)) * 1024) + lane * 16;
    *reinterpret_cast<u32x4_t*>(st) = regs[SET][q];
  };

  // prologue: slab 0 through the registers into LDS, slab 1 in registers, slab 2 requested
  auto prologue = [&](auto all_tag) {
    constexpr bool ALL = decltype(all_tag)::value != 0;  // at least four slabs, the first four whole
    if (ALL || 0 < nk) {
#pragma unroll
      for (int q = 0; q < P; ++q) fetch_one(w4r_detail::Int<0>{}, 0, q, all_tag);
      la.advance(); lb.advance();
    }
    if (ALL || 1 < nk) {
#pragma unroll
      for (int q = 0; q < P; ++q) fetch_one(w4r_detail::Int<1>{}, 1, q, all_tag);
      la.advance(); lb.advance();
    }
    if (ALL || 0 < nk) {
#pragma unroll
      for (int q = 0; q < P; ++q) commit_one(w4r_detail::Int<0>{}, 0, q);
    }
    if (ALL || 2 < nk) {
#pragma unroll
      for (int q = 0; q < P; ++q) fetch_one(w4r_detail::Int<0>{}, 2, q, all_tag);
      la.advance(); lb.advance();
    }
    if (ALL || 1 < nk) {
#pragma unroll
      for (int q = 0; q < HEAD; ++q) commit_one(w4r_detail::Int<1>{}, C::SLOT_BYTES, q);
    }
    if (ALL || 3 < nk) {
#pragma unroll
      for (int q = 0; q < HEAD; ++q) fetch_one(w4r_detail::Int<1>{}, 3, q, all_tag);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): slab 0 is written
    __builtin_amdgcn_s_barrier();
  };

  bf16x8_t fa[2][C::TM], fb[2][C::TN];
  auto first_fragments = [&]() {
    if (LIVE) {
#pragma unroll
      for (int i = 0; i < C::TM; ++i) fa[0][i] = fra.read(smem, i, 0);
#pragma unroll
      for (int j = 0; j < C::TN; ++j) fb[0][j] = frb.read(smem + C::A_BYTES, j, 0);
    }
  };

  // Slab t; NEXT = (t + 1) & 1 names the register set of slab t + 1 (and t + 3) and the LDS slot it goes to.
  // STEADY: slabs t + 1 and t + 3 exist and slab t + 3 is whole, so nothing in here is conditional.
  auto slab = [&](int t, auto next_tag, auto steady_tag) {
    constexpr int NEXT = decltype(next_tag)::value;
    constexpr bool STEADY = decltype(steady_tag)::value != 0;
    const int cur_off = (1 - NEXT) * C::SLOT_BYTES, next_off = NEXT * C::SLOT_BYTES;
    const unsigned char* ra = smem + cur_off;
    const unsigned char* rb = ra + C::A_BYTES;
    const bool write_next = STEADY || t + 1 < nk;  // slab t + 1 is still in registers (all but its first pieces)
    const bool fetch_far = STEADY || t + 3 < nk;
    const bool write_after = STEADY || t + 2 < nk, fetch_after = STEADY || t + 4 < nk;
    // ---- substeps 0 .. 2: MFMAs on (t, u), fragments of (t, u + 1); in substeps 0 and 1 the pieces of slab t + 1 go
    //      from registers to LDS, each followed by the load of the same piece of slab t + 3 ------------------------------
#pragma unroll
    for (int u = 0; u < 3; ++u) {
#pragma unroll
      for (int m = 0; m < MF; ++m) {
        const int i = m / C::TN, j = m % C::TN;
        if (LIVE) {
          if (m < C::TM) fa[(u + 1) & 1][m] = fra.read(ra, m, u + 1);
          else if (m < C::TM + C::TN) fb[(u + 1) & 1][m - C::TM] = frb.read(rb, m - C::TM, u + 1);
        }
        // after the fragment reads: a write in every other gap between MFMAs, the load that refills its registers in the
        // gap behind it
        if (m >= R0 && (m - R0) / 2 < HEAD) {
          const int q = HEAD + u * HEAD + (m - R0) / 2;
          if (((m - R0) & 1) == 0) { if (write_next) commit_one(next_tag, next_off, q); }
          else if (fetch_far) fetch_one(next_tag, t + 3, q, steady_tag);
        }
        if (LIVE) acc[i][j] = mfma_32x32x16<C::HALF>(fb[u & 1][j], fa[u & 1][i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (fetch_far) { la.advance(); lb.advance(); }
    // ---- own LDS reads of slab t returned, own pieces of slab t + 1 written; barrier: slab t + 1 is complete ----------
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // ---- substep 3: MFMAs on (t, 3), fragments of (t + 1, 0) ---------------------------------------------------------
    const bool next = STEADY || t + 1 < nk;
    const unsigned char* na = smem + next_off;
    const unsigned char* nb = na + C::A_BYTES;
#pragma unroll
    for (int m = 0; m < MF; ++m) {
      const int i = m / C::TN, j = m % C::TN;
      if (LIVE && next) {
        if (m < C::TM) fa[0][m] = fra.read(na, m, 0);
        else if (m < C::TM + C::TN) fb[0][m - C::TM] = frb.read(nb, m - C::TM, 0);
      }
      if (m >= R0 && (m - R0) / 2 < HEAD) {
        const int q = (m - R0) / 2;
        if (((m - R0) & 1) == 0) { if (write_after) commit_one(w4r_detail::Int<1 - NEXT>{}, cur_off, q); }
        else if (fetch_after) fetch_one(w4r_detail::Int<1 - NEXT>{}, t + 4, q, steady_tag);
      }
      if (LIVE) acc[i][j] = mfma_32x32x16<C::HALF>(fb[1][j], fa[1][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // The steady loop is entered straight from the unconditional prologue: the compiler counts the loads outstanding at
  // each register's use along every path into the loop, and a path on which slab 2 was not requested would halve them.
  const int n_steady = (klen / C::BK - 4) & ~1;  // slabs t < n_steady have (t + 5) * BK <= klen; an even count
  int t = 0;
  if (n_steady > 0) {
    prologue(w4r_detail::Int<1>{});
    first_fragments();
    for (; t < n_steady; t += 2) {
      slab(t, w4r_detail::Int<1>{}, w4r_detail::Int<1>{});
      slab(t + 1, w4r_detail::Int<0>{}, w4r_detail::Int<1>{});
    }
  } else {
    prologue(w4r_detail::Int<0>{});
    first_fragments();
  }
  for (; t < nk; t += 2) {
    slab(t, w4r_detail::Int<1>{}, w4r_detail::Int<0>{});
    if (t + 1 < nk) slab(t + 1, w4r_detail::Int<0>{}, w4r_detail::Int<0>{});
  }

  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_s_barrier();  // the slots are no longer read by any wave
}

template <class C>
__device__ __forceinline__ void gemm_tile_w4r(const bf16_bits* __restrict__ Ap, int lda, int a_lim,
                                              const bf16_bits* __restrict__ Bp, int ldb, int b_lim, int klen,
                                              bf16_bits* __restrict__ Op, int ldo, bf16_bits* smem_,
                                              const SplitK& sk = SplitK()) {
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const bool patch_live = wm * C::WM < a_lim && wn * C::WN < b_lim;

  f32x16_t acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  if (patch_live) w4r_kloop<C, true>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, smem, wave, lane, acc);
  else w4r_kloop<C, false>(Ap, lda, a_lim, Bp, ldb, b_lim, klen, smem, wave, lane, acc);

  if (!splitk_combine<C>(acc, sk, tid, smem)) return;
  store_accumulators<C>(acc, wm, wn, wave, lane, a_lim, b_lim, Op, ldo, smem);
}

}  // namespace rd
