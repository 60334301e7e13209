// Ping-pong GEMM core with one LDS ring per operand.  Same schedule as gemm_tile_pingpong() (two groups of four waves,
// memory phase / compute phase, K advancing 32 per phase), but an operand whose contraction index is contiguous in
// memory ("K-major") can be fetched in 64-wide slabs every other phase instead of 32-wide slabs every phase: its loads
// then cover whole 128-byte lines (8 rows x 128 B per wave-wide load instead of 16 rows x 64 B), which halves what the
// L1/texture path has to do for them - the bottleneck of the products that read x, dout or A[g,n,k] along rows.
#pragma once
#include "rd_gemm_dlds.h"

namespace rd {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, bool A_KMAJOR_, bool B_KMAJOR_, int A_W_, int A_S_, int B_W_,
          int B_S_>
struct PpCfg {
  typedef bf16_bits Elem;
  static constexpr bool F32 = false, HALF = false;
  static constexpr int BM = BM_, BN = BN_, BK = 32, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, VEC = true, DLDS = true, PINGPONG = true, MIXED = true,
                        SPLITK = true;
  static constexpr int A_W = A_W_, A_S = A_S_, B_W = B_W_, B_S = B_S_;  // slab width (contraction), ring slots
  static constexpr int STAGES = A_S < B_S ? A_S : B_S;
  static constexpr int NW = WAVES_M * WAVES_N, NT = 64 * NW;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int KSTEPS = 2;  // 16-wide MFMA substeps per phase
  static constexpr int WAVES_PER_EU = NW / 4;
  static constexpr int A_SLAB = BM * A_W * 2, B_SLAB = BN * B_W * 2;
  static constexpr int A_RING = A_S * A_SLAB, B_RING = B_S * B_SLAB;
  static constexpr int EPI_PITCH = WN * 2 + 16;
  static constexpr int EPI_BYTES = NW * WM * EPI_PITCH;
  static constexpr int RING_BYTES = A_RING + B_RING;
  static constexpr int LDS_BYTES = RING_BYTES > EPI_BYTES ? RING_BYTES : EPI_BYTES;
  static_assert(NW == 8 && WAVES_M == 2, "two groups of four waves");
  static_assert((A_W == 32 || (A_W == 64 && A_KMAJOR)) && (B_W == 32 || (B_W == 64 && B_KMAJOR)), "64-wide slabs are for K-major operands");
  static_assert(A_S >= 3 && B_S >= 3, "ring depth");
  static_assert(BM % 128 == 0 && BN % 128 == 0, "tile shape");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

namespace pp_detail {

template <int V>
struct Parity { static constexpr int value = V; };

// Loads a wave issues in a phase of the given parity, and how many of them come after operand `which`'s own loads
// (issue order inside a phase: A first, then B).
template <class C, class LdA, class LdB>
struct Counts {
  static constexpr int LA = LdA::PER, LB = LdB::PER;
  static constexpr int issued(int parity) {
    return ((C::A_W == 32 || parity == 0) ? LA : 0) + ((C::B_W == 32 || parity == 0) ? LB : 0);
  }
  static constexpr int after(int which, int parity) {  // which: 0 = A, 1 = B
    return which == 0 ? ((C::B_W == 32 || parity == 0) ? LB : 0) : 0;
  }
  static constexpr int between(int e, int p) {  // loads issued in phases e+1 .. p
    int n = 0;
    for (int t = e + 1; t <= p; ++t) n += issued(t & 1);
    return n;
  }
  // Largest number of still-outstanding loads at the end of memory phase p (steady state) such that every load the
  // next phase depends on has landed.
  static constexpr int allowed(int parity) {
    const int p = 64 + parity;
    int n = 1 << 20;
    // A
    if (C::A_W == 32) { const int e = p - C::A_S + 2; const int v = after(0, e & 1) + between(e, p); n = v < n ? v : n; }
    else if (parity == 1) { const int e = p - 2 * C::A_S + 3; const int v = after(0, e & 1) + between(e, p); n = v < n ? v : n; }
    // B
    if (C::B_W == 32) { const int e = p - C::B_S + 2; const int v = after(1, e & 1) + between(e, p); n = v < n ? v : n; }
    else if (parity == 1) { const int e = p - 2 * C::B_S + 3; const int v = after(1, e & 1) + between(e, p); n = v < n ? v : n; }
    return n > 63 ? 63 : n;
  }
};

}  // namespace pp_detail

template <class C>
__device__ __forceinline__ void gemm_tile_pingpong_mixed(const bf16_bits* __restrict__ Ap, int lda, int a_lim,
                                                         const bf16_bits* __restrict__ Bp, int ldb, int b_lim,
                                                         int klen, bf16_bits* __restrict__ Op, int ldo,
                                                         bf16_bits* smem_, const SplitK& sk = SplitK()) {
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const int group = wave >> 2;

  typedef DldsLoader<C::BM, C::A_W, C::NW, C::A_KMAJOR> LdA;
  typedef DldsLoader<C::BN, C::B_W, C::NW, C::B_KMAJOR> LdB;
  typedef pp_detail::Counts<C, LdA, LdB> Cnt;
  LdA la; LdB lb;
  la.init(Ap, lda, a_lim, klen, wave, lane);
  lb.init(Bp, ldb, b_lim, klen, wave, lane);
  DldsFragReader<C::BM, C::A_W, C::TM, C::A_KMAJOR> fra;
  DldsFragReader<C::BN, C::B_W, C::TN, C::B_KMAJOR> frb;
  fra.init(wm * C::WM, lane);
  frb.init(wn * C::WN, lane);
  const bool patch_live = wm * C::WM < a_lim && wn * C::WN < b_lim;

  f32x16_t acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int nk = (klen + 31) >> 5;                       // phases
  const int na = C::A_W == 64 ? (nk + 1) >> 1 : nk;      // slabs of A
  const int nb = C::B_W == 64 ? (nk + 1) >> 1 : nk;      // slabs of B
  unsigned char* ring_a = smem;
  unsigned char* ring_b = smem + C::A_RING;

  auto issue_a = [&](int slab) {
    unsigned char* st = ring_a + (slab % C::A_S) * C::A_SLAB;
    const int k0 = slab * C::A_W;
    const bool tail = k0 + C::A_W > klen;
    __amdgpu_buffer_rsrc_t r = la.resource();
#pragma unroll
    for (int q = 0; q < LdA::PER; ++q) {
      if (tail) la.template issue<true>(r, st, wave, q, k0, klen);
      else la.template issue<false>(r, st, wave, q, k0, klen);
    }
    la.advance();
  };
  auto issue_b = [&](int slab) {
    unsigned char* st = ring_b + (slab % C::B_S) * C::B_SLAB;
    const int k0 = slab * C::B_W;
    const bool tail = k0 + C::B_W > klen;
    __amdgpu_buffer_rsrc_t r = lb.resource();
#pragma unroll
    for (int q = 0; q < LdB::PER; ++q) {
      if (tail) lb.template issue<true>(r, st, wave, q, k0, klen);
      else lb.template issue<false>(r, st, wave, q, k0, klen);
    }
    lb.advance();
  };

  // prologue: fill each ring up to its look-ahead and let it all land
#pragma unroll
  for (int s = 0; s < C::A_S - 1; ++s)
    if (s < na) issue_a(s);
#pragma unroll
  for (int s = 0; s < C::B_S - 1; ++s)
    if (s < nb) issue_b(s);
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  if (group == 1) __builtin_amdgcn_s_barrier();

  // one phase; PAR = p & 1 is a compile-time constant so that the wait counts are immediates
  auto phase = [&](int p, auto par_tag) {
    constexpr int PAR = decltype(par_tag)::value;
    const int qa = C::A_W == 64 ? p >> 1 : p, qb = C::B_W == 64 ? p >> 1 : p;
    const unsigned char* ra = ring_a + (qa % C::A_S) * C::A_SLAB;
    const unsigned char* rb = ring_b + (qb % C::B_S) * C::B_SLAB;
    constexpr int KA = C::A_W == 64 ? 2 * PAR : 0, KB = C::B_W == 64 ? 2 * PAR : 0;  // substep offset inside a 64-wide slab
    // ---- memory phase ---------------------------------------------------------------------------------------------
    bf16x8_t fa[C::KSTEPS][C::TM], fb[C::KSTEPS][C::TN];
    // `steady`: both rings still have a slab to request at their look-ahead distance.  It can only turn false once,
    // towards the end of the K loop, so while it holds every earlier phase issued its full complement of loads.
    const bool steady = qa + C::A_S - 1 < na && qb + C::B_S - 1 < nb;
    const bool do_a = (C::A_W == 32 || PAR == 0) && qa + C::A_S - 1 < na;
    const bool do_b = (C::B_W == 32 || PAR == 0) && qb + C::B_S - 1 < nb;
    // Request the far slab before reading this phase's fragments: the texture path takes the requests at its own
    // pace while the LDS reads run, instead of after them.
    if (do_a) issue_a(qa + C::A_S - 1);
    if (do_b) issue_b(qb + C::B_S - 1);
    __builtin_amdgcn_sched_barrier(0);
    if (patch_live) {  // a wave without matrix-core work leaves the LDS bandwidth, which paces the loop, to the others
#pragma unroll
      for (int ks = 0; ks < C::KSTEPS; ++ks) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) fa[ks][i] = fra.read(ra, i, ks + KA);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) fb[ks][j] = frb.read(rb, j, ks + KB);
      }
    }
    // Own share of everything the next phase reads has landed.  The immediate count is exact in the steady state;
    // near the end, where fewer loads are in flight than it assumes, wait for all of them.
    if (steady) wait_vmcnt<Cnt::allowed(PAR)>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // ---- compute phase --------------------------------------------------------------------------------------------
    __builtin_amdgcn_s_setprio(1);
    if (patch_live) {
#pragma unroll
      for (int ks = 0; ks < C::KSTEPS; ++ks)
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
          for (int j = 0; j < C::TN; ++j)
            acc[i][j] = mfma_32x32x16<C::HALF>(fb[ks][j], fa[ks][i], acc[i][j]);
    }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  for (int p = 0; p < nk; p += 2) {
    phase(p, pp_detail::Parity<0>{});
    if (p + 1 < nk) phase(p + 1, pp_detail::Parity<1>{});
  }
  if (group == 0) __builtin_amdgcn_s_barrier();

  if (!splitk_combine<C>(acc, sk, tid, smem)) return;
  store_accumulators<C>(acc, wm, wn, wave, lane, a_lim, b_lim, Op, ldo, smem);
}

}  // namespace rd
