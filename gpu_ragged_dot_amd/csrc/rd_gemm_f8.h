// float8 (OCP e4m3fn) operands on the float8 matrix-core instruction v_mfma_f32_32x32x64_f8f6f4 (64 contraction indices
// per instruction, fp32 accumulation, twice the rate of the bf16 instruction).  Same structure as the direct-to-LDS core
// of rd_gemm_dlds.h - a ring of K-slabs filled by buffer_load ... lds, one barrier per slab, the accumulators stored
// through LDS as bf16 - with one-byte elements.  The bytes are moved by the loader of a bf16 slab with the same row
// length (so its chunk permutations apply unchanged):
//   K-major operand  (contraction index contiguous): slab [rows][BK bytes], BK = 64 or 128; a lane's fragment is 32
//                    consecutive bytes of its row, two ds_read_b128;
//   MN-major operand (weights [k, n], both operands of tgmm): slab [BK][rows bytes]; the 8-bit transposing LDS read
//                    (ds_read_b64_tr_b8: 16 lanes read an 8 x 16 byte block, lane i gets the 8 bytes of column i) hands a
//                    lane 8 contraction-consecutive bytes of its column, four of them a fragment.
// Every e4m3 product is exact in fp32, so the result is what the bf16 path gives for the same values up to the order of
// the additions.  Needs 16-byte row pitches (k % 16 == 0, and n % 16 == 0 where n is a row pitch).
#pragma once
#include <type_traits>
#include "rd_gemm_dlds.h"

namespace rd {

// BK: contraction indices (= bytes) per slab row, 64 or 128.  128 makes every load cover whole 128-byte lines, which is
// what a memory-bound tile wants; 64 halves the slab, which is what lets a 256 x 256 tile keep four of them.
// B_AUX: cache policy of the B operand's loads (kCachePolicyStream: weights read once, not kept in L2).
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int STAGES_, int BK_ = 64, int B_AUX_ = 0, bool A_KMAJOR_ = true,
          bool B_KMAJOR_ = true, bool PINGPONG_ = false>
struct F8Cfg {
  typedef fp8_bits Elem;
  typedef bf16_bits Out;
  static constexpr bool F32 = false, F8DIRECT = true, HALF = false;
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, STAGES = STAGES_;
  static constexpr int B_AUX = B_AUX_;
  static_assert(BK == 64 || BK == 128, "contraction slab");
  // an MN-major slab row holds the operand's whole tile extent, and its chunk permutation needs 16 chunks (256 bytes)
  static_assert((A_KMAJOR_ || BM_ % 256 == 0) && (B_KMAJOR_ || BN_ % 256 == 0), "MN-major tile extents");
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, VEC = true, DLDS = true, PINGPONG = PINGPONG_, MIXED = false,
                        SPLITK = true;
  static constexpr int NW = WAVES_M * WAVES_N;
  static constexpr int NT = 64 * NW;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int KSTEPS = BK / 64;  // matrix-core steps per slab
  static constexpr int TARGET_WGS = (TM * TN * 16 <= 64) ? (NW >= 8 ? 2 : 3) : 1;
  static constexpr int WAVES_PER_EU = (NW / 4) * TARGET_WGS;
  static constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int EPI_PITCH = WN * 2 + 16;
  static constexpr int EPI_BYTES = NW * WM * EPI_PITCH;
  static constexpr int RING_BYTES = STAGES * STAGE_BYTES;
  static constexpr int LDS_BYTES = RING_BYTES > EPI_BYTES ? RING_BYTES : EPI_BYTES;
  static_assert(BM % 64 == 0 && BN % 64 == 0 && BM % (32 * WAVES_M) == 0 && BN % (32 * WAVES_N) == 0, "tile shape");
  static_assert(STAGES >= 2 && LDS_BYTES <= 160 * 1024, "LDS budget");
  static_assert(!PINGPONG_ || (NW == 8 && WAVES_M_ == 2 && STAGES_ >= 3 && BK_ == 64), "ping-pong runs two groups of four waves");
};

template <class C, class = void>
struct IsF8Direct { static constexpr bool value = false; };
template <class C>
struct IsF8Direct<C, decltype((void)C::F8DIRECT)> { static constexpr bool value = true; };

// Fragments of v_mfma_f32_32x32x64_f8f6f4: lane l feeds row / column (l & 31) and the 32 contraction bytes
// 32 (l >> 5) .. + 31 of a 64-deep step, in byte order - whatever the instruction's own numbering of them is, both
// operands are read the same way, so equal positions hold equal contraction indices.
typedef int i32x8_t __attribute__((ext_vector_type(8)));
// K-major slab [rows][BK bytes], the 16-byte chunks of a row permuted as the loader of a bf16 slab of the same row length
// leaves them (chunk c of row r at position c ^ ((r >> 2) & 3) for 64-byte rows, c ^ ((r >> 1) & 7) for 128-byte rows):
// two 16-byte chunks of the lane's row.
template <int BK>
struct F8FragReader {
  int addr[BK / 64][2];
  __device__ __forceinline__ void init(int row0, int lane) {
    const int r = lane & 31;
    const int sw = BK == 128 ? ((r >> 1) & 7) : ((r >> 2) & 3);
#pragma unroll
    for (int ws = 0; ws < BK / 64; ++ws)
#pragma unroll
      for (int h = 0; h < 2; ++h) addr[ws][h] = (row0 + r) * BK + (((4 * ws + 2 * (lane >> 5) + h) ^ sw) << 4);
  }
  __device__ __forceinline__ i32x8_t read(const unsigned char* region, int tile, int ws) const {
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(region + addr[ws][0] + tile * 32 * BK);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(region + addr[ws][1] + tile * 32 * BK);
    return i32x8_t{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  }
};
// MN-major slab [BK][ROW_BYTES], chunk c of contraction row kk at position c ^ ((kk & 3) << 2) (the loader of an MN-major
// bf16 slab): four 8-bit transposing reads (ds_read_b64_tr_b8) of 8 contraction rows each.  In one such read a 16-lane
// group fetches an 8 x 16 byte block - lane i supplies the address of row (i >> 1), bytes 8 (i & 1) .. + 7 - and lane i
// receives the 8 contraction-consecutive bytes of column i.
template <int ROW_BYTES, int TILES>
struct F8FragReaderT {
  int addr[TILES];
  __device__ __forceinline__ void init(int col0, int lane) {
    const int q = lane >> 4, i = lane & 15;
    const int row = 32 * (q >> 1) + (i >> 1);
    const int s = ((i >> 1) & 3) << 2;
#pragma unroll
    for (int j = 0; j < TILES; ++j) {
      const int chunk = ((col0 >> 4) + 2 * j + (q & 1)) ^ s;
      addr[j] = row * ROW_BYTES + (chunk << 4) + (i & 1) * 8;
    }
  }
  __device__ __forceinline__ i32x8_t read(const unsigned char* region, int tile, int ws) const {
    typedef int v2i_t __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) v2i_t* lds_v2i_ptr;
    const unsigned char* p = region + addr[tile] + ws * 64 * ROW_BYTES;
    const v2i_t a = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(p));
    const v2i_t b = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(p + 8 * ROW_BYTES));
    const v2i_t c = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(p + 16 * ROW_BYTES));
    const v2i_t d = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(p + 24 * ROW_BYTES));
    return i32x8_t{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
  }
};
template <int T, int BK, int TILES, bool KMAJOR>
struct F8Frag {
  F8FragReader<BK> km;
  F8FragReaderT<T, TILES> mn;
  __device__ __forceinline__ void init(int idx0, int lane) { if (KMAJOR) km.init(idx0, lane); else mn.init(idx0, lane); }
  __device__ __forceinline__ i32x8_t read(const unsigned char* region, int tile, int ws) const {
    return KMAJOR ? km.read(region, tile, ws) : mn.read(region, tile, ws);
  }
};

// Same contract as gemm_tile_dlds(): Ap/Bp point at the tile's first row (K-major) or column (MN-major) and first
// contraction index, lda/ldb are row pitches in elements (multiples of 16), a_lim/b_lim the live rows / columns of each
// operand, klen the contraction length (a multiple of 16 for K-major operands).
template <class C>
__device__ __forceinline__ void gemm_tile_f8(const fp8_bits* __restrict__ Ap, int lda, int a_lim,
                                             const fp8_bits* __restrict__ Bp, int ldb, int b_lim, int klen,
                                             bf16_bits* __restrict__ Op, int ldo, fp8_bits* smem_,
                                             const SplitK& sk = SplitK()) {
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;

  // The byte mover of a bf16 slab of the same row length.  K-major: [T rows][BK / 2 elements], pitch, tail length and
  // slab advance in 2-byte units.  MN-major: [BK rows][T / 2 elements], extent limit in 2-byte units, whole rows of k.
  constexpr int BK2 = C::BK / 2;
  typedef DldsLoader<C::A_KMAJOR ? C::BM : C::BM / 2, C::A_KMAJOR ? BK2 : C::BK, C::NW, C::A_KMAJOR> LdA;
  typedef DldsLoader<C::B_KMAJOR ? C::BN : C::BN / 2, C::B_KMAJOR ? BK2 : C::BK, C::NW, C::B_KMAJOR, C::B_AUX> LdB;
  LdA la; LdB lb;
  const int klen2 = klen >> 1;
  la.init(reinterpret_cast<const bf16_bits*>(Ap), lda >> 1, C::A_KMAJOR ? a_lim : (a_lim + 1) >> 1, C::A_KMAJOR ? klen2 : klen, wave, lane);
  lb.init(reinterpret_cast<const bf16_bits*>(Bp), ldb >> 1, C::B_KMAJOR ? b_lim : (b_lim + 1) >> 1, C::B_KMAJOR ? klen2 : klen, wave, lane);
  F8Frag<C::BM, C::BK, C::TM, C::A_KMAJOR> fra;
  F8Frag<C::BN, C::BK, C::TN, C::B_KMAJOR> frb;
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

  const int nk = (klen + C::BK - 1) / C::BK;
  constexpr int L = LdA::PER + LdB::PER;  // loads per thread per K-step

  auto issue_loads = [&](int step, int first, int count) {
    unsigned char* st = smem + (step % C::STAGES) * C::STAGE_BYTES;
    // The tail test only concerns K-major operands (whose counts are in 2-byte units, like klen2): an MN-major slab's
    // rows past the contraction length lie outside the loader's buffer and read as zeros by themselves.
    const int k0 = step * BK2;
    const bool tail = k0 + BK2 > klen2;
    __amdgpu_buffer_rsrc_t ra_ = la.resource(), rb_ = lb.resource();
#pragma unroll
    for (int q = first; q < first + count; ++q) {
      if (q < LdA::PER) {
        if (tail) la.template issue<true>(ra_, st, wave, q, k0, klen2);
        else la.template issue<false>(ra_, st, wave, q, k0, klen2);
      } else {
        if (tail) lb.template issue<true>(rb_, st + C::A_BYTES, wave, q - LdA::PER, k0, klen2);
        else lb.template issue<false>(rb_, st + C::A_BYTES, wave, q - LdA::PER, k0, klen2);
      }
    }
  };

#pragma unroll
  for (int s = 0; s < C::STAGES - 1; ++s)
    if (s < nk) { issue_loads(s, 0, L); la.advance(); lb.advance(); }

  for (int kt = 0; kt < nk; ++kt) {
    if (kt + C::STAGES - 2 < nk) wait_vmcnt<(C::STAGES - 2) * L>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();  // every wave's part of slab kt is in LDS, and slab kt-1 is no longer being read
    const bool more = kt + C::STAGES - 1 < nk;
    const unsigned char* ra = smem + (kt % C::STAGES) * C::STAGE_BYTES;
    const unsigned char* rb = ra + C::A_BYTES;
    // Fragments of step ks + 1 are fetched from LDS while the matrix core works on step ks, and the loads of the slab
    // STAGES - 1 ahead are issued a few at a time between the steps.
    constexpr int NSTEP = C::KSTEPS;
    i32x8_t fa[2][C::TM], fb[2][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i) fa[0][i] = fra.read(ra, i, 0);
#pragma unroll
    for (int j = 0; j < C::TN; ++j) fb[0][j] = frb.read(rb, j, 0);
#pragma unroll
    for (int ks = 0; ks < NSTEP; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < NSTEP) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) fa[nxt][i] = fra.read(ra, i, ks + 1);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) fb[nxt][j] = frb.read(rb, j, ks + 1);
      }
      if (more) {
        const int first = (L * ks) / NSTEP, last = (L * (ks + 1)) / NSTEP;
        issue_loads(kt + C::STAGES - 1, first, last - first);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (patch_live) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
          for (int j = 0; j < C::TN; ++j)  // both formats e4m3, no block scales: the plain 32x32x64 instruction
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[cur][j], fa[cur][i], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) { la.advance(); lb.advance(); }
  }

  __builtin_amdgcn_s_barrier();  // the ring is no longer read by any wave
  if (!splitk_combine<C>(acc, sk, tid, smem)) return;
  store_accumulators<C>(acc, wm, wn, wave, lane, a_lim, b_lim, Op, ldo, smem);
}

// The ping-pong schedule of rd_gemm_dlds.h on the float8 fragments: the eight waves form two groups of four (one wave of
// each per SIMD) that alternate, half a period apart, between a memory phase (the slab's fragments LDS -> registers,
// the wave's share of the direct loads of a later slab) and a compute phase (matrix-core instructions only), one
// work-group barrier per phase.
template <class C>
__device__ __forceinline__ void gemm_tile_f8_pingpong(const fp8_bits* __restrict__ Ap, int lda, int a_lim,
                                                      const fp8_bits* __restrict__ Bp, int ldb, int b_lim, int klen,
                                                      bf16_bits* __restrict__ Op, int ldo, fp8_bits* smem_,
                                                      const SplitK& sk = SplitK()) {
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const int group = wave >> 2;

  constexpr int BK2 = C::BK / 2;
  typedef DldsLoader<C::A_KMAJOR ? C::BM : C::BM / 2, C::A_KMAJOR ? BK2 : C::BK, C::NW, C::A_KMAJOR> LdA;
  typedef DldsLoader<C::B_KMAJOR ? C::BN : C::BN / 2, C::B_KMAJOR ? BK2 : C::BK, C::NW, C::B_KMAJOR, C::B_AUX> LdB;
  LdA la; LdB lb;
  const int klen2 = klen >> 1;
  la.init(reinterpret_cast<const bf16_bits*>(Ap), lda >> 1, C::A_KMAJOR ? a_lim : (a_lim + 1) >> 1, C::A_KMAJOR ? klen2 : klen, wave, lane);
  lb.init(reinterpret_cast<const bf16_bits*>(Bp), ldb >> 1, C::B_KMAJOR ? b_lim : (b_lim + 1) >> 1, C::B_KMAJOR ? klen2 : klen, wave, lane);
  F8Frag<C::BM, C::BK, C::TM, C::A_KMAJOR> fra;
  F8Frag<C::BN, C::BK, C::TN, C::B_KMAJOR> frb;
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

  const int nk = (klen + C::BK - 1) / C::BK;
  constexpr int L = LdA::PER + LdB::PER;

  auto issue_slab = [&](int step) {
    unsigned char* st = smem + (step % C::STAGES) * C::STAGE_BYTES;
    const int k0 = step * BK2;
    const bool tail = k0 + BK2 > klen2;
    __amdgpu_buffer_rsrc_t ra_ = la.resource(), rb_ = lb.resource();
#pragma unroll
    for (int q = 0; q < LdA::PER; ++q) {
      if (tail) la.template issue<true>(ra_, st, wave, q, k0, klen2);
      else la.template issue<false>(ra_, st, wave, q, k0, klen2);
    }
#pragma unroll
    for (int q = 0; q < LdB::PER; ++q) {
      if (tail) lb.template issue<true>(rb_, st + C::A_BYTES, wave, q, k0, klen2);
      else lb.template issue<false>(rb_, st + C::A_BYTES, wave, q, k0, klen2);
    }
    la.advance();
    lb.advance();
  };

#pragma unroll
  for (int s = 0; s < C::STAGES - 1; ++s)
    if (s < nk) issue_slab(s);
  if (C::STAGES - 1 <= nk) wait_vmcnt<(C::STAGES - 2) * L>(); else wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  if (group == 1) __builtin_amdgcn_s_barrier();

  for (int kt = 0; kt < nk; ++kt) {
    // ---- memory phase ---------------------------------------------------------------------------------------------
    const unsigned char* ra = smem + (kt % C::STAGES) * C::STAGE_BYTES;
    const unsigned char* rb = ra + C::A_BYTES;
    i32x8_t fa[C::TM], fb[C::TN];
    if (patch_live) {
#pragma unroll
      for (int i = 0; i < C::TM; ++i) fa[i] = fra.read(ra, i, 0);
#pragma unroll
      for (int j = 0; j < C::TN; ++j) fb[j] = frb.read(rb, j, 0);
    }
    if (kt + C::STAGES - 1 < nk) issue_slab(kt + C::STAGES - 1);
    if (kt + C::STAGES - 1 < nk) wait_vmcnt<(C::STAGES - 2) * L>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // ---- compute phase --------------------------------------------------------------------------------------------
    __builtin_amdgcn_s_setprio(1);
    if (patch_live) {
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], acc[i][j], 0, 0, 0, 0, 0, 0);
    }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
  if (group == 0) __builtin_amdgcn_s_barrier();
  if (!splitk_combine<C>(acc, sk, tid, smem)) return;
  store_accumulators<C>(acc, wm, wn, wave, lane, a_lim, b_lim, Op, ldo, smem);
}

}  // namespace rd
