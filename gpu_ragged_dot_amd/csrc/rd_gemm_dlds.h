// The large-tile GEMM core: HBM -> LDS without a stop in registers (buffer_load_dwordx4 ... lds), STAGES-deep ring of
// K-slabs in LDS, one barrier per K-step.  Same contract as gemm_tile() in rd_gemm_tile.h; used for the tall tiles
// that carry the compute-bound shapes.  Needs 16-byte row pitches.
//
// LDS layout.  A wave-wide direct load deposits 64 x 16 B contiguously, so rows cannot be padded; bank conflicts are
// avoided by permuting which 16-byte chunk of a row each lane fetches (an XOR on the chunk index), undone by the
// matrix-core fragment reads:
//   K-major slab  [rows][BK]   : chunk c of row r sits at chunk c ^ ((r >> 1) & 7)        (BK = 64, 128-byte rows)
//                                                       or c ^ ((r >> 2) & 3)              (BK = 32,  64-byte rows)
//   MN-major slab [BK][rows]   : chunk c of contraction row kk sits at chunk c ^ ((kk & 3) << 2)
// so that the 16 rows of a 128-bit fragment read, and the 4 rows of a transposing 64-bit read, fall into different
// bank groups.
#pragma once
#include "rd_common.h"

namespace rd {

// B_AUX: cache policy of the B operand's loads (0 = default, kCachePolicyStream = read once, do not keep in L2).
template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, bool A_KMAJOR_, bool B_KMAJOR_, int STAGES_,
          bool PINGPONG_ = false, int B_AUX_ = 0, bool HALF_ = false>
struct DldsCfg {
  typedef bf16_bits Elem;  // 16 bits per element: bf16, or float16 with HALF (same data movement, another instruction)
  static constexpr bool F32 = false, HALF = HALF_;
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, STAGES = STAGES_;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, VEC = true, DLDS = true, PINGPONG = PINGPONG_, MIXED = false,
                        SPLITK = true;
  static constexpr int B_AUX = B_AUX_;
  static constexpr int NW = WAVES_M * WAVES_N;
  static constexpr int NT = 64 * NW;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int KSTEPS = BK / 16;
  // Tiles whose accumulators take <= 64 registers leave room for a second (third) work-group on the CU, which hides
  // the fill and drain of short K loops; tell the register allocator so.
  static constexpr int TARGET_WGS = (TM * TN * 16 <= 64) ? (NW >= 8 ? 2 : 3) : 1;
  static constexpr int WAVES_PER_EU = (NW / 4) * TARGET_WGS;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  // The epilogue re-uses LDS to turn accumulators into row-contiguous 16-byte stores: one [WM][WN] bf16 patch per
  // wave, rows padded by 16 bytes.
  static constexpr int EPI_PITCH = WN * 2 + 16;
  static constexpr int EPI_BYTES = NW * WM * EPI_PITCH;
  static constexpr int RING_BYTES = STAGES * STAGE_BYTES;
  static constexpr int LDS_BYTES = RING_BYTES > EPI_BYTES ? RING_BYTES : EPI_BYTES;
  static_assert(BK == 64 || BK == 32, "contraction slab");
  // an MN-major slab row holds the operand's whole tile extent and its chunk permutation needs 16 chunks (128 elements)
  static_assert((A_KMAJOR ? BM % 64 == 0 : BM % 128 == 0) && BN % 128 == 0, "direct-to-LDS tile extents");
  static_assert(BM % (32 * WAVES_M) == 0 && BN % (32 * WAVES_N) == 0, "tile shape");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
  static_assert(!PINGPONG || (NW == 8 && WAVES_M == 2 && STAGES >= 3), "ping-pong runs two groups of four waves");
};

typedef __attribute__((address_space(3))) void* lds_void_ptr;

constexpr int kBufferFlags = 0x00020000;   // raw buffer, 32-bit data format
constexpr int kOobOffset = 0x7ffffff0;     // byte offset past any buffer: the load returns zeros
constexpr int kCachePolicyStream = 2;      // nt in the aux operand of the buffer intrinsics: streamed data, first to be evicted

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is 6 bits");
  __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

// One operand's slab loader: which 16 bytes each lane fetches for each of its wave's load instructions.
template <int T, int BK, int NW, bool KMAJOR, int AUX = 0>
struct DldsLoader {
  static constexpr int ROW_BYTES = KMAJOR ? BK * 2 : T * 2;
  static constexpr int RPI = 1024 / ROW_BYTES;   // slab rows per wave-wide load
  static constexpr int CPR = ROW_BYTES / 16;     // 16-byte chunks per slab row
  static constexpr int ROWS = KMAJOR ? T : BK;
  static constexpr int INSTR = ROWS / RPI;       // wave-wide loads per slab
  static constexpr int PER = INSTR / NW;         // of which each wave issues
  static_assert(INSTR % NW == 0 && PER >= 1, "slab does not split evenly over the waves");
  static_assert(!KMAJOR || (NW * RPI) % 16 == 0, "the chunk permutation must repeat from one load slot to the next");

  const bf16_bits* base;  // advances with the K loop
  int records;            // bytes still addressable from base
  int step_bytes;         // K-step advance of base in bytes
  int voff[PER];          // per-lane byte offset of each load
  int kcol;               // K-major: contraction offset (elements) of this lane's chunk, for the tail predicate

  // (init and advance are plain integer arithmetic and also run on the host: tests/host_checks/loader_bounds.hip walks
  // every load of every slab through them and checks it against the operand's window)
  __host__ __device__ __forceinline__ void init(const bf16_bits* p, int ld, int lim, int klen, int wave, int lane) {
    base = p;
    if (KMAJOR) {
      records = ((lim - 1) * ld + klen) * 2;
      step_bytes = BK * 2;
    } else {
      records = ((klen - 1) * ld + lim) * 2;
      step_bytes = BK * ld * 2;
    }
    kcol = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int t = wave + NW * j;
      const int r = t * RPI + lane / CPR;
      const int pchunk = lane % CPR;
      if (KMAJOR) {
        const int c = pchunk ^ (BK == 64 ? ((r >> 1) & 7) : ((r >> 2) & 3));
        voff[j] = r < lim ? (r * ld + c * 8) * 2 : kOobOffset;  // rows past the tile's limit: no memory access, zeros
        kcol = c * 8;  // identical for every j: r advances by a multiple of 16 rows per instruction slot
      } else {
        const int c = pchunk ^ ((r & 3) << 2);
        voff[j] = c * 8 < lim ? (r * ld + c * 8) * 2 : kOobOffset;
      }
    }
  }

  __device__ __forceinline__ __amdgpu_buffer_rsrc_t resource() const {
    return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, __builtin_amdgcn_readfirstlane(records), kBufferFlags);
  }

  // Issue load j of this wave for the current slab into `lds` (byte address of the operand's region in one stage).
  // TAIL: the slab runs past the contraction length.
  template <bool TAIL>
  __device__ __forceinline__ void issue(__amdgpu_buffer_rsrc_t rsrc, unsigned char* lds, int wave, int j, int k0,
                                        int klen) const {
    int off = voff[j];
    if (TAIL && KMAJOR && k0 + kcol >= klen) off = kOobOffset;  // MN-major tails are out of `records` by themselves
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)(lds + (wave + NW * j) * 1024), 16, off, 0, 0, AUX);
  }

  __host__ __device__ __forceinline__ void advance() {
    base = reinterpret_cast<const bf16_bits*>(reinterpret_cast<const unsigned char*>(base) + step_bytes);
    records -= step_bytes;  // stays positive for every slab that is issued
  }
};

// Per-lane LDS byte offsets for the matrix-core fragment reads of one operand.
template <int T, int BK, int TILES, bool KMAJOR>
struct DldsFragReader {
  static constexpr int ROW_BYTES = KMAJOR ? BK * 2 : T * 2;
  static constexpr int KSTEPS = BK / 16;
  static constexpr int NADDR = KMAJOR ? KSTEPS : TILES;
  int addr[NADDR];

  __device__ __forceinline__ void init(int wave_idx0, int lane) {
    if (KMAJOR) {
      const int r = lane & 31;
      const int sw = BK == 64 ? ((r >> 1) & 7) : ((r >> 2) & 3);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        addr[ks] = (wave_idx0 + r) * ROW_BYTES + (((ks * 2 + (lane >> 5)) ^ sw) << 4);
    } else {
      const int q = lane >> 4, i = lane & 15;
      const int row = 8 * (q >> 1) + (i >> 2);
      const int s = (i >> 2) & 3;
      const int low = 2 * (q & 1) + ((i & 3) >> 1);
#pragma unroll
      for (int j = 0; j < TILES; ++j) {
        const int tile = (wave_idx0 >> 5) + j;
        addr[j] = row * ROW_BYTES + ((4 * (tile ^ s) + low) << 4) + (i & 1) * 8;
      }
    }
  }

  __device__ __forceinline__ bf16x8_t read(const unsigned char* region, int tile, int ks) const {
    if (KMAJOR) {
      return *reinterpret_cast<const bf16x8_t*>(region + addr[ks] + tile * 32 * ROW_BYTES);
    } else {
      typedef __attribute__((address_space(3))) s16x4_t* lds_v4_ptr;
      const unsigned char* p = region + addr[tile] + ks * 16 * ROW_BYTES;
      s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_ptr)(p));
      s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_ptr)(p + 4 * ROW_BYTES));
      s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8_t, v);
    }
  }
};

// One tile's contraction range cut into `parts` pieces that different work-groups compute.  Every piece drops its fp32
// accumulators into its slot of `partials` and bumps the tile's arrival counter; the piece that arrives last sums all
// pieces and is the one that stores the tile.  No work-group ever waits for another.
struct SplitK {
  float* partials = nullptr;    // [parts][NT * accumulators per thread] of this tile
  int32_t* counter = nullptr;   // arrivals so far; zero when the launch starts
  int parts = 1, part = 0;
};

// Returns true when the caller holds the complete sums and must store them.  All threads of the work-group call it,
// after the last barrier of the K loop (it uses the first bytes of LDS to broadcast the arrival index).
//
// The pieces of a tile run on different XCDs, whose L2 caches do not see each other's lines.  A device-scope fence would
// make them agree by writing back and invalidating a whole L2 - tens of microseconds each, one after the other, for
// every piece - so the partial sums go around the problem instead: they are stored and loaded with the sc1 cache policy
// (coherent at device scope: written through, re-fetched), and the only ordering needed is that a piece's stores have
// completed before its arrival is counted.
constexpr int kCachePolicyDevice = 16;  // sc1 in the aux operand of the buffer intrinsics

template <class C>
__device__ __forceinline__ bool splitk_combine(f32x16_t (&acc)[C::TM][C::TN], const SplitK& sk, int tid,
                                               unsigned char* smem) {
  if (sk.parts <= 1) return true;
  constexpr int QUADS = C::TM * C::TN * 4;             // 16-byte vectors per thread
  constexpr int PIECE_BYTES = QUADS * C::NT * 16;      // one piece's accumulators
  __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)sk.partials, 0, sk.parts * PIECE_BYTES, kBufferFlags);
  const int lane_off = tid * 16;
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        // whole-vector casts only: a bit cast of a single vector element reads element 0 whatever the index
        f32x4_t q;
        q[0] = acc[i][j][4 * g + 0]; q[1] = acc[i][j][4 * g + 1]; q[2] = acc[i][j][4 * g + 2]; q[3] = acc[i][j][4 * g + 3];
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, q), rsrc, lane_off + ((i * C::TN + j) * 4 + g) * (C::NT * 16),
                                                   sk.part * PIECE_BYTES, kCachePolicyDevice);
      }
  wait_vmcnt<0>();   // this thread's stores have completed (a work-group-scope fence would not wait for them)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();   // ... and every thread's
  int32_t* slot = reinterpret_cast<int32_t*>(smem);
  if (tid == 0) *slot = __hip_atomic_fetch_add(sk.counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const int arrived = *slot;
  __syncthreads();  // everyone has read the slot before the epilogue reuses LDS
  if (arrived != sk.parts - 1) return false;
  // Sum the pieces in index order, this work-group's own included, so that the result does not depend on which piece
  // happened to arrive last.
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  for (int s = 0; s < sk.parts; ++s) {
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32x4_t raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off + ((i * C::TN + j) * 4 + g) * (C::NT * 16),
                                                                        s * PIECE_BYTES, kCachePolicyDevice);
          const f32x4_t v = __builtin_bit_cast(f32x4_t, raw);
          acc[i][j][4 * g + 0] += v[0]; acc[i][j][4 * g + 1] += v[1]; acc[i][j][4 * g + 2] += v[2]; acc[i][j][4 * g + 3] += v[3];
        }
  }
  return true;
}

// Epilogue shared by the direct-to-LDS cores.  The matrix-core calls pass the B fragment as first operand, so the
// accumulators hold transposed 32x32 blocks: register v of lane l is C[l & 31][8*(v>>2) + 4*(l>>5) + (v&3)], i.e. four
// consecutive columns of one row per register quad.  Each wave drops its [WM][WN] patch into its own LDS area as bf16
// (8-byte writes), then streams it out with 16-byte loads/stores that cover whole 128-byte lines of the output rows.
// Only the wave itself touches its area, so no work-group barrier is needed in between.  The stores are nontemporal:
// nothing in the launch reads the output, and kept out of L2 it leaves the operand slabs there (measured 2-3 % on
// every product of a memory-bound shape, nothing on a matrix-core-bound one).
template <class C>
__device__ __forceinline__ void store_accumulators(const f32x16_t (&acc)[C::TM][C::TN], int wm, int wn, int wave,
                                                   int lane, int a_lim, int b_lim, bf16_bits* __restrict__ Op, int ldo,
                                                   unsigned char* smem) {
  unsigned char* st = smem + wave * (C::WM * C::EPI_PITCH);
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int row = i * 32 + (lane & 31);
        const int col = j * 32 + 8 * g + 4 * (lane >> 5);
        u32x2_t w;
        w[0] = pack_out_x2<C::HALF>(acc[i][j][4 * g + 0], acc[i][j][4 * g + 1]);
        w[1] = pack_out_x2<C::HALF>(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
        *reinterpret_cast<u32x2_t*>(st + row * C::EPI_PITCH + col * 2) = w;
      }
  constexpr int CPR = C::WN / 8;        // 16-byte chunks per patch row
  constexpr int ROWS_PER = 64 / CPR;    // patch rows per wave-wide store
  const int chunk = lane % CPR, r0 = lane / CPR;
  const int gcol = wn * C::WN + chunk * 8;
  // The tile's output window through a buffer resource: a row or column past the tile's limits gets an offset beyond
  // it and the hardware drops the store.  No branches, so the LDS reads run ahead of the stores (with a branch around
  // each store the compiler kept its LDS read inside and waited for it there: 32 round trips, one after the other -
  // 5.5 us per tile).  The window stays below 2 GiB (checked on the host with the operands' windows).
  const long long window = ((long long)(a_lim - 1) * ldo + b_lim) * 2;
  __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)Op, 0, __builtin_amdgcn_readfirstlane(window <= 0 ? 0 : (window < kOobOffset ? (int)window : kOobOffset)), kBufferFlags);
  const bool col_live = gcol < b_lim;
  constexpr int NIT = C::WM / ROWS_PER;       // wave-wide stores per patch
  constexpr int BATCH = NIT < 8 ? NIT : 8;    // LDS reads in flight ahead of their stores
  static_assert(NIT % BATCH == 0, "whole batches");
#pragma unroll
  for (int t0 = 0; t0 < NIT; t0 += BATCH) {
    u32x4_t v[BATCH];
#pragma unroll
    for (int b = 0; b < BATCH; ++b)
      v[b] = *reinterpret_cast<const u32x4_t*>(st + ((t0 + b) * ROWS_PER + r0) * C::EPI_PITCH + chunk * 16);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int grow = wm * C::WM + (t0 + b) * ROWS_PER + r0;
      const int off = (grow < a_lim && col_live) ? (grow * ldo + gcol) * 2 : kOobOffset;
      __builtin_amdgcn_raw_buffer_store_b128(v[b], orsrc, off, 0, kCachePolicyStream);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <class C>
__device__ __forceinline__ void gemm_tile_dlds(const bf16_bits* __restrict__ Ap, int lda, int a_lim,
                                               const bf16_bits* __restrict__ Bp, int ldb, int b_lim, int klen,
                                               bf16_bits* __restrict__ Op, int ldo, bf16_bits* smem_,
                                               const SplitK& sk = SplitK()) {
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;

  typedef DldsLoader<C::BM, C::BK, C::NW, C::A_KMAJOR> LdA;
  typedef DldsLoader<C::BN, C::BK, C::NW, C::B_KMAJOR, C::B_AUX> LdB;
  LdA la; LdB lb;
  la.init(Ap, lda, a_lim, klen, wave, lane);
  lb.init(Bp, ldb, b_lim, klen, wave, lane);
  DldsFragReader<C::BM, C::BK, C::TM, C::A_KMAJOR> fra;
  DldsFragReader<C::BN, C::BK, C::TN, C::B_KMAJOR> frb;
  fra.init(wm * C::WM, lane);
  frb.init(wn * C::WN, lane);
  // A group's last tile (and most tiles of a short group) has few valid rows: a wave whose whole patch lies past the
  // tile's limits skips its matrix-core work.
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

  // Loads [first, first + count) of slab `step` (the A loads come first in the numbering, then the B loads).
  auto issue_loads = [&](int step, int first, int count) {
    unsigned char* st = smem + (step % C::STAGES) * C::STAGE_BYTES;
    const int k0 = step * C::BK;
    const bool tail = k0 + C::BK > klen;
    __amdgpu_buffer_rsrc_t ra_ = la.resource(), rb_ = lb.resource();
#pragma unroll
    for (int q = first; q < first + count; ++q) {
      if (q < LdA::PER) {
        if (tail) la.template issue<true>(ra_, st, wave, q, k0, klen);
        else la.template issue<false>(ra_, st, wave, q, k0, klen);
      } else {
        if (tail) lb.template issue<true>(rb_, st + C::A_BYTES, wave, q - LdA::PER, k0, klen);
        else lb.template issue<false>(rb_, st + C::A_BYTES, wave, q - LdA::PER, k0, klen);
      }
    }
  };

  // prologue: STAGES-1 slabs in flight
#pragma unroll
  for (int s = 0; s < C::STAGES - 1; ++s)
    if (s < nk) { issue_loads(s, 0, L); la.advance(); lb.advance(); }

  for (int kt = 0; kt < nk; ++kt) {
    // Slab kt must have landed; the STAGES-2 younger ones may still be in flight.  Near the end fewer loads were
    // issued after slab kt than that, so wait for everything.
    if (kt + C::STAGES - 2 < nk) wait_vmcnt<(C::STAGES - 2) * L>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();  // every wave's part of slab kt is in LDS, and slab kt-1 is no longer being read
    const bool more = kt + C::STAGES - 1 < nk;

    const unsigned char* ra = smem + (kt % C::STAGES) * C::STAGE_BYTES;
    const unsigned char* rb = ra + C::A_BYTES;
    // Fragments for K-substep ks+1 are fetched from LDS while the matrix core works on substep ks, and the loads of
    // the slab STAGES-1 steps ahead are issued a few at a time between the substeps: the memory pipeline then works
    // through them in the shadow of the matrix-core instructions instead of stalling every wave at once.
    bf16x8_t fa[2][C::TM], fb[2][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i) fa[0][i] = fra.read(ra, i, 0);
#pragma unroll
    for (int j = 0; j < C::TN; ++j) fb[0][j] = frb.read(rb, j, 0);
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < C::KSTEPS) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) fa[nxt][i] = fra.read(ra, i, ks + 1);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) fb[nxt][j] = frb.read(rb, j, ks + 1);
      }
      if (more) {
        constexpr int lo = 0;
        const int first = (L * ks) / C::KSTEPS, last = (L * (ks + 1)) / C::KSTEPS;
        (void)lo;
        issue_loads(kt + C::STAGES - 1, first, last - first);
      }
      // Keep the compiler from sinking those reads and loads below the matrix-core work they are meant to overlap.
      __builtin_amdgcn_sched_barrier(0);
      if (patch_live) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
          for (int j = 0; j < C::TN; ++j)
            acc[i][j] = mfma_32x32x16<C::HALF>(fb[cur][j], fa[cur][i], acc[i][j]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) { la.advance(); lb.advance(); }
  }

  __builtin_amdgcn_s_barrier();  // the ring is no longer read by any wave
  if (!splitk_combine<C>(acc, sk, tid, smem)) return;
  store_accumulators<C>(acc, wm, wn, wave, lane, a_lim, b_lim, Op, ldo, smem);
}

// Ping-pong schedule.  The eight waves form two groups of four (one wave of each group per SIMD).  A wave alternates
// between a memory phase (LDS -> registers for one K-slab, plus issuing its share of the direct loads of a later slab)
// and a compute phase (nothing but matrix-core instructions on registers).  The groups run half a period apart, so on
// every SIMD one wave always has a full phase of matrix-core work while the other hides all LDS and HBM latency.
// Work-group barriers separate the phases; the second group passes one extra barrier up front, the first one at the end.
template <class C>
__device__ __forceinline__ void gemm_tile_pingpong(const bf16_bits* __restrict__ Ap, int lda, int a_lim,
                                                   const bf16_bits* __restrict__ Bp, int ldb, int b_lim, int klen,
                                                   bf16_bits* __restrict__ Op, int ldo, bf16_bits* smem_,
                                               const SplitK& sk = SplitK()) {
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;  // wm is also the group index
  const int group = wave >> 2;

  typedef DldsLoader<C::BM, C::BK, C::NW, C::A_KMAJOR> LdA;
  typedef DldsLoader<C::BN, C::BK, C::NW, C::B_KMAJOR> LdB;
  LdA la; LdB lb;
  la.init(Ap, lda, a_lim, klen, wave, lane);
  lb.init(Bp, ldb, b_lim, klen, wave, lane);
  DldsFragReader<C::BM, C::BK, C::TM, C::A_KMAJOR> fra;
  DldsFragReader<C::BN, C::BK, C::TN, C::B_KMAJOR> frb;
  fra.init(wm * C::WM, lane);
  frb.init(wn * C::WN, lane);
  // A group's last tile (and most tiles of a short group) has few valid rows: a wave whose whole patch lies past the
  // tile's limits skips its matrix-core work.
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
    const int k0 = step * C::BK;
    const bool tail = k0 + C::BK > klen;
    __amdgpu_buffer_rsrc_t ra_ = la.resource(), rb_ = lb.resource();
#pragma unroll
    for (int q = 0; q < LdA::PER; ++q) {
      if (tail) la.template issue<true>(ra_, st, wave, q, k0, klen);
      else la.template issue<false>(ra_, st, wave, q, k0, klen);
    }
#pragma unroll
    for (int q = 0; q < LdB::PER; ++q) {
      if (tail) lb.template issue<true>(rb_, st + C::A_BYTES, wave, q, k0, klen);
      else lb.template issue<false>(rb_, st + C::A_BYTES, wave, q, k0, klen);
    }
    la.advance();
    lb.advance();
  };

#pragma unroll
  for (int s = 0; s < C::STAGES - 1; ++s)
    if (s < nk) issue_slab(s);
  // slab 0 of every wave must be in LDS before the first memory phase reads it
  if (C::STAGES - 1 <= nk) wait_vmcnt<(C::STAGES - 2) * L>(); else wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  if (group == 1) __builtin_amdgcn_s_barrier();

  for (int kt = 0; kt < nk; ++kt) {
    // ---- memory phase -------------------------------------------------------------------------------------------
    const unsigned char* ra = smem + (kt % C::STAGES) * C::STAGE_BYTES;
    const unsigned char* rb = ra + C::A_BYTES;
    bf16x8_t fa[C::KSTEPS][C::TM], fb[C::KSTEPS][C::TN];
    if (patch_live) {  // a wave without matrix-core work leaves the LDS bandwidth, which paces the loop, to the others
#pragma unroll
      for (int ks = 0; ks < C::KSTEPS; ++ks) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) fa[ks][i] = fra.read(ra, i, ks);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) fb[ks][j] = frb.read(rb, j, ks);
      }
    }
    // The slot of slab kt-1 is free: both groups finished reading it before the barrier that opened this phase.
    if (kt + C::STAGES - 1 < nk) issue_slab(kt + C::STAGES - 1);
    // Before leaving: this wave's share of slab kt+1 has landed (the other group may read it in the very next
    // interval) and the fragment reads above have returned (the slot they came from may be overwritten next).
    if (kt + C::STAGES - 1 < nk) wait_vmcnt<(C::STAGES - 2) * L>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // ---- compute phase ------------------------------------------------------------------------------------------
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
  }
  if (group == 0) __builtin_amdgcn_s_barrier();

  if (!splitk_combine<C>(acc, sk, tid, smem)) return;
  store_accumulators<C>(acc, wm, wn, wave, lane, a_lim, b_lim, Op, ldo, smem);
}

}  // namespace rd
