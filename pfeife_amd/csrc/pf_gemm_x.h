// The direct-to-LDS 16-bit MFMA kernel and its launchers.  Included by one translation unit per
// operand dtype and tile shape (the instantiations take minutes to compile; separate units build in parallel).
#pragma once
#include "pf_gemm_common.h"

namespace {

// ---------------------------------------------------------------------------
// 16-bit MFMA kernel, direct-to-LDS pipeline (the throughput path)
//
// Operand tiles go from global memory straight into LDS (buffer_load_dwordx4 ... lds:
// no staging registers, no LDS store instructions), ST tiles deep.  One such
// instruction fills 1024 consecutive LDS bytes, lane l supplying the 16-byte chunk at
// position l, but every lane fetches from an address of its own: the chunk order inside
// LDS is therefore free, and it is chosen (XOR swizzle) so that the MFMA fragment reads
// are bank-conflict free without padding:
//   reduction-contiguous operand  [row][k]: chunk c of a row sits at c ^ f(row), fragments
//                                           are single ds_read_b128;
//   reduction-strided operand     [k][row]: kept in that order (8-row chunk c of k-row k at
//                                           c ^ 4*(k%4)) and read with ds_read_b64_tr_b16,
//                                           the transposing LDS read, which hands a lane
//                                           four consecutive k of one row.
// Each wavefront owns a (BM/WGM) x (BN/WGN) block of accumulators (up to 128x128 =
// 16 MFMA tiles, one fragment read per two MFMAs).  The K loop has ONE barrier per tile,
// placed before the tile's last 16-deep MFMA group: by then the group's fragments are in
// registers, so the buffer can be refilled at once, and the first fragments of the next
// tile are read under that last group's MFMAs (no LDS latency exposed at the barrier).
// ---------------------------------------------------------------------------
#define PF_LDS(T) __attribute__((address_space(3))) T*
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

typedef short short8_t __attribute__((ext_vector_type(8)));
// MFMA operand fragment as it comes out of LDS: one 16-byte read, or (transposing reads) two
// 8-byte halves that are only joined where the MFMA consumes them, so that nothing in the
// group that issues the reads depends on their data
template <bool TRANS> struct Frag;
template <> struct Frag<false> {
  short8_t v;
  __device__ __forceinline__ short8_t get() const { return v; }
};
template <> struct Frag<true> {
  short4_t lo, hi;
  __device__ __forceinline__ short8_t get() const { return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7); }
};
// Keeps the registers of a fragment that inline assembly reads into allocated to it up to this
// point of the program: the compiler takes the output of such a read for complete where the read
// is issued, and once the value is dead it is free to put something else into the register, which
// the read, arriving later, would then overwrite.
__device__ __forceinline__ void frag_hold(Frag<false>&) {}
__device__ __forceinline__ void frag_hold(Frag<true>& f) { asm volatile("" : "+v"(f.lo), "+v"(f.hi)); }
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int R, int BK, int NW, bool TRANS> struct DTile {
  static constexpr int BYTES = R * BK * 2;
  static constexpr int NI = BYTES / 1024;  // wavefront-wide load instructions per tile
  static constexpr int IPW = NI / NW;      // ... per wavefront
  static_assert(NI % NW == 0 && IPW >= 1, "tile does not divide over the wavefronts");
  static constexpr int CPR = BK / 8;       // [row][k]: 16-byte chunks per row
  static constexpr int RPI = 64 / CPR;     //           rows per instruction
  static constexpr int ROWB = TRANS ? R * 2 : BK * 2;  // bytes per LDS row
  static constexpr int CPK = R / 8;        // [k][row]: chunks per k-row
  static constexpr int KPI = 64 / CPK;     //           k-rows per instruction
  static_assert(!TRANS || (R == 128 || R == 256), "transposed tiles are 128 or 256 rows wide");
  static_assert(BK == 64 || BK == 32, "BK is 32 or 64");
  static constexpr int NFRAG = TRANS ? 0 : BK / 16;

  static __device__ __forceinline__ int swz_row(int row) { return BK == 64 ? ((row >> 1) & 7) : ((row >> 2) & 3); }
  static __device__ __forceinline__ int swz_k(int k) { return (k & 3) << 2; }

  static __device__ __forceinline__ uint32_t extent(int64_t R_total, int64_t K, int64_t ld) {
    return TRANS ? (uint32_t)(((K - 1) * ld + (R_total + 7) / 8 * 8) * 2)
                 : (uint32_t)(((R_total - 1) * ld + (K + 7) / 8 * 8) * 2);
  }
  // byte offset (inside K-tile 0) of the chunk this lane fetches in its q-th instruction
  static __device__ __forceinline__ void init(uint32_t (&off)[IPW], int64_t ld, int64_t r0, int wave, int lane) {
#pragma unroll
    for (int q = 0; q < IPW; ++q) {
      const int ii = wave * IPW + q;
      if (!TRANS) {
        const int row = ii * RPI + lane / CPR;
        const int c = (lane % CPR) ^ swz_row(row);
        off[q] = (uint32_t)(((r0 + row) * ld + c * 8) * 2);
      } else {
        const int k = ii * KPI + lane / CPK;
        const int mc = (lane % CPK) ^ swz_k(k);
        off[q] = (uint32_t)((k * ld + r0 + mc * 8) * 2);
      }
    }
  }
  static __device__ __forceinline__ uint32_t tile_step(int64_t ld) { return TRANS ? (uint32_t)(BK * ld * 2) : (uint32_t)(BK * 2); }
  // lds: byte address of this operand's tile inside LDS (wave-uniform); issues the wavefront's
  // instructions Q0 <= q < Q1 (clipped to [0, IPW))
  template <int Q0, int Q1>
  static __device__ __forceinline__ void issue(__amdgpu_buffer_rsrc_t rs, const uint32_t (&off)[IPW], uint32_t adv,
                                               uint32_t lds, int wave) {
#pragma unroll
    for (int q = (Q0 < 0 ? 0 : Q0); q < (Q1 > IPW ? IPW : Q1); ++q)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (PF_LDS(void))(uintptr_t)(lds + (uint32_t)(wave * IPW + q) * 1024u), 16,
                                               (int)(off[q] + adv), 0, 0, 0);
  }
  // Fragment addressing.  w0: first row of the wavefront's block inside the tile.
  //   [row][k]: foff[kk] = byte offset of (row w0 + lane%32, chunk 2*kk + lane/32); + i*32*ROWB per MFMA tile
  //   [k][row]: foff[i]  = byte offset for MFMA tile i at kk = 0, first half; + (16*kk + 4*h)*ROWB
  static constexpr int NOFF_T = 4;
  // kk0: first 16-deep MFMA group of a tile that this wavefront multiplies (wavefronts that split
  // a tile's reduction depth between them start at different groups)
  template <int NF>
  static __device__ __forceinline__ void frag_init(uint32_t (&foff)[NF], int w0, int lane, int kk0) {
    if constexpr (!TRANS) {
      const int row = w0 + (lane & 31), half = lane >> 5;
#pragma unroll
      for (int kk = 0; kk < NF; ++kk) foff[kk] = (uint32_t)(row * ROWB + ((((kk0 + kk) * 2 + half) ^ swz_row(row)) * 16));
    } else {
      const int g = lane >> 4, j = lane & 15;
      const int k = (g >> 1) * 8 + (j >> 2);
#pragma unroll
      for (int i = 0; i < NF; ++i) {
        const int m = w0 + i * 32 + (g & 1) * 16 + 4 * (j & 3);
        foff[i] = (uint32_t)((k + kk0 * 16) * ROWB + (((m >> 3) ^ swz_k(k)) * 16) + (m & 7) * 2);
      }
    }
  }
  template <int NF, int I, int KKI>
  static __device__ __forceinline__ Frag<TRANS> frag(uint32_t lds, const uint32_t (&foff)[NF]) {
    Frag<TRANS> f;
    if constexpr (!TRANS) {
      f.v = *(PF_LDS(const short8_t))(uintptr_t)(lds + foff[KKI] + (uint32_t)(I * 32 * ROWB));
    } else {
      // Inline assembly on purpose: the compiler makes an LDS read it cannot tell apart from the
      // destination of an earlier direct-to-LDS load wait for ALL outstanding loads, and it cannot
      // for this instruction, which would serialise the whole tile pipeline.  The price: it does
      // not know that these results arrive asynchronously either; the K loop waits for them by
      // hand (TR_READS instructions per fragment count in lgkmcnt).
      const uint32_t a = lds + foff[I];
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f.lo) : "v"(a), "n"(KKI * 16 * ROWB) : "memory");
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f.hi) : "v"(a), "n"(KKI * 16 * ROWB + 4 * ROWB) : "memory");
    }
    return f;
  }
  static constexpr int TR_READS = 2;
};

// 32-row accumulator blocks each wavefront stages through LDS at a time in the epilogue
// (nw wavefronts, wn columns per wavefront block, tm blocks in all): as many as 160 KB hold.
constexpr int epi_row_blocks(int nw, int wn, int tm) {
  const int fit = (160 * 1024) / (nw * 32 * (wn + 8) * 4);
  int rb = fit >= tm ? tm : fit;
  while (rb > 1 && tm % rb != 0) --rb;
  return rb < 1 ? 1 : rb;
}

typedef float float8_t __attribute__((ext_vector_type(8)));

template <int DT> __device__ __forceinline__ float8_t unpack16(v4i_t r) {
  float8_t o;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t w = (uint32_t)r[k];
    if (DT == PF_BF16) {
      o[2 * k] = __uint_as_float(w << 16);
      o[2 * k + 1] = __uint_as_float(w & 0xffff0000u);
    } else {
      o[2 * k] = pf_f16_bits_to_f32((uint16_t)(w & 0xffffu));
      o[2 * k + 1] = pf_f16_bits_to_f32((uint16_t)(w >> 16));
    }
  }
  return o;
}
template <int DT> __device__ __forceinline__ v4i_t pack16(const float8_t& v) {
  v4i_t o;
#pragma unroll
  for (int k = 0; k < 4; ++k)
    o[k] = (int)(DT == PF_BF16 ? pf_pack2_bf16(v[2 * k], v[2 * k + 1]) : pf_pack2_f16(v[2 * k], v[2 * k + 1]));
  return o;
}

// `pid`: index of this workgroup among the workgroups of its problem (the launch may hold several
// problems, see gemm16x_group_kernel)
template <int DT, int BM, int BN, int BK, int WGM, int WGN, int KS, int ST, bool AT, bool BT, int EC>
__device__ __forceinline__ void gemm16x_body(const pf_gemm_desc& p, const GemmGrid& g, const int pid) {
  // KS = 2: the wavefronts form two WGM x WGN grids; grid h multiplies the h-th half of every
  // tile's 16-deep MFMA groups, and the two partial accumulator blocks are added through LDS
  // before the epilogue.  Eight wavefronts (two per SIMD, so that one's LDS reads and waits run
  // under the other's MFMAs) then read no more fragment bytes from LDS than four do, and the
  // LDS port (128 B/clk per CU for fragment reads and arriving tiles together) is what bounds
  // these tiles.
  constexpr int NWMN = WGM * WGN;
  constexpr int NW = NWMN * KS;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int KK = BK / 16 / KS;     // MFMA groups per tile and wavefront
  static_assert(KS == 1 || KS == 2, "the reduction depth of a tile is split over one or two wavefront grids");
  static_assert((BK / 16) % KS == 0, "MFMA groups do not divide over the wavefront grids");
  using TA = DTile<BM, BK, NW, AT>;
  using TB = DTile<BN, BK, NW, BT>;
  constexpr int STAGE = TA::BYTES + TB::BYTES;
  constexpr int LPW = TA::IPW + TB::IPW;  // load instructions per wavefront per tile
  static_assert((ST - 2) * LPW <= 63, "too many loads in flight for the 6-bit counter");
  static_assert(KK % 2 == 0, "fragment double buffer assumes an even number of MFMA groups per tile");
  constexpr int NFA = AT ? TM : KK, NFB = BT ? TN : KK;
  extern __shared__ __align__(16) uint16_t smem[];

  const int t = gemm_tile_id(pid, g.tiles_m * g.tiles_n, g.per_xcd);
  if (t < 0) return;
  int tm, tn;
  gemm_tile_rc(t, g.tiles_m, g.tiles_n, tm, tn);
  const int64_t M = p.M, N = p.N, K = p.K, lda = p.lda, ldb = p.ldb;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  const int64_t z = blockIdx.y, z1 = z / p.batch2, z2 = z % p.batch2;
  const uint16_t* A = (const uint16_t*)p.A + z1 * p.a_stride1 + z2 * p.a_stride2;
  const uint16_t* B = (const uint16_t*)p.B + z1 * p.b_stride1 + z2 * p.b_stride2;
  const int64_t c_base = z1 * p.c_stride1 + z2 * p.c_stride2;
  const Epi epi = make_epi(p);
  const int vec_epi = g.vec_epi;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_k = wave / NWMN, wave_mn = wave % NWMN;
  const int wm0 = (wave_mn / WGN) * WM, wn0 = (wave_mn % WGN) * WN;
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const __amdgpu_buffer_rsrc_t rs_a = make_rsrc(A, TA::extent(M, K, lda));
  const __amdgpu_buffer_rsrc_t rs_b = make_rsrc(B, TB::extent(N, K, ldb));
  uint32_t offa[TA::IPW], offb[TB::IPW];
  TA::init(offa, lda, m0, wave, lane);
  TB::init(offb, ldb, n0, wave, lane);
  const uint32_t step_a = TA::tile_step(lda), step_b = TB::tile_step(ldb);
  uint32_t foa[NFA], fob[NFB];
  TA::template frag_init<NFA>(foa, wm0, lane, wave_k * KK);
  TB::template frag_init<NFB>(fob, wn0, lane, wave_k * KK);

  const int nk = (int)((K + BK - 1) / BK);

  // fast epilogues: this lane's 8 bias values, fetched now so that the K loop hides the latency
  constexpr int LPR = WN / 8;        // epilogue: lanes per row of the wavefront's block
  constexpr int RPP = 64 / LPR;      //           rows per pass
  const int rd_row = lane / LPR, rd_col = (lane % LPR) * 8;
  const int64_t c8 = n0 + wn0 + rd_col;
  float8_t bias8 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if constexpr (EC != EC_GENERIC) {
    if (epi.bias != nullptr && c8 < N) {
      float t[8];
      ld_vec<8>(epi.bias, c8, epi.bias_dtype, t);
#pragma unroll
      for (int k = 0; k < 8; ++k) bias8[k] = t[k];
    }
  }

  // Tiles past the end of K are requested too: their addresses lie beyond the buffer
  // extent, so the hardware range check drops them, and every iteration of the K loop
  // is the same straight-line code with the same number of loads in flight.
  // The loads of one tile are issued in KK-1 slices, one per MFMA group: a burst of them
  // would fill the memory pipeline's queue and stall the wavefront (and with it the SIMD's
  // MFMA pipe, there is one wavefront per SIMD) for as long as the tile takes to stream in.
  static_assert(ST >= 3, "the refill of a stage is spread over the following tile's MFMA groups");
  constexpr int NSL = KK - 1;                         // slices
  constexpr int SLW = (LPW + NSL - 1) / NSL;          // loads per slice
  auto issue_all = [&](int kt, uint32_t sb) {
    TA::template issue<0, TA::IPW>(rs_a, offa, (uint32_t)kt * step_a, sb, wave);
    TB::template issue<0, TB::IPW>(rs_b, offb, (uint32_t)kt * step_b, sb + TA::BYTES, wave);
  };
  // One 16-deep MFMA group ("phase") = NMFMA matrix instructions on the fragments in register
  // set kk&1, the LDS reads that fill the other set for the next phase, and (all phases but a
  // tile's last) one slice of the loads that refill the stage freed by the previous tile.  The
  // three kinds are dealt round-robin into G sub-groups fenced by scheduling barriers, so the
  // single wavefront of a SIMD always has matrix work queued while its LDS reads and its
  // load instructions (which wait for room in the memory pipeline) trickle out.
  constexpr int NFRAG = TM + TN;
  constexpr int NMFMA = TM * TN;
  constexpr int G = NFRAG < NMFMA ? NFRAG : NMFMA;
  Frag<AT> fa[2][TM];
  Frag<BT> fb[2][TN];
  // kkn: MFMA group whose fragments are read (from stage sbr) into register set `slot`;
  // kk: MFMA group multiplied now; SL: slice of tile loads issued now (-1: none)
  auto phase = [&](uint32_t sbr, auto kknc, auto kkc, auto slc, int ktl, uint32_t sbl) {
    constexpr int kkn = decltype(kknc)::value, kk = decltype(kkc)::value, SL = decltype(slc)::value;
    constexpr int slot = kkn & 1, cur = kk & 1;
    static_for<G>([&](auto gc) {
      constexpr int gi = decltype(gc)::value;
      {
        static_for<NFRAG>([&](auto fc) {
          constexpr int f = decltype(fc)::value;
          if constexpr (f * G / NFRAG == gi) {
            if constexpr (f < TM) fa[slot][f] = TA::template frag<NFA, f, kkn>(sbr, foa);
            else fb[slot][f - TM] = TB::template frag<NFB, f - TM, kkn>(sbr + TA::BYTES, fob);
          }
        });
      }
      if constexpr (AT && BT && gi == 0) {
        // fragments of this phase's MFMAs were read (by inline assembly) during the previous
        // phase: LDS returns in order, so they are all there once no more reads are outstanding
        // than this group has just issued
        constexpr int mine = ((NFRAG + G - 1) / G) * 2;
        asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(mine) : "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (SL >= 0) {
        {
          static_for<SLW>([&](auto qc) {
            constexpr int q = SL * SLW + decltype(qc)::value;   // index into A's then B's list of loads
            if constexpr (decltype(qc)::value * G / SLW == gi && q < LPW) {
              if constexpr (q < TA::IPW) TA::template issue<q, q + 1>(rs_a, offa, (uint32_t)ktl * step_a, sbl, wave);
              else TB::template issue<q - TA::IPW, q - TA::IPW + 1>(rs_b, offb, (uint32_t)ktl * step_b, sbl + TA::BYTES, wave);
            }
          });
        }
      }
      // 256x128 shared by eight wavefronts: the wavefront that has MFMAs to issue goes first among
      // the two of its SIMD (measured -2 % on 4096-row products; no gain on the other tiles)
      constexpr bool PRIO = NW == 8 && KS == 1 && BM == 256 && BN == 128;
      if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
      static_for<NMFMA>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        if constexpr (m * G / NMFMA == gi) {
          constexpr int i = m / TN, j = m % TN;
          acc[i][j] = Mfma<DT>::run8(fa[cur][i].get(), fb[cur][j].get(), acc[i][j]);
        }
      });
      if constexpr (PRIO) __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // prologue: fill all stages but the last, wait for tile 0
#pragma unroll
  for (int s = 0; s < ST - 1; ++s) issue_all(s, lds0 + (uint32_t)s * STAGE);
  wait_vm<(ST - 2) * LPW>();
  lds_barrier();
  static_for<TM>([&](auto ic) { fa[0][decltype(ic)::value] = TA::template frag<NFA, decltype(ic)::value, 0>(lds0, foa); });
  static_for<TN>([&](auto jc) { fb[0][decltype(jc)::value] = TB::template frag<NFB, decltype(jc)::value, 0>(lds0 + TA::BYTES, fob); });
  __builtin_amdgcn_sched_barrier(0);

  uint32_t sb = lds0;                                   // stage of tile kt
  uint32_t sb_prev = lds0 + (uint32_t)(ST - 1) * STAGE; // stage of tile kt-1: free, refilled with tile kt+ST-1
  for (int kt = 0; kt < nk; ++kt) {
    const uint32_t sb_next = (sb + STAGE == lds0 + (uint32_t)ST * STAGE) ? lds0 : sb + STAGE;
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value;
      if constexpr (kk + 1 < KK) {
        phase(sb, std::integral_constant<int, kk + 1>{}, kkc, std::integral_constant<int, kk>{}, kt + ST - 1, sb_prev);
      } else {
        wait_vm<(ST - 2) * LPW>();
        lds_barrier();                              // tile kt+1 landed everywhere, stage sb no longer read
        phase(sb_next, std::integral_constant<int, 0>{}, kkc, std::integral_constant<int, -1>{}, 0, 0u);
      }
    });
    sb_prev = sb;
    sb = sb_next;
  }
  // The last tile's last phase has read fragments of a tile that does not exist, and nothing
  // consumes them: the reads issued by inline assembly may still be in flight here, and the
  // compiler, which knows nothing of that, would hand their registers to the epilogue's first
  // values (seen: the lane's row inside the block, overwritten with a fragment of zeros whenever
  // other kernels on the same compute unit delayed the LDS: every lane then took itself for a
  // lane of row 0 and 15 rows in 16 of the wavefront's block were never written).
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
  for (int sl = 0; sl < 2; ++sl) {
#pragma unroll
    for (int i = 0; i < TM; ++i) frag_hold(fa[sl][i]);
#pragma unroll
    for (int j = 0; j < TN; ++j) frag_hold(fb[sl][j]);
  }
  // (the dropped requests past K are counted too)  The builtin, not inline assembly: the compiler
  // tracks the LDS-writing loads itself and, unless it sees them retired here, makes every LDS
  // read of the epilogue wait for ALL vector memory operations, i.e. for the epilogue's own
  // stores to drain, once per row pass.
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)

  // Epilogue.  D layout of v_mfma_f32_32x32x*: lane l holds column (l % 32) and rows
  // 8*(r/4) + 4*(l/32) + (r%4), r = 0..15.  Each wavefront re-lays its block through a private
  // LDS patch (no workgroup barrier, no wait for earlier stores to drain), as many 32-row blocks
  // at a time as LDS holds; afterwards WN/8 adjacent lanes cover one whole row of the block, 8
  // columns each, so every store instruction writes complete rows of 2*WN (16-bit C) or 4*WN
  // (fp32 C) bytes.  The arithmetic exists ONCE, in a rolled loop over the staged rows: a kernel
  // of a few tens of microseconds cannot afford to stream 100 KB of unrolled epilogue code
  // through the instruction cache, which starts cold at every launch.
  lds_barrier();  // every wavefront is done with the operand tiles
  if constexpr (KS == 2) {
    // the second grid hands its partial sums over (16 bytes per lane, lanes side by side: no bank
    // conflicts) and leaves; a barrier only counts the wavefronts that are still running
    float4* xch = (float4*)smem + wave_mn * (TM * TN * 4 * 64) + lane;
    if (wave_k == 1) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            xch[((i * TN + j) * 4 + q) * 64] = make_float4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
    }
    lds_barrier();
    if (wave_k == 1) return;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 t = xch[((i * TN + j) * 4 + q) * 64];
          acc[i][j][4 * q] += t.x; acc[i][j][4 * q + 1] += t.y; acc[i][j][4 * q + 2] += t.z; acc[i][j][4 * q + 3] += t.w;
        }
    lds_barrier();  // all partial sums are read before the epilogue patches overwrite them
  }
  constexpr int SLD = WN + 8;        // floats per staged row: lanes 32..63 (4 rows down) land 32 banks away
  constexpr int RB = epi_row_blocks(NWMN, WN, TM);   // 32-row blocks staged together
  float* stage = (float*)smem + wave * (RB * 32 * SLD);
  const int wr_off = ((lane >> 5) * 4) * SLD + (lane & 31);

  if constexpr (EC != EC_GENERIC) {
    // Compact branch-free epilogue: 16 rows of the wavefront's block at a time, ONE copy of the
    // arithmetic in a rolled loop (unrolled, an epilogue runs to 200 KB of code that streams once
    // through an instruction cache which starts cold at every launch).
    // All global accesses are raw buffer operations whose range check drops rows past M (and
    // lanes past N, which get an out-of-range offset): no branch, so no join at which the
    // compiler would wait for every outstanding vector memory operation (loads AND the stores of
    // the previous pass share one in-order counter).  The one operand a class reads (residual,
    // old C or aux_in) comes in by direct-to-LDS loads, double buffered: the loads of the next 16
    // rows are issued before the stores of the current ones, and since the counter retires in
    // order, "those loads have landed" is "at most <the operations issued after them>
    // outstanding", a compile-time number because nothing here is predicated.
    constexpr bool C32 = EC == EC_STORE32 || EC == EC_RES32 || EC == EC_ACC32;
    constexpr bool LOADS = EC == EC_RES32 || EC == EC_ACC32 || EC == EC_DACT16 || EC == EC_ACC16 || EC == EC_RES16;
    constexpr bool LOAD32 = EC == EC_RES32 || EC == EC_ACC32;
    constexpr int HB = 16;                 // rows per step
    constexpr int NHB = TM * 2;            // steps
    constexpr int NP = HB / RPP;           // passes per step (a pass: every lane 8 columns of one row)
    constexpr int LPP = LOADS ? (LOAD32 ? 2 : 1) : 0;               // load instructions per pass
    constexpr int SPP = (C32 ? 2 : 1) + (EC == EC_ACT16 ? 1 : 0);   // store instructions per pass
    constexpr int ESC = C32 ? 4 : 2;
    constexpr int WAVE_LDS = HB * SLD * 4 + 2 * NP * 2 * 1024;      // stage + two operand buffers
    static_assert(NWMN * WAVE_LDS <= 160 * 1024, "epilogue patches exceed LDS");
    static_assert(NP * (SPP + LPP) <= 63, "too many operations in flight for the 6-bit counter");
    float* stg = (float*)((char*)smem + wave * WAVE_LDS);
    const uint32_t raw0 = lds0 + (uint32_t)(wave * WAVE_LDS + HB * SLD * 4);
    const uint32_t OOB = 0x80000000u;
    const int64_t row0 = m0 + wm0 + rd_row;
    const bool col_ok = c8 < N;
    const __amdgpu_buffer_rsrc_t rs_c = make_rsrc((const char*)epi.C + c_base * ESC, (uint32_t)(((M - 1) * epi.ldc + N) * ESC));
    const uint32_t off_c = col_ok ? (uint32_t)((row0 * epi.ldc + c8) * ESC) : OOB;
    const uint32_t step_c = (uint32_t)(epi.ldc * ESC);
    const void* lp = (EC == EC_RES32 || EC == EC_RES16) ? epi.residual
                                                            : (EC == EC_DACT16 ? epi.aux_in : (const void*)((const char*)epi.C + c_base * ESC));
    const int64_t ld_l = (EC == EC_RES32 || EC == EC_RES16) ? epi.ld_res : (EC == EC_DACT16 ? epi.ld_aux_in : epi.ldc);
    constexpr int ESL = LOAD32 ? 4 : 2;
    // (a product that stores, beta = 0, inside a launch of the accumulate class, i.e. one member of a
    // grouped weight-gradient launch, reads its old C through a descriptor of extent 0: all zeros)
    const bool loads_on = LOADS && !(EC == EC_ACC32 && epi.beta == 0);
    const __amdgpu_buffer_rsrc_t rs_l = make_rsrc(LOADS ? lp : epi.C, loads_on ? (uint32_t)(((M - 1) * ld_l + N) * ESL) : 0u);
    const uint32_t off_l = col_ok ? (uint32_t)((row0 * ld_l + c8) * ESL) : OOB;
    const uint32_t step_l = (uint32_t)(ld_l * ESL);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(EC == EC_ACT16 ? epi.aux_out : epi.C,
                                                  EC == EC_ACT16 ? (uint32_t)(((M - 1) * epi.ld_aux_out + N) * 2) : 0u);
    const uint32_t off_x = col_ok ? (uint32_t)((row0 * epi.ld_aux_out + c8) * 2) : OOB;
    const uint32_t step_x = (uint32_t)(epi.ld_aux_out * 2);
    const float alpha = epi.alpha;
    const bool round_mid = epi.round_mid != 0;

    auto fetch = [&](int hb) {   // rows past the block (hb == NHB) are requested too; nobody reads them
      if constexpr (LOADS) {
        const uint32_t dst = raw0 + (uint32_t)((hb & 1) * NP * LPP) * 1024u;
#pragma unroll
        for (int pp = 0; pp < NP; ++pp) {
          const uint32_t o = off_l + (uint32_t)(hb * HB + pp * RPP) * step_l;
#pragma unroll
          for (int h = 0; h < LPP; ++h)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_l, (PF_LDS(void))(uintptr_t)(dst + (uint32_t)(pp * LPP + h) * 1024u), 16,
                                                     (int)(o + 16 * h), 0, 0, 0);
        }
      }
    };
    float8_t csum = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};   // EC_DACT16: column sums of the stored values
    float worst = 0.f;   // fp32 classes: sum of v - v over the values written: 0 if all are finite, NaN otherwise
    fetch(0);
#pragma nounroll
    for (int hb = 0; hb < NHB; ++hb) {
      static_for<NHB>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        if (hb == c) {
          static_for<TN>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
#pragma unroll
            for (int r8 = 0; r8 < 8; ++r8)
              stg[wr_off + (8 * (r8 >> 2) + (r8 & 3)) * SLD + j * 32] = acc[c / 2][j][(c % 2) * 8 + r8];
          });
        }
      });
      if constexpr (LOADS) {
        fetch(hb + 1);
        if (hb == 0) wait_vm<NP * LPP>(); else wait_vm<NP * (SPP + LPP)>();
      }
      const uint32_t rawb = raw0 + (uint32_t)((hb & 1) * NP * LPP) * 1024u + (uint32_t)lane * 16u;
      const uint32_t stg_addr = lds0 + (uint32_t)(wave * WAVE_LDS + (rd_row * SLD + rd_col) * 4);
      // LDS reads by inline assembly: the compiler cannot tell these addresses from the
      // destinations of the direct-to-LDS loads in flight and would wait for all of them (and,
      // the counter being shared, for every store issued so far) before each ordinary read.
      // The reads of all passes of a step are issued together and waited for once: a rolled
      // pass loop exposed one LDS round trip per pass.
      v4i_t sxs[NP], sys[NP], ras[NP], rbs[NP];
#pragma unroll
      for (int pp = 0; pp < NP; ++pp) {
        const uint32_t sa = stg_addr + (uint32_t)((pp * RPP) * SLD * 4);
        asm volatile("ds_read_b128 %0, %1" : "=v"(sxs[pp]) : "v"(sa) : "memory");
        asm volatile("ds_read_b128 %0, %1 offset:16" : "=v"(sys[pp]) : "v"(sa) : "memory");
        if constexpr (LOADS) {
          const uint32_t rp = rawb + (uint32_t)(pp * LPP) * 1024u;
          asm volatile("ds_read_b128 %0, %1" : "=v"(ras[pp]) : "v"(rp) : "memory");
          if constexpr (LOAD32) asm volatile("ds_read_b128 %0, %1 offset:1024" : "=v"(rbs[pp]) : "v"(rp) : "memory");
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      // (the values are only complete from here on: nothing that uses them may move above the wait)
#pragma unroll
      for (int pp = 0; pp < NP; ++pp) {
        asm volatile("" : "+v"(sxs[pp]), "+v"(sys[pp]));
        if constexpr (LOADS) asm volatile("" : "+v"(ras[pp]));
        if constexpr (LOAD32) asm volatile("" : "+v"(rbs[pp]));
      }
#pragma unroll
      for (int pp = 0; pp < NP; ++pp) {
        const v4i_t sx = sxs[pp], sy = sys[pp], ra = ras[pp], rb = rbs[pp];
        float8_t v;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          v[k] = __int_as_float(sx[k]);
          v[4 + k] = __int_as_float(sy[k]);
        }
        v = v * alpha + bias8;
        // (the plain 16-bit store rounds once, when it packs: rounding to the same format before
        // that changes nothing and cost 16 of the pass's 30 vector instructions)
        if constexpr (EC != EC_STORE16) {
          if (round_mid) {
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = Codec<DT>::round(v[k]);
          }
        }
        const uint32_t rowk = (uint32_t)(hb * HB + pp * RPP);
        if constexpr (EC == EC_ACT16) {   // GELU only (other activations take the generic class)
          __builtin_amdgcn_raw_buffer_store_b128(pack16<DT>(v), rs_x, (int)(off_x + rowk * step_x), 0, 0);
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] = pf_gelu_erf(v[k]);
        }
        if constexpr (EC == EC_DACT16 || EC == EC_ACC16 || EC == EC_RES16) {
          const float8_t t = unpack16<DT>(ra);
          if constexpr (EC == EC_DACT16) {
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] *= pf_gelu_erf_grad(t[k]);
          } else {
            v += t;
          }
        }
        if constexpr (LOAD32) {
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            v[k] += __int_as_float(ra[k]);
            v[4 + k] += __int_as_float(rb[k]);
          }
        }
        const uint32_t oc = off_c + rowk * step_c;
        if constexpr (C32) {
          if constexpr (EC == EC_STORE32 || EC == EC_ACC32) {
#pragma unroll
            for (int k = 0; k < 8; ++k) worst += (row0 + (int64_t)rowk < M) ? (v[k] - v[k]) : 0.f;
          }
          v4i_t lo, hi;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            lo[k] = __float_as_int(v[k]);
            hi[k] = __float_as_int(v[4 + k]);
          }
          __builtin_amdgcn_raw_buffer_store_b128(lo, rs_c, (int)oc, 0, 0);
          __builtin_amdgcn_raw_buffer_store_b128(hi, rs_c, (int)(oc + 16), 0, 0);
        } else {
          const v4i_t packed = pack16<DT>(v);
          if constexpr (EC == EC_DACT16) {   // sums run over the ROUNDED values, rows past M excluded
            const float keep = (row0 + (int64_t)rowk < M) ? 1.f : 0.f;
            csum += unpack16<DT>(packed) * keep;
          }
          __builtin_amdgcn_raw_buffer_store_b128(packed, rs_c, (int)oc, 0, 0);
        }
      }
    }
    if constexpr (EC == EC_STORE32 || EC == EC_ACC32) {
      // every writer writes the same value: no atomic needed
      if (epi.nonfinite != nullptr && worst != 0.f) *epi.nonfinite = 1.f;
    }
    if constexpr (EC == EC_DACT16) {
      if (epi.colsum_ws != nullptr) {   // uniform over the grid
        // lanes l, l + LPR, l + 2 LPR, ... hold the same 8 columns (different rows)
#pragma unroll
        for (int off = LPR; off < 64; off <<= 1)
#pragma unroll
          for (int k = 0; k < 8; ++k) csum[k] += __shfl_xor(csum[k], off, 64);
        // wavefronts of one block column add up in wavefront-row order through LDS (every wavefront
        // is done with its own epilogue patch at the barrier; the patch of partial sums lies below
        // the first wavefront's operand buffers, which the last, unused prefetch may still be filling)
        float* red = (float*)smem;
        static_assert(NWMN * WN * 4 <= HB * SLD * 4, "partial column sums overlap the operand buffers");
        lds_barrier();
        if (lane < LPR) {
#pragma unroll
          for (int k = 0; k < 8; ++k) red[wave * WN + lane * 8 + k] = csum[k];
        }
        lds_barrier();
        if (wave / WGN == 0 && lane < LPR && c8 < N) {
          float t[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) t[k] = 0.f;
#pragma unroll
          for (int w = 0; w < WGM; ++w)
#pragma unroll
            for (int k = 0; k < 8; ++k) t[k] += red[(w * WGN + wave % WGN) * WN + lane * 8 + k];
          float* dst = epi.colsum_ws + (int64_t)tm * N + c8;
          *(float4*)dst = make_float4(t[0], t[1], t[2], t[3]);
          *(float4*)(dst + 4) = make_float4(t[4], t[5], t[6], t[7]);
        }
      }
    }
    return;
  }

#pragma nounroll
  for (int h = 0; h < TM / RB; ++h) {
    static_for<TM / RB>([&](auto hc) {
      constexpr int c = decltype(hc)::value;
      if (h == c) {
        static_for<RB>([&](auto ibc) {
          constexpr int ib = decltype(ibc)::value;
          static_for<TN>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
#pragma unroll
            for (int r = 0; r < 16; ++r)
              stage[ib * 32 * SLD + wr_off + (8 * (r >> 2) + (r & 3)) * SLD + j * 32] = acc[c * RB + ib][j][r];
          });
        });
      }
    });
#pragma nounroll
    for (int it = 0; it < RB * 32 / RPP; ++it) {
      const int rr = it * RPP + rd_row;
      const int64_t row = m0 + wm0 + h * (RB * 32) + rr;
      if (row >= M || c8 >= N) continue;
      const float4* src = (const float4*)(stage + rr * SLD + rd_col);
      const float4 x = src[0], y = src[1];
      float v[8] = {x.x, x.y, x.z, x.w, y.x, y.y, y.z, y.w};
      if (vec_epi && c8 + 8 <= N) {
        epilogue_vec8(epi, c_base, row, c8, v);
      } else {
#pragma nounroll
        for (int k = 0; k < 8; ++k)
          if (c8 + k < N) epilogue_scalar(epi, c_base, row, c8 + k, v[k]);
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
}

#define PF_X_BOUNDS __launch_bounds__(64 * WGM * WGN * KS, (ST * (BM + BN) * BK * 2 <= 80 * 1024 && 64 * WGM * WGN * KS <= 256) ? 2 : 1)
template <int DT, int BM, int BN, int BK, int WGM, int WGN, int KS, int ST, bool AT, bool BT, int EC>
__global__ PF_X_BOUNDS void gemm16x_kernel(const pf_gemm_desc p, const GemmGrid g) {
  gemm16x_body<DT, BM, BN, BK, WGM, WGN, KS, ST, AT, BT, EC>(p, g, (int)blockIdx.x);
}

// Several independent problems of the same kind in one launch: problem i owns the workgroups
// [start[i], start[i+1]).  Weight-gradient products are independent of everything that follows
// them in a backward job; small ones (64 tiles for a 1024x1024 weight) are launched together so
// that they fill the 256 CUs.
constexpr int GEMM_GROUP_MAX = PF_GEMM_GROUP_MAX;   // 8 problems: 2.3 KB of kernel arguments
struct GemmGroup {
  pf_gemm_desc p[GEMM_GROUP_MAX];
  GemmGrid g[GEMM_GROUP_MAX];
  int start[GEMM_GROUP_MAX];
  int n;
};
template <int DT, int BM, int BN, int BK, int WGM, int WGN, int KS, int ST, bool AT, bool BT, int EC>
__global__ PF_X_BOUNDS void gemm16x_group_kernel(const GemmGroup ga) {
  int i = 0;
#pragma unroll
  for (int k = 1; k < GEMM_GROUP_MAX; ++k)
    if (k < ga.n && (int)blockIdx.x >= ga.start[k]) i = k;
  i = __builtin_amdgcn_readfirstlane(i);
  gemm16x_body<DT, BM, BN, BK, WGM, WGN, KS, ST, AT, BT, EC>(ga.p[i], ga.g[i], (int)blockIdx.x - ga.start[i]);
}

template <int DT, int BM, int BN, int BK, int WGM, int WGN, int KS, int ST, bool AT, bool BT, int EC>
int launch16x_t(const pf_gemm_desc& d, const GemmGrid& g, hipStream_t st) {
  constexpr int NT = 64 * WGM * WGN * KS;
  constexpr size_t lds_xch = KS == 2 ? (size_t)BM * BN * 4 : 0;   // one grid's partial sums on their way to the other
  constexpr size_t lds_main = ((size_t)ST * (BM + BN) * BK * 2 > lds_xch) ? (size_t)ST * (BM + BN) * BK * 2 : lds_xch;
  constexpr size_t lds_gen = (size_t)(WGM * WGN) * epi_row_blocks(WGM * WGN, BN / WGN, BM / WGM / 32) * 32 * (BN / WGN + 8) * sizeof(float);
  constexpr size_t lds_fast = (size_t)(WGM * WGN) * (16 * (BN / WGN + 8) * 4 + 2 * (16 / (64 / (BN / WGN / 8))) * 2 * 1024);
  constexpr size_t lds_epi = EC == EC_GENERIC ? lds_gen : lds_fast;
  constexpr size_t lds = lds_main > lds_epi ? lds_main : lds_epi;
  static_assert(lds <= 160 * 1024, "tile pipeline exceeds the 160 KB of LDS");
  auto kern = gemm16x_kernel<DT, BM, BN, BK, WGM, WGN, KS, ST, AT, BT, EC>;
  if (lds > 64 * 1024) {  // opt in to the large LDS carve-out once per instantiation and device
    static std::mutex mu;
    static bool raised[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    std::lock_guard<std::mutex> lock(mu);
    if (!raised[dev]) {
      const hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) {
        pf_set_error("pf_gemm: cannot raise dynamic LDS to %zu bytes: %s", lds, hipGetErrorString(e));
        return PF_ERR_HIP;
      }
      raised[dev] = true;
    }
  }
  const dim3 grid((unsigned)(g.per_xcd * 8), (unsigned)(d.batch1 * d.batch2), 1);
  hipLaunchKernelGGL(kern, grid, dim3(NT), lds, st, d, g);
  PF_CHECK_LAUNCH("pf_gemm");
  return PF_OK;
}

template <int DT, int BM, int BN, int BK, int WGM, int WGN, int KS, int ST>
int launch16x(const pf_gemm_desc& d, hipStream_t st) {
  GemmGrid g;
  g.tiles_m = (int)((d.M + BM - 1) / BM);
  g.tiles_n = (int)((d.N + BN - 1) / BN);
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  g.per_xcd = (int)((total + 7) / 8);
  g.vec_epi = epi_vec_ok(d);
  // A ragged reduction tail is zero-filled by the hardware range check only when whole k-rows
  // fall outside the operand, i.e. when both operands are stored [k][row].
  if (d.K % BK != 0 && !(d.a_trans && d.b_trans)) {
    pf_set_error("pf_gemm: this variant needs K %% %d == 0 unless both operands are transposed", BK);
    return PF_ERR_INVALID;
  }
  const int ec = epi_class(d, g.vec_epi);
#define PF_X(AT, BT, EC) launch16x_t<DT, BM, BN, BK, WGM, WGN, KS, ST, AT, BT, EC>(d, g, st)
  if (!d.a_trans && !d.b_trans) {   // forward and input-gradient products
    switch (ec) {
      case EC_STORE16: return PF_X(false, false, EC_STORE16);
      case EC_STORE32: return PF_X(false, false, EC_STORE32);
      case EC_ACT16: return PF_X(false, false, EC_ACT16);
      case EC_RES32: return PF_X(false, false, EC_RES32);
      case EC_ACC32: return PF_X(false, false, EC_ACC32);
      case EC_DACT16: return PF_X(false, false, EC_DACT16);
      case EC_ACC16: return PF_X(false, false, EC_ACC16);
      case EC_RES16: return PF_X(false, false, EC_RES16);
      default: return PF_X(false, false, EC_GENERIC);
    }
  }
  // transposed (reduction-strided) tiles exist for 128 and 256 rows only
  if constexpr ((BM == 128 || BM == 256) && (BN == 128 || BN == 256)) {
    if (d.a_trans && d.b_trans) {   // weight-gradient products
      if (ec == EC_ACC32) return PF_X(true, true, EC_ACC32);
      if (ec == EC_STORE32) return PF_X(true, true, EC_STORE32);
      return PF_X(true, true, EC_GENERIC);
    }
  }
#undef PF_X
  pf_set_error("pf_gemm: tile %dx%d has no variant for a_trans=%d b_trans=%d", BM, BN, d.a_trans, d.b_trans);
  return PF_ERR_INVALID;
}

// Several weight-gradient products (both operands reduction-strided, fp32 C accumulated) in one
// launch; the caller has checked that they all take tile BMxBN and the EC_ACC32 epilogue.
template <int DT, int BM, int BN, int BK, int WGM, int WGN, int KS, int ST>
int launch16x_group(const pf_gemm_desc* d, int n, hipStream_t st) {
  if constexpr ((BM == 128 || BM == 256) && (BN == 128 || BN == 256)) {
    constexpr int NT = 64 * WGM * WGN * KS;
    constexpr size_t lds_xch = KS == 2 ? (size_t)BM * BN * 4 : 0;
    constexpr size_t lds_main = ((size_t)ST * (BM + BN) * BK * 2 > lds_xch) ? (size_t)ST * (BM + BN) * BK * 2 : lds_xch;
    constexpr size_t lds_fast = (size_t)(WGM * WGN) * (16 * (BN / WGN + 8) * 4 + 2 * (16 / (64 / (BN / WGN / 8))) * 2 * 1024);
    constexpr size_t lds = lds_main > lds_fast ? lds_main : lds_fast;
    GemmGroup ga;
    int blocks = 0;
    for (int i = 0; i < n; ++i) {
      ga.p[i] = d[i];
      ga.g[i].tiles_m = (int)((d[i].M + BM - 1) / BM);
      ga.g[i].tiles_n = (int)((d[i].N + BN - 1) / BN);
      ga.g[i].per_xcd = (int)(((int64_t)ga.g[i].tiles_m * ga.g[i].tiles_n + 7) / 8);
      ga.g[i].vec_epi = epi_vec_ok(d[i]);
      ga.start[i] = blocks;          // a multiple of 8: the workgroup -> XCD dealing stays aligned
      blocks += ga.g[i].per_xcd * 8;
    }
    for (int i = n; i < GEMM_GROUP_MAX; ++i) {
      ga.p[i] = d[0];
      ga.g[i] = ga.g[0];
      ga.start[i] = blocks;
    }
    ga.n = n;
    auto kern = gemm16x_group_kernel<DT, BM, BN, BK, WGM, WGN, KS, ST, true, true, EC_ACC32>;
    if (lds > 64 * 1024) {
      static std::mutex mu;
      static bool raised[64] = {};
      int dev = 0;
      if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
      std::lock_guard<std::mutex> lock(mu);
      if (!raised[dev]) {
        const hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
          pf_set_error("pf_gemm_grouped: cannot raise dynamic LDS to %zu bytes: %s", lds, hipGetErrorString(e));
          return PF_ERR_HIP;
        }
        raised[dev] = true;
      }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks, 1, 1), dim3(NT), lds, st, ga);
    PF_CHECK_LAUNCH("pf_gemm_grouped");
    return PF_OK;
  }
  pf_set_error("pf_gemm_grouped: tile %dx%d has no transposed variant", BM, BN);
  return PF_ERR_INVALID;
}

// one tile shape per translation unit (see pf_gemm_x_inst.hip)
template <int DT, int XT>
int gemm_x_group_launch(const pf_gemm_desc* d, int n, hipStream_t st) {
  using T = XTile<XT>;
  return launch16x_group<DT, T::BM, T::BN, T::BK, T::WGM, T::WGN, T::KS, T::ST>(d, n, st);
}
template <int DT, int XT>
int gemm_x_launch(const pf_gemm_desc& d, hipStream_t st) {
  using T = XTile<XT>;
  return launch16x<DT, T::BM, T::BN, T::BK, T::WGM, T::WGN, T::KS, T::ST>(d, st);
}

}  // namespace
