// Dense contractions of a pipeline stage on gfx950.
//
//   16-bit operands (fp16 / bf16): LDS-staged, double-buffered tiles feeding
//   v_mfma_f32_32x32x16_{f16,bf16}; 256 threads = 4 wavefronts in a 2x2 grid,
//   each wavefront owning a (BM/2) x (BN/2) sub-tile held in fp32 accumulators.
//   Operands whose reduction dimension is NOT the contiguous one (dX and dW
//   products) are transposed in registers (8x8 blocks of 16-bit values) on their
//   way from global memory to LDS, so that every MFMA fragment is one 16-byte
//   LDS read regardless of the storage order.
//   The epilogue re-lays each 32x32 accumulator tile through LDS so that a lane
//   owns 16 consecutive columns of one output row: bias / auxiliary / residual
//   reads and the result store are 16-byte vector accesses.
//
//   fp32 operands: a plain register-tiled FMA kernel (full fp32 accuracy; it is
//   the parity path, not the throughput path).
#include "pf_gemm_common.h"

// direct-to-LDS kernels, one object file per (operand dtype id, tile id): pf_gemm_x_inst.hip
#define PF_X_DECL(DT, XT)                                              \
  int pf_gemm_x_##DT##_##XT(const pf_gemm_desc& d, hipStream_t st);    \
  int pf_gemm_xgroup_##DT##_##XT(const pf_gemm_desc* d, int n, hipStream_t st);
#define PF_X_DECL_DT(DT) \
  PF_X_DECL(DT, 1) PF_X_DECL(DT, 2) PF_X_DECL(DT, 3) PF_X_DECL(DT, 4) PF_X_DECL(DT, 5) PF_X_DECL(DT, 6) PF_X_DECL(DT, 7) PF_X_DECL(DT, 8) PF_X_DECL(DT, 9)
PF_X_DECL_DT(1)
PF_X_DECL_DT(2)
#undef PF_X_DECL_DT
#undef PF_X_DECL
static_assert(PF_F16 == 1 && PF_BF16 == 2 && PF_XT_COUNT == 10, "the table below is written out for these ids");
typedef int (*pf_x_fn)(const pf_gemm_desc&, hipStream_t);
typedef int (*pf_xgroup_fn)(const pf_gemm_desc*, int, hipStream_t);
#define PF_X_ROW(P, DT) {nullptr, P##DT##_1, P##DT##_2, P##DT##_3, P##DT##_4, P##DT##_5, P##DT##_6, P##DT##_7, P##DT##_8, P##DT##_9}
static const pf_x_fn pf_x_table[3][PF_XT_COUNT] = {{}, PF_X_ROW(pf_gemm_x_, 1), PF_X_ROW(pf_gemm_x_, 2)};
static const pf_xgroup_fn pf_xgroup_table[3][PF_XT_COUNT] = {{}, PF_X_ROW(pf_gemm_xgroup_, 1), PF_X_ROW(pf_gemm_xgroup_, 2)};
#undef PF_X_ROW

namespace {

// Global -> register -> LDS staging of one operand tile: R rows of the output
// dimension x BK reduction elements, LDS rows padded by 8 halves (16 bytes) so
// that the 16-byte fragment reads are bank-conflict free.
//   TRANS = false: stored [row][k]  -> R*BK/2048 16-byte vectors per thread
//   TRANS = true : stored [k][row]  -> one 8(k) x 8(row) block (8 vectors) per participating
//                                      thread, transposed in registers before the LDS store
// Loads are raw buffer loads (buffer_load_dwordx4) on a descriptor whose extent
// is the operand's valid byte range: rows past the end of the matrix come back
// as zeros from the hardware range check, with no branch and a single 32-bit
// offset register per vector, so a whole tile's loads are in flight together.
// Only the reduction tail (K not a multiple of BK, last tile) is masked in
// software, at LDS-store time.
template <int R, int BK, int NT, bool TRANS> struct Stage;

template <int R, int BK, int NT> struct Stage<R, BK, NT, false> {
  static constexpr int LD = BK + 8;
  static constexpr int VPR = BK / 8;              // vectors per row
  static constexpr int NV = R * VPR / NT;         // vectors per thread
  static constexpr int NBLK = 0;                  // (transposing path only)
  static constexpr int NREG = NV;
  static_assert(NV >= 1 && NV <= 8 && NV * NT == R * VPR, "tile does not divide over the workgroup");
  // readable bytes of an R_total x K operand with row stride ld: whole 16-byte vectors (ld is a
  // multiple of 8 and >= K, so the last row's vector tail is inside the row pitch; the hardware
  // range check works on whole dwords, an extent cut inside a vector would zero valid elements)
  static __device__ __forceinline__ uint32_t extent(int64_t R_total, int64_t K, int64_t ld) {
    return (uint32_t)(((R_total - 1) * ld + (K + 7) / 8 * 8) * 2);
  }
  // byte offsets of this thread's vectors inside K-tile 0
  static __device__ __forceinline__ void init(uint32_t (&off)[NV], int64_t ld, int64_t r0, int tid, int /*first*/) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + i * NT;
      off[i] = (uint32_t)(((r0 + e / VPR) * ld + (e % VPR) * 8) * 2);
    }
  }
  static __device__ __forceinline__ uint32_t tile_step(int64_t /*ld*/) { return BK * 2; }
  static __device__ __forceinline__ void load(uint4 (&v)[NV], __amdgpu_buffer_rsrc_t rs, const uint32_t (&off)[NV],
                                              uint32_t adv, int /*tid*/, int /*first*/) {
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = buf_load16(rs, off[i] + adv);
  }
  static __device__ __forceinline__ void store(const uint4 (&v)[NV], uint16_t* s, int64_t k0, int64_t K, int tid,
                                               int /*first*/) {
    const bool tail = k0 + BK > K;  // workgroup-uniform: only the last K-tile of a ragged K
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + i * NT;
      const int row = e / VPR, kv = e % VPR;
      uint4 x = v[i];
      if (tail) {
        const int64_t gk = k0 + kv * 8;
        uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (gk + 2 * q >= K) w[q] = 0;
          else if (gk + 2 * q + 1 >= K) w[q] &= 0xffffu;
        }
        x = make_uint4(w[0], w[1], w[2], w[3]);
      }
      *(uint4*)(s + row * LD + kv * 8) = x;
    }
  }
};

template <int R, int BK, int NT> struct Stage<R, BK, NT, true> {
  static constexpr int LD = BK + 8;
  static constexpr int KB = BK / 8;                 // 8(k) x 8(row) blocks along k
  static constexpr int NBLK = (R / 8) * KB;         // one block per participating thread
  static constexpr int NREG = 8;
  static_assert(NBLK <= NT, "tile too large for one transposing block per thread");
  // readable bytes of a K x R_total operand with row stride ld (whole vectors): rows k >= K
  // are out of range and come back as zeros
  static __device__ __forceinline__ uint32_t extent(int64_t R_total, int64_t K, int64_t ld) {
    return (uint32_t)(((K - 1) * ld + (R_total + 7) / 8 * 8) * 2);
  }
  // `first` = id of the first participating thread (lets A and B use disjoint threads).
  // Consecutive threads take consecutive 8-column blocks of the same 8 k-rows, so that a
  // wavefront's load covers long contiguous runs in global memory.  Their LDS stores then
  // land 8 rows apart; the 16-byte chunk index inside the LDS row is XOR-swizzled with the
  // row-block number so that those stores (and the fragment reads) spread over the banks.
  static_assert(KB == 8, "the LDS swizzle assumes 8 chunks of 16 bytes per row");
  static __device__ __forceinline__ void init(uint32_t (&off)[8], int64_t ld, int64_t r0, int tid, int first) {
    const int b = tid - first;
    const int rb = b % (R / 8), kb = b / (R / 8);
#pragma unroll
    for (int r = 0; r < 8; ++r) off[r] = (uint32_t)((((int64_t)kb * 8 + r) * ld + r0 + rb * 8) * 2);
  }
  static __device__ __forceinline__ uint32_t tile_step(int64_t ld) { return (uint32_t)(BK * ld * 2); }
  static __device__ __forceinline__ void load(uint4 (&v)[8], __amdgpu_buffer_rsrc_t rs, const uint32_t (&off)[8],
                                              uint32_t adv, int tid, int first) {
    const int b = tid - first;
    if (b < 0 || b >= NBLK) return;  // wavefront-uniform when NBLK is a multiple of 64
    // columns beyond R_total inside a valid row read neighbouring data; they only feed
    // output rows/columns that are never stored
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = buf_load16(rs, off[r] + adv);
  }
  static __device__ __forceinline__ void store(const uint4 (&v)[8], uint16_t* s, int64_t /*k0*/, int64_t /*K*/,
                                               int tid, int first) {
    const int b = tid - first;
    if (b < 0 || b >= NBLK) return;
    const int rb = b % (R / 8), kb = b / (R / 8);
    const int chunk = kb ^ (rb & 7);
    // 8x8 transpose of 16-bit values: 2x2 transposes inside 32-bit words, the
    // 4x4 transpose of the words is pure register renaming.
    const uint32_t in[8][4] = {{v[0].x, v[0].y, v[0].z, v[0].w}, {v[1].x, v[1].y, v[1].z, v[1].w},
                               {v[2].x, v[2].y, v[2].z, v[2].w}, {v[3].x, v[3].y, v[3].z, v[3].w},
                               {v[4].x, v[4].y, v[4].z, v[4].w}, {v[5].x, v[5].y, v[5].z, v[5].w},
                               {v[6].x, v[6].y, v[6].z, v[6].w}, {v[7].x, v[7].y, v[7].z, v[7].w}};
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      uint32_t lo[4], hi[4];
#pragma unroll
      for (int I = 0; I < 4; ++I) {
        const uint32_t a = in[2 * I][J], c = in[2 * I + 1][J];
        lo[I] = (a & 0xffffu) | (c << 16);          // (k=2I, row 2J), (k=2I+1, row 2J)
        hi[I] = (a >> 16) | (c & 0xffff0000u);      // (k=2I, row 2J+1), (k=2I+1, row 2J+1)
      }
      *(uint4*)(s + (rb * 8 + 2 * J) * LD + chunk * 8) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
      *(uint4*)(s + (rb * 8 + 2 * J + 1) * LD + chunk * 8) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    }
  }
};

// Software pipeline: global loads run TWO K-tiles ahead of the MFMAs (two sets of
// staging registers, two LDS buffers).  While tile kt is multiplied out of LDS,
// tile kt+1 is already in registers (or landing) and tile kt+2 is being issued,
// which covers the ~1 us L2/HBM latency at two workgroups per CU.
template <int DT, int BM, int BN, int BK, int WGM, int WGN, bool AT, bool BT>
__global__ __launch_bounds__(64 * WGM * WGN, ((BM * BN > 128 * 128 || (AT && BT)) ? 1 : 2)  /* 8 wavefronts: 1 or 2 workgroups = 2 or 4 waves per SIMD */) void gemm16_kernel(const pf_gemm_desc p,
                                                                                              const GemmGrid g) {
  constexpr int NT = 64 * WGM * WGN;           // threads: WGM x WGN wavefronts
  constexpr int WM = BM / WGM, WN = BN / WGN;  // per-wavefront sub-tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int LD = BK + 8;
  using SA = Stage<BM, BK, NT, AT>;
  using SB = Stage<BN, BK, NT, BT>;
  extern __shared__ __align__(16) uint16_t smem[];

  const int t = gemm_tile_id((int)blockIdx.x, g.tiles_m * g.tiles_n, g.per_xcd);
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

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
  // disjoint loader threads when both operands take the transposing path
  constexpr int A_FIRST = 0;
  constexpr int B_FIRST = (AT && BT && (SA::NBLK + SB::NBLK <= NT)) ? (NT - SB::NBLK) : 0;

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  uint4 ra0[SA::NREG], rb0[SB::NREG], ra1[SA::NREG], rb1[SB::NREG];
  uint32_t offa[SA::NREG], offb[SB::NREG];
  const int nk = (int)((K + BK - 1) / BK);
  constexpr int BUF = (BM + BN) * LD;
  uint16_t* const buf0 = smem;
  uint16_t* const buf1 = smem + BUF;
  const int l31 = lane & 31, half = lane >> 5;
  const __amdgpu_buffer_rsrc_t rs_a = make_rsrc(A, SA::extent(M, K, lda));
  const __amdgpu_buffer_rsrc_t rs_b = make_rsrc(B, SB::extent(N, K, ldb));
  SA::init(offa, lda, m0, tid, A_FIRST);
  SB::init(offb, ldb, n0, tid, B_FIRST);
  const uint32_t step_a = SA::tile_step(lda), step_b = SB::tile_step(ldb);

  auto compute = [&](const uint16_t* s_a) {
    const uint16_t* s_b = s_a + BM * LD;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      uint4 fa[TM], fb[TN];
      // 16-byte chunk (kk*2 + half) of the row; tiles written by the transposing loader
      // keep it XOR-swizzled with the row's 8-row block number
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wm0 + i * 32 + l31;
        const int chunk = AT ? ((kk * 2 + half) ^ ((row >> 3) & 7)) : (kk * 2 + half);
        fa[i] = *(const uint4*)(s_a + row * LD + chunk * 8);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int row = wn0 + j * 32 + l31;
        const int chunk = BT ? ((kk * 2 + half) ^ ((row >> 3) & 7)) : (kk * 2 + half);
        fb[j] = *(const uint4*)(s_b + row * LD + chunk * 8);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<DT>::run(fa[i], fb[j], acc[i][j]);
    }
  };

  SA::load(ra0, rs_a, offa, 0, tid, A_FIRST);
  SB::load(rb0, rs_b, offb, 0, tid, B_FIRST);
  if (nk > 1) {
    SA::load(ra1, rs_a, offa, step_a, tid, A_FIRST);
    SB::load(rb1, rs_b, offb, step_b, tid, B_FIRST);
  }
  SA::store(ra0, buf0, 0, K, tid, A_FIRST);
  SB::store(rb0, buf0 + BM * LD, 0, K, tid, B_FIRST);
  __syncthreads();

  for (int kt = 0; kt < nk; kt += 2) {
    // even phase: tile kt is in buf0, tile kt+1 is in (or landing in) set 1, set 0 is free
    if (kt + 2 < nk) {
      SA::load(ra0, rs_a, offa, (uint32_t)(kt + 2) * step_a, tid, A_FIRST);
      SB::load(rb0, rs_b, offb, (uint32_t)(kt + 2) * step_b, tid, B_FIRST);
    }
    compute(buf0);
    if (kt + 1 < nk) {
      const int64_t k1 = (int64_t)(kt + 1) * BK;
      SA::store(ra1, buf1, k1, K, tid, A_FIRST);
      SB::store(rb1, buf1 + BM * LD, k1, K, tid, B_FIRST);
    }
    __syncthreads();
    // odd phase: tile kt+1 is in buf1, tile kt+2 is landing in set 0, set 1 is free.  (No early
    // exit between the phases: a single loop exit keeps the accumulators' live ranges simple,
    // which saves ~50 registers per lane.)
    if (kt + 3 < nk) {
      SA::load(ra1, rs_a, offa, (uint32_t)(kt + 3) * step_a, tid, A_FIRST);
      SB::load(rb1, rs_b, offb, (uint32_t)(kt + 3) * step_b, tid, B_FIRST);
    }
    if (kt + 1 < nk) compute(buf1);
    if (kt + 2 < nk) {
      const int64_t k2 = (int64_t)(kt + 2) * BK;
      SA::store(ra0, buf0, k2, K, tid, A_FIRST);
      SB::store(rb0, buf0 + BM * LD, k2, K, tid, B_FIRST);
    }
    __syncthreads();
  }

  // Epilogue.  D layout of v_mfma_f32_32x32x*: lane l holds column (l % 32) and
  // rows 8*(r/4) + 4*(l/32) + (r%4), r = 0..15.  Each wavefront re-lays one
  // row of TN 32x32 tiles at a time through its private LDS patch; afterwards
  // lane l owns row l/2, columns 16*(l%2) .. +16 of each tile.
  float* stage = (float*)smem + wave * (TN * 32 * EPI_LD);
  const int wr_off = ((lane >> 5) * 4) * EPI_LD + (lane & 31);
  const int rd_row = lane >> 2, rd_col = (lane & 3) * 8;
  // The accumulators are only ever indexed with compile-time constants (a dynamic
  // index would push them out of the register file): one row of TN tiles is
  // dumped with static indices, then a rolled loop runs the arithmetic on it.
  // Read-back: 4 adjacent lanes cover the 32 columns of one tile row, so every store
  // instruction writes whole 64-byte (16-bit C) or 128-byte (fp32 C) runs per row.
  static_for<TM>([&](auto ic) {
    constexpr int i = decltype(ic)::value;
    __syncthreads();  // previous tiles fully read (and, first time, main-loop tiles no longer needed)
    static_for<TN>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        stage[j * (32 * EPI_LD) + wr_off + (8 * (r >> 2) + (r & 3)) * EPI_LD] = acc[i][j][r];
    });
    __syncthreads();
#pragma nounroll
    for (int jp = 0; jp < 2 * TN; ++jp) {
      const int j = jp >> 1, rr = rd_row + 16 * (jp & 1);
      const int64_t row = m0 + wm0 + i * 32 + rr;
      const int64_t c8 = n0 + wn0 + j * 32 + rd_col;
      if (row >= M || c8 >= N) continue;
      const float4* src = (const float4*)(stage + j * (32 * EPI_LD) + rr * EPI_LD + rd_col);
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
  });
}

// ---------------------------------------------------------------------------
// fp32 FMA kernel (parity path): 64x64 tile, 16-deep, 4x4 outputs per thread
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm32_kernel(const pf_gemm_desc p, const GemmGrid g) {
  constexpr int TB = 64, TK = 16, PAD = 4;
  __shared__ float sA[TK][TB + PAD];
  __shared__ float sB[TK][TB + PAD];

  const int t = gemm_tile_id((int)blockIdx.x, g.tiles_m * g.tiles_n, g.per_xcd);
  if (t < 0) return;
  int tm, tn;
  gemm_tile_rc(t, g.tiles_m, g.tiles_n, tm, tn);
  const int64_t M = p.M, N = p.N, K = p.K;
  const int a_trans = p.a_trans, b_trans = p.b_trans;
  const int64_t m0 = (int64_t)tm * TB, n0 = (int64_t)tn * TB;
  const int64_t z = blockIdx.y, z1 = z / p.batch2, z2 = z % p.batch2;
  const float* A = (const float*)p.A + z1 * p.a_stride1 + z2 * p.a_stride2;
  const float* B = (const float*)p.B + z1 * p.b_stride1 + z2 * p.b_stride2;
  const int64_t c_base = z1 * p.c_stride1 + z2 * p.c_stride2;
  const Epi epi = make_epi(p);
  // element (m,k) of op(A) at A[m*sam + k*sak]; element (k,n) of op(B) at B[n*sbn + k*sbk]
  const int64_t sam = a_trans ? 1 : p.lda, sak = a_trans ? p.lda : 1;
  const int64_t sbn = b_trans ? 1 : p.ldb, sbk = b_trans ? p.ldb : 1;

  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int64_t k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + i * 256;
      int m, k;
      if (a_trans) { m = e & 63; k = e >> 6; } else { k = e & 15; m = e >> 4; }
      const int64_t gm = m0 + m, gk = k0 + k;
      sA[k][m] = (gm < M && gk < K) ? A[gm * sam + gk * sak] : 0.f;
      int n, kb;
      if (b_trans) { n = e & 63; kb = e >> 6; } else { kb = e & 15; n = e >> 4; }
      const int64_t gn = n0 + n, gkb = k0 + kb;
      sB[kb][n] = (gn < N && gkb < K) ? B[gn * sbn + gkb * sbk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = sA[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = sB[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t row = m0 + ty * 4 + i;
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t col = n0 + tx * 4 + j;
      if (col < N) epilogue_scalar(epi, c_base, row, col, acc[i][j]);
    }
  }
}

// ---------------------------------------------------------------------------
// fp32 MFMA kernel (v_mfma_f32_32x32x2_f32): BM x BN tile, TK deep, four wavefronts as 2 x 2, each
// owning (BM/2) x (BN/2) outputs.  Operand tiles sit in LDS reduction-major ([k][row], the order in
// which a lane reads its one element per matrix instruction: row = lane % 32, k = lane / 32); the
// next tile is fetched into registers while the current one is multiplied (two LDS buffers where
// they fit, else one and a second barrier).  The small tile is 64 deep: its problems leave one
// workgroup per CU, so a tile's matrix work has to cover the latency of the next tile's loads.
// Any layout and any size: rows / reduction indices out of range read as zero.
// ---------------------------------------------------------------------------
template <int BM, int BN, int TK, bool AT, bool BT, bool VEC>
__global__ __launch_bounds__(256) void gemm32x_kernel(const pf_gemm_desc p, const GemmGrid g) {
  constexpr int PAD = 4;
  constexpr int NBUF = (2 * TK * (BM + BN + 2 * PAD) * 4 <= 60 * 1024) ? 2 : 1;
  constexpr int TMW = BM / 64, TNW = BN / 64;          // 32x32 accumulator tiles per wavefront
  constexpr int NA = BM * TK / 256 / 4, NB = BN * TK / 256 / 4;   // 4-element loads per thread and tile
  constexpr int WN = BN / 2, SLD = WN + 8;             // epilogue: floats per staged row of a wavefront's block
  constexpr int TILE_FLOATS = NBUF * TK * (BM + BN + 2 * PAD), EPI_FLOATS = 4 * 32 * SLD;
  __shared__ __align__(16) float smem[TILE_FLOATS > EPI_FLOATS ? TILE_FLOATS : EPI_FLOATS];
  float (*sA)[TK][BM + PAD] = (float (*)[TK][BM + PAD])smem;
  float (*sB)[TK][BN + PAD] = (float (*)[TK][BN + PAD])(smem + NBUF * TK * (BM + PAD));

  const int t = gemm_tile_id((int)blockIdx.x, g.tiles_m * g.tiles_n, g.per_xcd);
  if (t < 0) return;
  int tm, tn;
  gemm_tile_rc(t, g.tiles_m, g.tiles_n, tm, tn);
  const int64_t M = p.M, N = p.N, K = p.K;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  const int64_t z = blockIdx.y, z1 = z / p.batch2, z2 = z % p.batch2;
  const float* A = (const float*)p.A + z1 * p.a_stride1 + z2 * p.a_stride2;
  const float* B = (const float*)p.B + z1 * p.b_stride1 + z2 * p.b_stride2;
  const int64_t c_base = z1 * p.c_stride1 + z2 * p.c_stride2;
  const Epi epi = make_epi(p);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * (BM / 2), wn0 = (wave & 1) * (BN / 2);

  // One operand tile -> registers, 4 consecutive elements along the operand's contiguous dimension
  // (reduction index for a row-major operand, row index for a reduction-strided one).  No branches:
  // indices are clamped into the operand and out-of-range elements are zeroed afterwards, so all of
  // a tile's loads are in flight together (a branch around a load makes the compiler wait for it at
  // the join).  VEC: one 16-byte load (the launcher has checked alignment and that the extent along
  // the contiguous dimension is a multiple of 4, so a group of 4 is inside or outside as a whole).
  auto fetch = [&](const float* X, int64_t ld, auto trans_c, int64_t r0, int64_t R, int64_t k0, int rows, int q,
                   float (&v)[4]) {
    constexpr bool TR = decltype(trans_c)::value;
    const int e = tid + q * 256;
    int r, k;
    if (TR) { r = (e % (rows / 4)) * 4; k = e / (rows / 4); } else { k = (e % (TK / 4)) * 4; r = e / (TK / 4); }
    const int64_t gr = r0 + r, gk = k0 + k;
    if (VEC) {
      const bool ok = gr < R && gk < K;
      const int64_t cr = TR ? (gr < R ? gr : R - 4) : (gr < R ? gr : R - 1);
      const int64_t ck = TR ? (gk < K ? gk : K - 1) : (gk < K ? gk : K - 4);
      const float4 x = *(const float4*)(X + (TR ? ck * ld + cr : cr * ld + ck));
      v[0] = ok ? x.x : 0.f; v[1] = ok ? x.y : 0.f; v[2] = ok ? x.z : 0.f; v[3] = ok ? x.w : 0.f;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t er = TR ? gr + j : gr, ek = TR ? gk : gk + j;
        const bool ok = er < R && ek < K;
        const int64_t cr = er < R ? er : R - 1, ck = ek < K ? ek : K - 1;
        const float x = X[TR ? ck * ld + cr : cr * ld + ck];
        v[j] = ok ? x : 0.f;
      }
    }
  };
  auto stash = [&](float* S, int ldS, auto trans_c, int rows, int q, const float (&v)[4]) {   // S: [TK][ldS]
    constexpr bool TR = decltype(trans_c)::value;
    const int e = tid + q * 256;
    if (TR) {
      const int r = (e % (rows / 4)) * 4, k = e / (rows / 4);
      *(float4*)(S + k * ldS + r) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      const int k = (e % (TK / 4)) * 4, r = e / (TK / 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) S[(k + j) * ldS + r] = v[j];
    }
  };
  constexpr std::integral_constant<bool, AT> a_trans{};
  constexpr std::integral_constant<bool, BT> b_trans{};

  float16_t acc[TMW][TNW];
#pragma unroll
  for (int i = 0; i < TMW; ++i)
#pragma unroll
    for (int j = 0; j < TNW; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Two register sets: while tile `it` is multiplied out of LDS, tile it+1 waits in one set (stored
  // to LDS at the end of the iteration) and tile it+2 is being fetched into the other, so a load has
  // two tiles' worth of matrix instructions to arrive.  (Tiles past the end of K are requested too:
  // the indices are clamped and nothing branches around the loads.)
  float ra[2][NA][4], rb[2][NB][4];
  auto fetch_tile = [&](int64_t k0, auto set_c) {
    constexpr int S = decltype(set_c)::value;
#pragma unroll
    for (int q = 0; q < NA; ++q) fetch(A, p.lda, a_trans, m0, M, k0, BM, q, ra[S][q]);
#pragma unroll
    for (int q = 0; q < NB; ++q) fetch(B, p.ldb, b_trans, n0, N, k0, BN, q, rb[S][q]);
  };
  auto stash_tile = [&](int buf, auto set_c) {
    constexpr int S = decltype(set_c)::value;
#pragma unroll
    for (int q = 0; q < NA; ++q) stash(&sA[buf][0][0], BM + PAD, a_trans, BM, q, ra[S][q]);
#pragma unroll
    for (int q = 0; q < NB; ++q) stash(&sB[buf][0][0], BN + PAD, b_trans, BN, q, rb[S][q]);
  };
  constexpr std::integral_constant<int, 0> set0{};
  constexpr std::integral_constant<int, 1> set1{};
  int cur = 0;
  fetch_tile(0, set0);
  stash_tile(0, set0);
  fetch_tile(TK, set1);
  __syncthreads();
  auto body = [&](int64_t k0, auto mine, auto other) {   // tile at k0 is in LDS, `other` holds the next one
    fetch_tile(k0 + 2 * TK, mine);
#pragma unroll
    for (int kk = 0; kk < TK / 2; ++kk) {
      const int k = 2 * kk + (lane >> 5);
      float a[TMW], b[TNW];
#pragma unroll
      for (int i = 0; i < TMW; ++i) a[i] = sA[cur][k][wm0 + i * 32 + (lane & 31)];
#pragma unroll
      for (int j = 0; j < TNW; ++j) b[j] = sB[cur][k][wn0 + j * 32 + (lane & 31)];
#pragma unroll
      for (int i = 0; i < TMW; ++i)
#pragma unroll
        for (int j = 0; j < TNW; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (NBUF == 1) __syncthreads();   // the single buffer is no longer read
    const int nxt = NBUF == 2 ? cur ^ 1 : 0;
    if (k0 + TK < K) stash_tile(nxt, other);
    __syncthreads();   // the next tile is complete (and, with two buffers, this one no longer read)
    cur = nxt;
  };
  for (int64_t k0 = 0; k0 < K; k0 += 2 * TK) {
    body(k0, set0, set1);
    if (k0 + TK < K) body(k0 + TK, set1, set0);
  }
  // Epilogue.  D layout of v_mfma_f32_32x32x*: lane l holds column l % 32 and rows 8*(r/4) + 4*(l/32) + r%4.
  // Each wavefront re-lays one 32-row block at a time through a private LDS patch, after which WN/8
  // adjacent lanes cover a whole row, 8 columns each: every global access of the epilogue moves 8
  // elements (an element-wise epilogue pays one memory round trip per element and operand).
  // (the last barrier of the K loop has passed: nobody reads the operand tiles any more)
  float* stage = smem + wave * (32 * SLD);
  constexpr int LPR = WN / 8, RPP = 64 / LPR;
  const int rd_row = lane / LPR, rd_col = (lane % LPR) * 8;
  const int64_t c8 = n0 + wn0 + rd_col;
#pragma unroll
  for (int i = 0; i < TMW; ++i) {
#pragma unroll
    for (int j = 0; j < TNW; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * SLD + j * 32 + (lane & 31)] = acc[i][j][r];
#pragma nounroll
    for (int it = 0; it < 32 / RPP; ++it) {
      const int rr = it * RPP + rd_row;
      const int64_t row = m0 + wm0 + i * 32 + rr;
      const float4 x = *(const float4*)(stage + rr * SLD + rd_col), y = *(const float4*)(stage + rr * SLD + rd_col + 4);
      if (row >= M || c8 >= N) continue;
      float v[8] = {x.x, x.y, x.z, x.w, y.x, y.y, y.z, y.w};
      if (g.vec_epi && c8 + 8 <= N) {
        epilogue_vec8(epi, c_base, row, c8, v);
      } else {
#pragma nounroll
        for (int k = 0; k < 8; ++k)
          if (c8 + k < N) epilogue_scalar(epi, c_base, row, c8 + k, v[k]);
      }
    }
  }
}

// fp32 problems: the matrix-instruction kernel with 128x128 tiles when those fill the GPU, with 64x64
// tiles otherwise (also for a handful of rows: its staged epilogue beats the FMA kernel's element-wise
// one); the plain FMA kernel for an empty reduction.
inline int f32_variant(const pf_gemm_desc& d) {
  if (d.K < 1) return 0;
  const int64_t nb = (d.batch1 > 0 ? d.batch1 : 1) * (d.batch2 > 0 ? d.batch2 : 1);
  const int64_t t128 = ((d.M + 127) / 128) * ((d.N + 127) / 128) * nb;
  return t128 >= 192 ? 128 : 64;
}

template <int DT, int BM, int BN, int BK, int WGM, int WGN>
int launch16(const pf_gemm_desc& d, hipStream_t st) {
  constexpr int NT = 64 * WGM * WGN;
  GemmGrid g;
  g.tiles_m = (int)((d.M + BM - 1) / BM);
  g.tiles_n = (int)((d.N + BN - 1) / BN);
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  g.per_xcd = (int)((total + 7) / 8);
  g.vec_epi = epi_vec_ok(d);
  const dim3 grid((unsigned)(g.per_xcd * 8), (unsigned)(d.batch1 * d.batch2), 1);
  size_t lds = 2 * (size_t)(BM + BN) * (BK + 8) * sizeof(uint16_t);
  const size_t lds_epi = (size_t)(WGM * WGN) * (BN / WGN / 32) * 32 * EPI_LD * sizeof(float);
  if (lds < lds_epi) lds = lds_epi;
  if (lds > 64 * 1024) {  // opt in to the large LDS carve-out once per instantiation
    static bool raised[4] = {false, false, false, false};
    const int v = (d.a_trans ? 2 : 0) + (d.b_trans ? 1 : 0);
    if (!raised[v]) {
      hipError_t e = hipSuccess;
      if (v == 0) e = hipFuncSetAttribute((const void*)gemm16_kernel<DT, BM, BN, BK, WGM, WGN, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (v == 1) e = hipFuncSetAttribute((const void*)gemm16_kernel<DT, BM, BN, BK, WGM, WGN, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (v == 2) e = hipFuncSetAttribute((const void*)gemm16_kernel<DT, BM, BN, BK, WGM, WGN, true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (v == 3) e = hipFuncSetAttribute((const void*)gemm16_kernel<DT, BM, BN, BK, WGM, WGN, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) {
        pf_set_error("pf_gemm: cannot raise dynamic LDS to %zu bytes: %s", lds, hipGetErrorString(e));
        return PF_ERR_HIP;
      }
      raised[v] = true;
    }
  }
#define PF_LAUNCH16(AT, BT)                                                                           \
  hipLaunchKernelGGL((gemm16_kernel<DT, BM, BN, BK, WGM, WGN, AT, BT>), grid, dim3(NT), lds, st, d, g)
  if (!d.a_trans && !d.b_trans) PF_LAUNCH16(false, false);
  else if (!d.a_trans && d.b_trans) PF_LAUNCH16(false, true);
  else if (d.a_trans && !d.b_trans) PF_LAUNCH16(true, false);
  else PF_LAUNCH16(true, true);
#undef PF_LAUNCH16
  PF_CHECK_LAUNCH("pf_gemm");
  return PF_OK;
}

// Variant ids (pf_gemm_desc.variant; 0 = automatic):
//   1..9   direct-to-LDS kernel, tiles PF_XT_256x256 / 256x128 / 128x128 / 192x256 / 128x128k2 / 256x128k2 /
//          256x256w8 / 128x128w8 / 256x128w8
//   11..14 register-staged kernel: 128x128 by 8 wavefronts, 128x128, 128x64, 64x64 by 4
enum { V_AUTO = 0, V_X256 = 1, V_X256x128 = 2, V_X128 = 3, V_X192x256 = 4, V_X128K2 = 5, V_X256x128K2 = 6, V_X256W8 = 7, V_X128W8 = 8, V_X256x128W8 = 9,
       V_R128W8 = 11, V_R128 = 12, V_R128x64 = 13, V_R64 = 14 };
inline bool is_x_variant(int v) { return v >= V_X256 && v <= V_X256x128W8; }

// Register-staged tiles: 128x128 with two workgroups resident per CU is the largest that keeps
// accumulators, two sets of staging registers and fragments in the register file; smaller tiles
// are for problems that would otherwise leave most of the 256 CUs without a workgroup.
int choose_staged(const pf_gemm_desc& d) {
  const int64_t nb = d.batch1 * d.batch2;
  auto tiles = [&](int bm, int bn) { return ((d.M + bm - 1) / bm) * ((d.N + bn - 1) / bn) * nb; };
  const bool big = (tiles(128, 128) >= 256 || (d.a_trans && d.b_trans && d.K >= 1024 && tiles(128, 128) >= 96)) &&
                   d.M >= 128 && d.N >= 128;
  // eight wavefronts (32x64 each) hide more latency per workgroup; measured +5..20% when both
  // operands use the same loader, -30% when exactly one of them is transposed
  if (big) return d.a_trans == d.b_trans ? V_R128W8 : V_R128;
  if (tiles(128, 64) >= 256 && d.M >= 128) return V_R128x64;
  return V_R64;
}

// Can the direct-to-LDS kernel run this problem with tile `xt`?  It takes both operands
// reduction-contiguous or both reduction-strided; a ragged reduction tail is zero-filled by the
// hardware range check only in the second case (whole k-rows fall outside the operand).
bool x_supports(const pf_gemm_desc& d, int xt) {
  const int bk = x_tile_bk(xt);
  if (xt == PF_XT_192x256 && d.a_trans) return false;   // no reduction-strided 192-row tile
  if (d.a_trans != d.b_trans) return false;
  if (!d.a_trans && d.K % bk != 0) return false;
  return d.K >= bk;
}

// Automatic choice: a small cost model fitted to measurements on MI355X (microseconds).  One
// workgroup per CU; a tile step of 64 along K costs t64 (MFMA issue for the big tile, operand
// delivery from L2 for the small ones, which also slow down once every CU streams at the same
// time); a launch costs ~8 us of fixed latency (dispatch, first tile, epilogue).  The candidates
// are the eight-wavefront tiles (two wavefronts per SIMD: one's LDS reads, waits and barrier
// arrivals run under the other's MFMAs; 4-13 % faster than the same tiles shared by four
// wavefronts on every shape of the five workloads) and the 192x256 tile for outputs that 256-wide
// row blocks cover badly.  On a sweep of 21 forward / input-gradient shapes of the workloads the
// choice is the fastest variant or within 3 % of it, but for long reductions: from about 4300
// deep on, the 256x128 tile whose eight wavefronts split every tile step's depth between two
// 2 x 2 grids (variant 6) is 4-8 % faster when launches of one shape run back to back (each
// wavefront reads half the fragment bytes from LDS per MFMA; the exchange of partial sums costs
// about 3 us).  It is NOT a candidate: inside the pipeline step, with other streams' kernels
// around it, the Llama and UNet-stage steps that would use it ran 0.7 % slower with it in two
// A/B runs each, so it stays a variant that can be pinned.
int choose_variant(const pf_gemm_desc& d) {
  const int64_t nb = d.batch1 * d.batch2;
  if (d.M < 128 || d.N < 128 || d.M * d.N < 128 * 128 * 16) return choose_staged(d);
  struct Cand { int v, xt, bm, bn; double t64, t64_busy, fixed; };
  static const Cand cands[4] = {{V_X256W8, PF_XT_256x256w8, 256, 256, 1.20, 1.20, 8.0},
                                {V_X192x256, PF_XT_192x256, 192, 256, 1.05, 1.05, 8.0},
                                {V_X256x128W8, PF_XT_256x128w8, 256, 128, 0.70, 0.70, 8.0},
                                {V_X128W8, PF_XT_128x128w8, 128, 128, 0.45, 0.55, 8.0}};
  int best = -1;
  double best_t = 0;
  for (const Cand& c : cands) {
    if (!x_supports(d, c.xt)) continue;
    const int64_t tiles = ((d.M + c.bm - 1) / c.bm) * ((d.N + c.bn - 1) / c.bn) * nb;
    const int64_t rounds = (tiles + 255) / 256;
    const double t = c.fixed + (double)rounds * ((double)d.K / 64.0) * (tiles > 256 ? c.t64_busy : c.t64);
    if (best < 0 || t < best_t) { best = c.v; best_t = t; }
  }
  return best < 0 ? choose_staged(d) : best;
}

// PF_GEMM_TILE_MAP="3:5,1:6": the automatic choice's tile 3 runs as tile 5, tile 1 as tile 6 (where the
// replacement supports the problem); a measurement aid, read once.
int remap_variant(const pf_gemm_desc& d, int v) {
  static int map[PF_XT_COUNT];
  static std::once_flag once;
  std::call_once(once, [] {
    for (int i = 0; i < PF_XT_COUNT; ++i) map[i] = i;
    const char* e = getenv("PF_GEMM_TILE_MAP");
    while (e && *e) {
      int a = 0, b = 0, used = 0;
      if (sscanf(e, "%d:%d%n", &a, &b, &used) == 2 && a > 0 && a < PF_XT_COUNT && b > 0 && b < PF_XT_COUNT) map[a] = b;
      e += used > 0 ? used : 1;
      while (*e == ',' || *e == ' ') ++e;
    }
  });
  if (!is_x_variant(v)) return v;
  const int w = map[v];
  return (w != v && x_supports(d, w)) ? w : v;
}

int resolve_variant(const pf_gemm_desc& d) { return d.variant == V_AUTO ? remap_variant(d, choose_variant(d)) : d.variant; }

template <int DT>
int dispatch16(const pf_gemm_desc& d, hipStream_t st) {
  const int v = resolve_variant(d);
  if (d.colsum_ws != nullptr) {   // only the GELU' class of the direct-to-LDS kernel sums its columns
    if (!is_x_variant(v) || d.a_trans || d.b_trans || !x_supports(d, v) || epi_class(d, epi_vec_ok(d)) != EC_DACT16 ||
        !pf_aligned(d.colsum_ws, 16)) {
      pf_set_error("pf_gemm: colsum_ws needs a 16-bit product with the GELU' epilogue on the direct-to-LDS kernel");
      return PF_ERR_UNSUPPORTED;
    }
  }
  if (d.nonfinite_flag != nullptr) {   // only the fp32 classes of the direct-to-LDS kernel check what they write
    const int ec = epi_class(d, epi_vec_ok(d));
    if (!is_x_variant(v) || !x_supports(d, v) || (ec != EC_STORE32 && ec != EC_ACC32) ||
        (d.a_trans != d.b_trans)) {
      pf_set_error("pf_gemm: nonfinite_flag needs a 16-bit product with fp32 C (stored or accumulated) on the direct-to-LDS kernel");
      return PF_ERR_UNSUPPORTED;
    }
  }
  switch (v) {
    case V_X256: case V_X256x128: case V_X128: case V_X192x256: case V_X128K2: case V_X256x128K2: case V_X256W8: case V_X128W8: case V_X256x128W8: {
      const int xt = v;   // variant ids 1..9 are the PF_XT_* tile ids
      if (!x_supports(d, xt)) {
        pf_set_error("pf_gemm: variant %d needs both operands stored alike and (unless transposed) K a multiple of the stage depth", v);
        return PF_ERR_INVALID;
      }
      return pf_x_table[DT][xt](d, st);
    }
    case V_R128W8: return launch16<DT, 128, 128, 64, 4, 2>(d, st);
    case V_R128: return launch16<DT, 128, 128, 64, 2, 2>(d, st);
    case V_R128x64: return launch16<DT, 128, 64, 64, 2, 2>(d, st);
    case V_R64: return launch16<DT, 64, 64, 64, 2, 2>(d, st);
    default: pf_set_error("pf_gemm: unknown variant %d", d.variant); return PF_ERR_INVALID;
  }
}

}  // namespace

extern "C" int pf_gemm(const pf_gemm_desc* desc, void* stream) {
  PF_REQUIRE(desc != nullptr, "pf_gemm: null descriptor");
  pf_gemm_desc d = *desc;
  hipStream_t st = (hipStream_t)stream;
  PF_REQUIRE(d.M >= 0 && d.N >= 0 && d.K >= 0, "pf_gemm: negative dimension");
  PF_REQUIRE(d.in_dtype == PF_F32 || d.in_dtype == PF_F16 || d.in_dtype == PF_BF16, "pf_gemm: bad in_dtype %d",
             d.in_dtype);
  PF_REQUIRE(pf_is_float_dtype(d.c_dtype), "pf_gemm: bad c_dtype %d", d.c_dtype);
  if (d.batch1 <= 0) d.batch1 = 1;
  if (d.batch2 <= 0) d.batch2 = 1;
  const int64_t nb = d.batch1 * d.batch2;
  PF_REQUIRE(nb <= 65535, "pf_gemm: batch %lld exceeds 65535", (long long)nb);
  if (d.M == 0 || d.N == 0) return PF_OK;
  PF_REQUIRE(d.A && d.B && d.C, "pf_gemm: null operand");
  PF_REQUIRE(d.beta == 0 || d.beta == 1, "pf_gemm: beta must be 0 or 1");
  PF_REQUIRE(d.lda >= (d.a_trans ? d.M : d.K), "pf_gemm: lda %lld too small", (long long)d.lda);
  PF_REQUIRE(d.ldb >= (d.b_trans ? d.N : d.K), "pf_gemm: ldb %lld too small", (long long)d.ldb);
  PF_REQUIRE(d.ldc >= d.N, "pf_gemm: ldc %lld too small", (long long)d.ldc);
  if (d.bias || d.aux_out || d.aux_in || d.residual)
    PF_REQUIRE(nb == 1, "pf_gemm: bias/aux/residual epilogues need batch == 1");
  if (d.bias) PF_REQUIRE(pf_is_float_dtype(d.bias_dtype), "pf_gemm: bad bias dtype");
  if (d.residual) PF_REQUIRE(pf_is_float_dtype(d.res_dtype) && d.ld_res >= d.N, "pf_gemm: bad residual");
  if (d.aux_out) PF_REQUIRE(d.ld_aux_out >= d.N, "pf_gemm: ld_aux_out too small");
  if (d.dact != PF_ACT_NONE) PF_REQUIRE(d.aux_in && d.ld_aux_in >= d.N, "pf_gemm: dact needs aux_in");
  const int64_t tm64 = (d.M + 63) / 64, tn64 = (d.N + 63) / 64;
  PF_REQUIRE(tm64 * tn64 < (1ll << 30), "pf_gemm: problem too large for one launch");

  if (d.in_dtype == PF_F32) {
    if (d.colsum_ws != nullptr) {
      pf_set_error("pf_gemm: colsum_ws needs a 16-bit product with the GELU' epilogue on the direct-to-LDS kernel");
      return PF_ERR_UNSUPPORTED;
    }
    if (d.nonfinite_flag != nullptr || d.unscale_by != nullptr) {
      pf_set_error("pf_gemm: unscale_by / nonfinite_flag need a 16-bit product");
      return PF_ERR_UNSUPPORTED;
    }
    GemmGrid g;
    g.vec_epi = 0;
    const int v32 = f32_variant(d);
    if (v32 == 0) {
      g.tiles_m = (int)tm64;
      g.tiles_n = (int)tn64;
      g.per_xcd = (int)((tm64 * tn64 + 7) / 8);
      hipLaunchKernelGGL(gemm32_kernel, dim3((unsigned)(g.per_xcd * 8), (unsigned)nb, 1), dim3(256), 0, st, d, g);
    } else {
      g.tiles_m = (int)((d.M + v32 - 1) / v32);
      g.tiles_n = (int)((d.N + v32 - 1) / v32);
      g.per_xcd = (int)(((int64_t)g.tiles_m * g.tiles_n + 7) / 8);
      g.vec_epi = epi_vec_ok(d);
      const dim3 grid((unsigned)(g.per_xcd * 8), (unsigned)nb, 1);
      // 16-byte loads need aligned operands whose extent along the contiguous dimension is a multiple of 4
      const bool vec = pf_aligned(d.A, 16) && pf_aligned(d.B, 16) && d.lda % 4 == 0 && d.ldb % 4 == 0 &&
                       d.a_stride1 % 4 == 0 && d.a_stride2 % 4 == 0 && d.b_stride1 % 4 == 0 && d.b_stride2 % 4 == 0 &&
                       (d.a_trans ? d.M : d.K) % 4 == 0 && (d.b_trans ? d.N : d.K) % 4 == 0 && d.K >= 4 && d.M >= 4 && d.N >= 4;
#define PF_G32(BMN, TK, AT, BT, V) hipLaunchKernelGGL((gemm32x_kernel<BMN, BMN, TK, AT, BT, V>), grid, dim3(256), 0, st, d, g)
#define PF_G32V(BMN, TK, AT, BT) do { if (vec) PF_G32(BMN, TK, AT, BT, true); else PF_G32(BMN, TK, AT, BT, false); } while (0)
#define PF_G32L(BMN, TK)                                   \
  do {                                                     \
    if (d.a_trans && d.b_trans) PF_G32V(BMN, TK, true, true);   \
    else if (d.a_trans) PF_G32V(BMN, TK, true, false);          \
    else if (d.b_trans) PF_G32V(BMN, TK, false, true);          \
    else PF_G32V(BMN, TK, false, false);                        \
  } while (0)
      if (v32 == 128) PF_G32L(128, 16);
      else PF_G32L(64, 64);
#undef PF_G32L
#undef PF_G32V
#undef PF_G32
    }
    PF_CHECK_LAUNCH("pf_gemm(f32)");
    return PF_OK;
  }
  // 16-byte vector path requirements
  PF_REQUIRE(pf_aligned(d.A, 16) && pf_aligned(d.B, 16), "pf_gemm: 16-bit operands must be 16-byte aligned");
  PF_REQUIRE(d.lda % 8 == 0 && d.ldb % 8 == 0, "pf_gemm: lda/ldb must be multiples of 8 for 16-bit operands");
  PF_REQUIRE(d.a_stride1 % 8 == 0 && d.a_stride2 % 8 == 0 && d.b_stride1 % 8 == 0 && d.b_stride2 % 8 == 0,
             "pf_gemm: batch strides of 16-bit operands must be multiples of 8");
  // operands are addressed with 32-bit byte offsets inside a buffer descriptor
  const int64_t a_bytes = ((d.a_trans ? d.K : d.M) + 256) * d.lda * 2, b_bytes = ((d.b_trans ? d.K : d.N) + 256) * d.ldb * 2;
  PF_REQUIRE(a_bytes < (1ll << 31) && b_bytes < (1ll << 31),
             "pf_gemm: a 16-bit operand (per batch entry) must be smaller than 2 GiB");
  if (d.K == 0) {  // nothing to reduce: the fp32 kernel's epilogue-only path handles it
    GemmGrid g;
    const int64_t tm = (d.M + 63) / 64, tn = (d.N + 63) / 64;
    g.tiles_m = (int)tm;
    g.tiles_n = (int)tn;
    g.per_xcd = (int)((tm * tn + 7) / 8);
    g.vec_epi = 0;
    hipLaunchKernelGGL(gemm32_kernel, dim3((unsigned)(g.per_xcd * 8), (unsigned)nb, 1), dim3(256), 0, st, d, g);
    PF_CHECK_LAUNCH("pf_gemm(K=0)");
    return PF_OK;
  }
  if (d.in_dtype == PF_F16) return dispatch16<PF_F16>(d, st);
  return dispatch16<PF_BF16>(d, st);
}

// Checks shared by pf_gemm and pf_gemm_grouped for one 16-bit descriptor that is to run on the
// direct-to-LDS weight-gradient kernel as part of a group.
namespace {
bool groupable(const pf_gemm_desc& d, int& variant) {
  if (d.in_dtype != PF_F16 && d.in_dtype != PF_BF16) return false;
  if (!(d.a_trans && d.b_trans) || d.c_dtype != PF_F32 || (d.beta != 0 && d.beta != 1)) return false;
  if (d.batch1 > 1 || d.batch2 > 1 || d.bias || d.residual || d.aux_in || d.aux_out || d.act || d.dact) return false;
  if (d.M <= 0 || d.N <= 0 || d.K <= 0 || !d.A || !d.B || !d.C) return false;
  if (!pf_aligned(d.A, 16) || !pf_aligned(d.B, 16) || d.lda % 8 || d.ldb % 8 || d.lda < d.M || d.ldb < d.N ||
      d.ldc < d.N)
    return false;
  const int64_t a_bytes = (d.K + 256) * d.lda * 2, b_bytes = (d.K + 256) * d.ldb * 2;
  if (a_bytes >= (1ll << 31) || b_bytes >= (1ll << 31)) return false;
  variant = resolve_variant(d);
  if (!is_x_variant(variant) || variant == V_X192x256) return false;
  if (!x_supports(d, variant)) return false;
  // (a product that stores rides in the accumulate launch: its old C reads as zeros)
  const int ec = epi_class(d, epi_vec_ok(d));
  return ec == EC_ACC32 || ec == EC_STORE32;
}
}  // namespace

extern "C" int pf_gemm_grouped(const pf_gemm_desc* descs, int n, void* stream) {
  PF_REQUIRE(n >= 0 && (n == 0 || descs != nullptr), "pf_gemm_grouped: bad arguments");
  int i = 0;
  while (i < n) {
    // longest run (up to the kernel's group size) of problems that share one instantiation
    int v0 = 0, run = 0;
    if (groupable(descs[i], v0)) {
      run = 1;
      int v = 0;
      while (i + run < n && run < PF_GEMM_GROUP_MAX && descs[i + run].in_dtype == descs[i].in_dtype && groupable(descs[i + run], v) &&
             v == v0)
        ++run;
    }
    if (run >= 2) {
      pf_gemm_desc d[PF_GEMM_GROUP_MAX];
      for (int k = 0; k < run; ++k) {
        d[k] = descs[i + k];
        d[k].batch1 = d[k].batch2 = 1;
      }
      const int rc = pf_xgroup_table[descs[i].in_dtype][v0](d, run, (hipStream_t)stream);
      if (rc != PF_OK) return rc;
      i += run;
    } else {
      const int rc = pf_gemm(&descs[i], stream);
      if (rc != PF_OK) return rc;
      ++i;
    }
  }
  return PF_OK;
}

extern "C" int pf_gemm_variant(const pf_gemm_desc* desc, char* out, int cap) {
  PF_REQUIRE(desc && out && cap > 0, "pf_gemm_variant: bad arguments");
  pf_gemm_desc d = *desc;
  if (d.batch1 <= 0) d.batch1 = 1;
  if (d.batch2 <= 0) d.batch2 = 1;
  if (d.in_dtype == PF_F32 || d.K == 0) {
    const int v32 = (d.in_dtype == PF_F32 && d.K > 0) ? f32_variant(d) : 0;
    if (v32) snprintf(out, (size_t)cap, "gemm32x_kernel<%d, %d, %d>", v32, v32, v32 == 128 ? 16 : 64);
    else snprintf(out, (size_t)cap, "gemm32_kernel");
    return PF_OK;
  }
  const char* at = d.a_trans ? "true" : "false";
  const char* bt = d.b_trans ? "true" : "false";
  const int v = resolve_variant(d);
  switch (v) {
    case V_X256: case V_X256x128: case V_X128: case V_X192x256: case V_X128K2: case V_X256x128K2: case V_X256W8: case V_X128W8: case V_X256x128W8: {
      // BM, BN, BK, wavefront rows, columns, reduction split, stages: as rocprofv3 prints the instantiation
      static const char* shapes[PF_XT_COUNT] = {"", "256, 256, 32, 2, 2, 1, 5", "256, 128, 64, 2, 2, 1, 3", "128, 128, 64, 2, 2, 1, 3",
                                                "192, 256, 32, 2, 2, 1, 5", "128, 128, 64, 2, 2, 2, 3", "256, 128, 64, 2, 2, 2, 3",
                                                "256, 256, 32, 2, 4, 1, 5", "128, 128, 64, 2, 4, 1, 3", "256, 128, 64, 4, 2, 1, 3"};
      if (!x_supports(d, v)) {   // a pinned tile that cannot run this product: say so here, not at launch time
        pf_set_error("pf_gemm_variant: variant %d needs both operands stored alike, K >= %d and (unless both are "
                     "reduction-strided) K a multiple of %d", v, x_tile_bk(v), x_tile_bk(v));
        return PF_ERR_INVALID;
      }
      int ec = epi_class(d, epi_vec_ok(d));
      if (d.a_trans && ec != EC_ACC32 && ec != EC_STORE32) ec = EC_GENERIC;
      snprintf(out, (size_t)cap, "gemm16x_kernel<%d, %s, %s, %s, %d>", d.in_dtype, shapes[v], at, bt, ec);
      return PF_OK;
    }
    case V_R128W8: snprintf(out, (size_t)cap, "gemm16_kernel<%d, 128, 128, 64, 4, 2, %s, %s>", d.in_dtype, at, bt); return PF_OK;
    case V_R128: snprintf(out, (size_t)cap, "gemm16_kernel<%d, 128, 128, 64, 2, 2, %s, %s>", d.in_dtype, at, bt); return PF_OK;
    case V_R128x64: snprintf(out, (size_t)cap, "gemm16_kernel<%d, 128, 64, 64, 2, 2, %s, %s>", d.in_dtype, at, bt); return PF_OK;
    case V_R64: snprintf(out, (size_t)cap, "gemm16_kernel<%d, 64, 64, 64, 2, 2, %s, %s>", d.in_dtype, at, bt); return PF_OK;
    default: pf_set_error("pf_gemm_variant: unknown variant %d", d.variant); return PF_ERR_INVALID;
  }
}
