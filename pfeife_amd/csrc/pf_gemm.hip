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
#include <type_traits>

#include "pf_common.h"

namespace {

struct GemmGrid {
  int tiles_m, tiles_n, per_xcd;
  int vec_epi;  // every epilogue operand is 16-byte aligned with leading dimensions % 8 == 0
};

// Epilogue operands, copied out of the descriptor so that they live in scalar registers.
struct Epi {
  float alpha;
  int beta, round_mid, act, dact, in_dtype, c_dtype, bias_dtype, res_dtype;
  const void* bias;
  void* aux_out;
  const void* aux_in;
  const void* residual;
  void* C;
  int64_t ldc, ld_aux_out, ld_aux_in, ld_res;
};

__device__ __forceinline__ Epi make_epi(const pf_gemm_desc& p) {
  Epi e;
  e.alpha = p.alpha; e.beta = p.beta; e.round_mid = p.round_mid; e.act = p.act; e.dact = p.dact;
  e.in_dtype = p.in_dtype; e.c_dtype = p.c_dtype; e.bias_dtype = p.bias_dtype; e.res_dtype = p.res_dtype;
  e.bias = p.bias; e.aux_out = p.aux_out; e.aux_in = p.aux_in; e.residual = p.residual; e.C = p.C;
  e.ldc = p.ldc; e.ld_aux_out = p.ld_aux_out; e.ld_aux_in = p.ld_aux_in; e.ld_res = p.ld_res;
  return e;
}

// one element (scalar path: fp32 kernel and ragged / unaligned tails)
__device__ __forceinline__ void epilogue_scalar(const Epi& e, int64_t c_base, int64_t row, int64_t col, float acc) {
  float v = e.alpha * acc;
  if (e.bias) v += pf_load_as_f32(e.bias, col, e.bias_dtype);
  if (e.round_mid) v = pf_round_to(e.in_dtype, v);
  if (e.aux_out) pf_store_from_f32(e.aux_out, row * e.ld_aux_out + col, e.in_dtype, v);
  if (e.act != PF_ACT_NONE) v = pf_act(e.act, v);
  if (e.dact != PF_ACT_NONE) v *= pf_act_grad(e.dact, pf_load_as_f32(e.aux_in, row * e.ld_aux_in + col, e.in_dtype));
  if (e.residual) v += pf_load_as_f32(e.residual, row * e.ld_res + col, e.res_dtype);
  const int64_t ci = c_base + row * e.ldc + col;
  if (e.beta) v += pf_load_as_f32(e.C, ci, e.c_dtype);
  pf_store_from_f32(e.C, ci, e.c_dtype, v);
}

// 8 consecutive columns of one row (vector path)
__device__ __forceinline__ void epilogue_vec8(const Epi& e, int64_t c_base, int64_t row, int64_t col, float (&v)[8]) {
  float t[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) v[k] *= e.alpha;
  if (e.bias) {
    ld_vec<8>(e.bias, col, e.bias_dtype, t);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] += t[k];
  }
  if (e.round_mid) {
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = pf_round_to(e.in_dtype, v[k]);
  }
  if (e.aux_out) st_vec<8>(e.aux_out, row * e.ld_aux_out + col, e.in_dtype, v);
  if (e.act != PF_ACT_NONE) {
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = pf_act(e.act, v[k]);
  }
  if (e.dact != PF_ACT_NONE) {
    ld_vec<8>(e.aux_in, row * e.ld_aux_in + col, e.in_dtype, t);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] *= pf_act_grad(e.dact, t[k]);
  }
  if (e.residual) {
    ld_vec<8>(e.residual, row * e.ld_res + col, e.res_dtype, t);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] += t[k];
  }
  const int64_t ci = c_base + row * e.ldc + col;
  if (e.beta) {
    ld_vec<8>(e.C, ci, e.c_dtype, t);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] += t[k];
  }
  st_vec<8>(e.C, ci, e.c_dtype, v);
}

// XCD-aware tile id: consecutive workgroup ids are dealt round-robin to the 8
// XCDs, so give each XCD a contiguous range of tiles (its L2 then sees a compact
// set of A rows / B columns). Returns -1 for the padding workgroups.
__device__ __forceinline__ int gemm_tile_id(int tiles, int per_xcd) {
  const int pid = blockIdx.x;
  const int t = (pid & 7) * per_xcd + (pid >> 3);
  return t < tiles ? t : -1;
}

// ---------------------------------------------------------------------------
// 16-bit MFMA kernel
// ---------------------------------------------------------------------------
constexpr int BK = 64;           // reduction elements per LDS tile
constexpr int LDS_LD = BK + 8;   // padded LDS row (halves): 144 B keeps 16-byte reads conflict-free
constexpr int EPI_LD = 40;       // floats per row of the 32x32 epilogue staging tile

template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

template <int DT> struct Mfma;
template <> struct Mfma<PF_F16> {
  static __device__ __forceinline__ float16_t run(uint4 a, uint4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0,
                                                  0, 0);
  }
};
template <> struct Mfma<PF_BF16> {
  static __device__ __forceinline__ float16_t run(uint4 a, uint4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  }
};

// Global -> register staging of one operand tile (R rows of the output dimension x BK).
//   TRANS = false: stored [row][k]  -> R/32 16-byte vectors per thread
//   TRANS = true : stored [k][row]  -> one 8x8 block (8 vectors) per participating thread
template <int R, bool TRANS> struct Stage;

template <int R> struct Stage<R, false> {
  static constexpr int NV = R / 32;  // R*8 vectors over 256 threads
  static __device__ __forceinline__ void load(uint4 (&v)[8], const uint16_t* base, int64_t ld, int64_t r0,
                                              int64_t R_total, int64_t k0, int64_t K, int tid, int /*first*/) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + i * 256;
      const int row = e >> 3, kv = e & 7;
      const int64_t gr = r0 + row, gk = k0 + kv * 8;
      uint4 x = make_uint4(0, 0, 0, 0);
      if (gr < R_total && gk < K) {
        x = *(const uint4*)(base + gr * ld + gk);
        if (gk + 8 > K) {  // K tail inside this vector: zero the elements >= K
          uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (gk + 2 * q >= K) w[q] = 0;
            else if (gk + 2 * q + 1 >= K) w[q] &= 0xffffu;
          }
          x = make_uint4(w[0], w[1], w[2], w[3]);
        }
      }
      v[i] = x;
    }
  }
  static __device__ __forceinline__ void store(const uint4 (&v)[8], uint16_t* s, int tid, int /*first*/) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + i * 256;
      const int row = e >> 3, kv = e & 7;
      *(uint4*)(s + row * LDS_LD + kv * 8) = v[i];
    }
  }
};

template <int R> struct Stage<R, true> {
  // R/8 x 8 blocks of 8(k) x 8(row) elements; one block per thread, R <= 256.
  static constexpr int NBLK = R;  // (R/8) * (BK/8)
  // `first` = id of the first participating thread (lets A and B use disjoint threads)
  static __device__ __forceinline__ void load(uint4 (&v)[8], const uint16_t* base, int64_t ld, int64_t r0,
                                              int64_t R_total, int64_t k0, int64_t K, int tid, int first) {
    const int b = tid - first;
    const bool mine = b >= 0 && b < NBLK;
    const int rb = b % (R / 8), kb = b / (R / 8);
    const int64_t gr = r0 + rb * 8;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int64_t gk = k0 + kb * 8 + r;
      uint4 x = make_uint4(0, 0, 0, 0);
      // rows of the output dimension beyond R_total only feed output rows that
      // are never stored, but the read itself must stay inside the allocation:
      // ld is a multiple of 8 and >= R_total, so gr + 8 <= ld whenever gr < R_total.
      if (mine && gk < K && gr < R_total) x = *(const uint4*)(base + gk * ld + gr);
      v[r] = x;
    }
  }
  static __device__ __forceinline__ void store(const uint4 (&v)[8], uint16_t* s, int tid, int first) {
    const int b = tid - first;
    if (b < 0 || b >= NBLK) return;
    const int rb = b % (R / 8), kb = b / (R / 8);
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
      *(uint4*)(s + (rb * 8 + 2 * J) * LDS_LD + kb * 8) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
      *(uint4*)(s + (rb * 8 + 2 * J + 1) * LDS_LD + kb * 8) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    }
  }
};

template <int DT, int BM, int BN, bool AT, bool BT>
__global__ __launch_bounds__(256) void gemm16_kernel(const pf_gemm_desc p, const GemmGrid g) {
  constexpr int WM = BM / 2, WN = BN / 2;  // per-wavefront sub-tile
  constexpr int TM = WM / 32, TN = WN / 32;
  extern __shared__ __align__(16) uint16_t smem[];

  const int t = gemm_tile_id(g.tiles_m * g.tiles_n, g.per_xcd);
  if (t < 0) return;
  const int tm = t % g.tiles_m, tn = t / g.tiles_m;
  const int64_t M = p.M, N = p.N, K = p.K, lda = p.lda, ldb = p.ldb;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  const int64_t z = blockIdx.y, z1 = z / p.batch2, z2 = z % p.batch2;
  const uint16_t* A = (const uint16_t*)p.A + z1 * p.a_stride1 + z2 * p.a_stride2;
  const uint16_t* B = (const uint16_t*)p.B + z1 * p.b_stride1 + z2 * p.b_stride2;
  const int64_t c_base = z1 * p.c_stride1 + z2 * p.c_stride2;
  const Epi epi = make_epi(p);
  const int vec_epi = g.vec_epi;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
  // disjoint loader threads when both operands take the transposing path
  constexpr int A_FIRST = 0;
  constexpr int B_FIRST = (AT && BT && (BM + BN <= 256)) ? (256 - BN) : 0;

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  uint4 ra[8], rb[8];
  const int nk = (int)((K + BK - 1) / BK);
  constexpr int BUF = (BM + BN) * LDS_LD;

  Stage<BM, AT>::load(ra, A, lda, m0, M, 0, K, tid, A_FIRST);
  Stage<BN, BT>::load(rb, B, ldb, n0, N, 0, K, tid, B_FIRST);
  Stage<BM, AT>::store(ra, smem, tid, A_FIRST);
  Stage<BN, BT>::store(rb, smem + BM * LDS_LD, tid, B_FIRST);
  __syncthreads();

  const int frag_off = (lane & 31) * LDS_LD + (lane >> 5) * 8;
  for (int kt = 0; kt < nk; ++kt) {
    const bool more = kt + 1 < nk;
    if (more) {
      const int64_t k0 = (int64_t)(kt + 1) * BK;
      Stage<BM, AT>::load(ra, A, lda, m0, M, k0, K, tid, A_FIRST);
      Stage<BN, BT>::load(rb, B, ldb, n0, N, k0, K, tid, B_FIRST);
    }
    const uint16_t* s_a = smem + (kt & 1) * BUF;
    const uint16_t* s_b = s_a + BM * LDS_LD;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      uint4 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = *(const uint4*)(s_a + (wm0 + i * 32) * LDS_LD + frag_off + kk * 16);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = *(const uint4*)(s_b + (wn0 + j * 32) * LDS_LD + frag_off + kk * 16);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<DT>::run(fa[i], fb[j], acc[i][j]);
    }
    if (more) {
      uint16_t* s = smem + ((kt + 1) & 1) * BUF;
      Stage<BM, AT>::store(ra, s, tid, A_FIRST);
      Stage<BN, BT>::store(rb, s + BM * LDS_LD, tid, B_FIRST);
    }
    __syncthreads();
  }

  // Epilogue.  D layout of v_mfma_f32_32x32x*: lane l holds column (l % 32) and
  // rows 8*(r/4) + 4*(l/32) + (r%4), r = 0..15.  Each wavefront re-lays one
  // 32x32 tile at a time through its private LDS patch; afterwards lane l owns
  // row l/2, columns 16*(l%2) .. +16 of the tile.
  float* stage = (float*)smem + wave * (TN * 32 * EPI_LD);
  const int wr_off = ((lane >> 5) * 4) * EPI_LD + (lane & 31);
  const int rd_row = lane >> 1, rd_col = (lane & 1) * 16;
  // The accumulators are only ever indexed with compile-time constants (a dynamic
  // index would push them out of the register file): one row of TN tiles is
  // dumped with static indices, then a rolled loop runs the arithmetic on it.
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
    const int64_t row = m0 + wm0 + i * 32 + rd_row;
    if (row < M) {
#pragma nounroll
      for (int jh = 0; jh < 2 * TN; ++jh) {
        const int j = jh >> 1, h = jh & 1;
        const int64_t c8 = n0 + wn0 + j * 32 + rd_col + h * 8;
        if (c8 >= N) continue;
        const float4* src = (const float4*)(stage + j * (32 * EPI_LD) + rd_row * EPI_LD + rd_col + h * 8);
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
  });
}

// ---------------------------------------------------------------------------
// fp32 FMA kernel (parity path): 64x64 tile, 16-deep, 4x4 outputs per thread
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm32_kernel(const pf_gemm_desc p, const GemmGrid g) {
  constexpr int TB = 64, TK = 16, PAD = 4;
  __shared__ float sA[TK][TB + PAD];
  __shared__ float sB[TK][TB + PAD];

  const int t = gemm_tile_id(g.tiles_m * g.tiles_n, g.per_xcd);
  if (t < 0) return;
  const int tm = t % g.tiles_m, tn = t / g.tiles_m;
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

bool epi_ptr_ok(const void* p, int64_t ld) { return p == nullptr || (pf_aligned(p, 16) && ld % 8 == 0); }

template <int DT, int BM, int BN>
int launch16(const pf_gemm_desc& d, hipStream_t st) {
  GemmGrid g;
  g.tiles_m = (int)((d.M + BM - 1) / BM);
  g.tiles_n = (int)((d.N + BN - 1) / BN);
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  g.per_xcd = (int)((total + 7) / 8);
  g.vec_epi = epi_ptr_ok(d.C, d.ldc) && d.c_stride1 % 8 == 0 && d.c_stride2 % 8 == 0 &&
              (d.bias == nullptr || pf_aligned(d.bias, 16)) && epi_ptr_ok(d.aux_out, d.ld_aux_out) &&
              epi_ptr_ok(d.aux_in, d.ld_aux_in) && epi_ptr_ok(d.residual, d.ld_res);
  const dim3 grid((unsigned)(g.per_xcd * 8), (unsigned)(d.batch1 * d.batch2), 1);
  size_t lds = 2 * (size_t)(BM + BN) * LDS_LD * sizeof(uint16_t);
  const size_t lds_epi = 4 * (size_t)(BN / 64) * 32 * EPI_LD * sizeof(float);
  if (lds < lds_epi) lds = lds_epi;
  if (lds > 64 * 1024) {  // opt in to the large LDS carve-out once per instantiation
    static bool raised[4] = {false, false, false, false};
    const int v = (d.a_trans ? 2 : 0) + (d.b_trans ? 1 : 0);
    if (!raised[v]) {
      hipError_t e = hipSuccess;
      if (v == 0) e = hipFuncSetAttribute((const void*)gemm16_kernel<DT, BM, BN, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (v == 1) e = hipFuncSetAttribute((const void*)gemm16_kernel<DT, BM, BN, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (v == 2) e = hipFuncSetAttribute((const void*)gemm16_kernel<DT, BM, BN, true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (v == 3) e = hipFuncSetAttribute((const void*)gemm16_kernel<DT, BM, BN, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) {
        pf_set_error("pf_gemm: cannot raise dynamic LDS to %zu bytes: %s", lds, hipGetErrorString(e));
        return PF_ERR_HIP;
      }
      raised[v] = true;
    }
  }
#define PF_LAUNCH16(AT, BT)                                                                           \
  hipLaunchKernelGGL((gemm16_kernel<DT, BM, BN, AT, BT>), grid, dim3(256), lds, st, d, g)
  if (!d.a_trans && !d.b_trans) PF_LAUNCH16(false, false);
  else if (!d.a_trans && d.b_trans) PF_LAUNCH16(false, true);
  else if (d.a_trans && !d.b_trans) PF_LAUNCH16(true, false);
  else PF_LAUNCH16(true, true);
#undef PF_LAUNCH16
  PF_CHECK_LAUNCH("pf_gemm");
  return PF_OK;
}

// Tile choice: the largest tile that still yields at least ~one workgroup per
// CU (256 CUs); small problems (attention heads, narrow projections) take
// smaller tiles so the launch fills the chip.  tile = 0: 256x128, 1: 128x128,
// 2: 128x64, 3: 64x64.
int choose_tile(const pf_gemm_desc& d) {
  const int64_t nb = (d.batch1 > 0 ? d.batch1 : 1) * (d.batch2 > 0 ? d.batch2 : 1);
  auto tiles = [&](int bm, int bn) { return ((d.M + bm - 1) / bm) * ((d.N + bn - 1) / bn) * nb; };
  if (tiles(256, 128) >= 512 && d.M >= 256) return 0;
  if (tiles(128, 128) >= 256 && d.M >= 128 && d.N >= 128) return 1;
  if (tiles(128, 64) >= 256 && d.M >= 128) return 2;
  return 3;
}

template <int DT>
int dispatch16(const pf_gemm_desc& d, hipStream_t st) {
  switch (choose_tile(d)) {
    case 0: return launch16<DT, 256, 128>(d, st);
    case 1: return launch16<DT, 128, 128>(d, st);
    case 2: return launch16<DT, 128, 64>(d, st);
    default: return launch16<DT, 64, 64>(d, st);
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
    GemmGrid g;
    g.tiles_m = (int)tm64;
    g.tiles_n = (int)tn64;
    g.per_xcd = (int)((tm64 * tn64 + 7) / 8);
    g.vec_epi = 0;
    hipLaunchKernelGGL(gemm32_kernel, dim3((unsigned)(g.per_xcd * 8), (unsigned)nb, 1), dim3(256), 0, st, d, g);
    PF_CHECK_LAUNCH("pf_gemm(f32)");
    return PF_OK;
  }
  // 16-byte vector path requirements
  PF_REQUIRE(pf_aligned(d.A, 16) && pf_aligned(d.B, 16), "pf_gemm: 16-bit operands must be 16-byte aligned");
  PF_REQUIRE(d.lda % 8 == 0 && d.ldb % 8 == 0, "pf_gemm: lda/ldb must be multiples of 8 for 16-bit operands");
  PF_REQUIRE(d.a_stride1 % 8 == 0 && d.a_stride2 % 8 == 0 && d.b_stride1 % 8 == 0 && d.b_stride2 % 8 == 0,
             "pf_gemm: batch strides of 16-bit operands must be multiples of 8");
  if (d.in_dtype == PF_F16) return dispatch16<PF_F16>(d, st);
  return dispatch16<PF_BF16>(d, st);
}

extern "C" int pf_gemm_variant(const pf_gemm_desc* desc, char* out, int cap) {
  PF_REQUIRE(desc && out && cap > 0, "pf_gemm_variant: bad arguments");
  static const char* tile_names[4] = {"256, 128", "128, 128", "128, 64", "64, 64"};
  if (desc->in_dtype == PF_F32) {
    snprintf(out, (size_t)cap, "gemm32_kernel");
  } else {
    snprintf(out, (size_t)cap, "gemm16_kernel<%d, %s, %s, %s>", desc->in_dtype, tile_names[choose_tile(*desc)],
             desc->a_trans ? "true" : "false", desc->b_trans ? "true" : "false");
  }
  return PF_OK;
}
