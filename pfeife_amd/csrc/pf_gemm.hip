// Dense contractions of a pipeline stage on gfx950.
//
//   16-bit operands (fp16 / bf16): LDS-staged, double-buffered tiles feeding
//   v_mfma_f32_32x32x16_{f16,bf16}; 256 threads = 4 wavefronts in a 2x2 grid,
//   each wavefront owning a (BM/2) x (BN/2) sub-tile held in fp32 accumulators.
//   Operands whose reduction dimension is NOT the contiguous one (dX and dW
//   products) are transposed in registers (8x8 blocks of 16-bit values) on their
//   way from global memory to LDS, so that every MFMA fragment is one 16-byte
//   LDS read regardless of the storage order.
//
//   fp32 operands: a plain register-tiled FMA kernel (full fp32 accuracy; it is
//   the parity path, not the throughput path).
//
// The epilogue (bias, 16-bit rounding, activation, activation gradient, residual,
// fp32 accumulate) is shared by both.
#include "pf_common.h"

namespace {

struct GemmGrid {
  int tiles_m, tiles_n, per_xcd;
};

__device__ __forceinline__ void gemm_epilogue(const pf_gemm_desc& p, int64_t c_base, int64_t row, int64_t col,
                                              float acc) {
  float v = p.alpha * acc;
  if (p.bias) v += pf_load_as_f32(p.bias, col, p.bias_dtype);
  if (p.round_mid) v = pf_round_to(p.in_dtype, v);
  if (p.aux_out) pf_store_from_f32(p.aux_out, row * p.ld_aux_out + col, p.in_dtype, v);
  if (p.act != PF_ACT_NONE) v = pf_act(p.act, v);
  if (p.dact != PF_ACT_NONE) v *= pf_act_grad(p.dact, pf_load_as_f32(p.aux_in, row * p.ld_aux_in + col, p.in_dtype));
  if (p.residual) v += pf_load_as_f32(p.residual, row * p.ld_res + col, p.res_dtype);
  const int64_t ci = c_base + row * p.ldc + col;
  if (p.beta) v += pf_load_as_f32(p.C, ci, p.c_dtype);
  pf_store_from_f32(p.C, ci, p.c_dtype, v);
}

// XCD-aware tile id: consecutive workgroup ids are dealt round-robin to the 8
// XCDs, so give each XCD a contiguous range of tiles (its L2 then sees a compact
// set of A rows / B columns). Returns -1 for the padding workgroups.
__device__ __forceinline__ int gemm_tile_id(const GemmGrid& g) {
  const int pid = blockIdx.x;
  const int t = (pid & 7) * g.per_xcd + (pid >> 3);
  return t < g.tiles_m * g.tiles_n ? t : -1;
}

// ---------------------------------------------------------------------------
// 16-bit MFMA kernel
// ---------------------------------------------------------------------------
constexpr int BK = 64;           // reduction elements per LDS tile
constexpr int LDS_LD = BK + 8;   // padded LDS row (halves): 144 B keeps 16-byte reads conflict-free

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

// Register staging of one operand tile (R rows of the output dimension x BK).
//   TRANS = false: stored [row][k]  -> R/32 16-byte vectors per thread
//   TRANS = true : stored [k][row]  -> one 8x8 block (8 vectors) per participating thread
template <int R, bool TRANS> struct Stage;

template <int R> struct Stage<R, false> {
  static constexpr int NV = R / 32;  // R*8 vectors over 256 threads
  uint4 v[NV];
  __device__ __forceinline__ void load(const uint16_t* base, int64_t ld, int64_t r0, int64_t R_total, int64_t k0,
                                       int64_t K, int tid) {
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
  __device__ __forceinline__ void store(uint16_t* s, int tid) const {
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
  uint4 v[8];
  // `first` = id of the first participating thread (lets A and B use disjoint threads)
  __device__ __forceinline__ void load(const uint16_t* base, int64_t ld, int64_t r0, int64_t R_total, int64_t k0,
                                       int64_t K, int tid, int first) {
    const int b = tid - first;
    if (b < 0 || b >= NBLK) return;
    const int rb = b % (R / 8), kb = b / (R / 8);
    const int64_t gr = r0 + rb * 8;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int64_t gk = k0 + kb * 8 + r;
      uint4 x = make_uint4(0, 0, 0, 0);
      // rows of the output dimension beyond R_total only feed output rows that
      // are never stored, but the read itself must stay inside the allocation:
      // ld is a multiple of 8 and >= R_total, so gr + 8 <= ld whenever gr < R_total.
      if (gk < K && gr < R_total) x = *(const uint4*)(base + gk * ld + gr);
      v[r] = x;
    }
  }
  __device__ __forceinline__ void store(uint16_t* s, int tid, int first) const {
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

  const int t = gemm_tile_id(g);
  if (t < 0) return;
  const int tm = t % g.tiles_m, tn = t / g.tiles_m;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  const int64_t z = blockIdx.y, z1 = z / p.batch2, z2 = z % p.batch2;
  const uint16_t* A = (const uint16_t*)p.A + z1 * p.a_stride1 + z2 * p.a_stride2;
  const uint16_t* B = (const uint16_t*)p.B + z1 * p.b_stride1 + z2 * p.b_stride2;
  const int64_t c_base = z1 * p.c_stride1 + z2 * p.c_stride2;

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

  Stage<BM, AT> sa;
  Stage<BN, BT> sb;
  const int nk = (int)((p.K + BK - 1) / BK);
  constexpr int BUF = (BM + BN) * LDS_LD;

  auto load_tiles = [&](int kt) {
    const int64_t k0 = (int64_t)kt * BK;
    if constexpr (AT) sa.load(A, p.lda, m0, p.M, k0, p.K, tid, A_FIRST);
    else sa.load(A, p.lda, m0, p.M, k0, p.K, tid);
    if constexpr (BT) sb.load(B, p.ldb, n0, p.N, k0, p.K, tid, B_FIRST);
    else sb.load(B, p.ldb, n0, p.N, k0, p.K, tid);
  };
  auto store_tiles = [&](int buf) {
    uint16_t* s = smem + buf * BUF;
    if constexpr (AT) sa.store(s, tid, A_FIRST);
    else sa.store(s, tid);
    if constexpr (BT) sb.store(s + BM * LDS_LD, tid, B_FIRST);
    else sb.store(s + BM * LDS_LD, tid);
  };

  load_tiles(0);
  store_tiles(0);
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const bool more = kt + 1 < nk;
    if (more) load_tiles(kt + 1);

    const uint16_t* s_a = smem + (kt & 1) * BUF;
    const uint16_t* s_b = s_a + BM * LDS_LD;
    const int frag_off = (lane & 31) * LDS_LD + (lane >> 5) * 8;
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

    if (more) store_tiles((kt + 1) & 1);
    __syncthreads();
  }

  // D layout of v_mfma_f32_32x32x*: lane l holds column (l % 32) and rows
  // 8*(r/4) + 4*(l/32) + (r%4), r = 0..15.
  const int col_l = lane & 31, row_l = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int64_t col = n0 + wn0 + j * 32 + col_l;
      if (col >= p.N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = m0 + wm0 + i * 32 + 8 * (r >> 2) + row_l + (r & 3);
        if (row < p.M) gemm_epilogue(p, c_base, row, col, acc[i][j][r]);
      }
    }
}

// ---------------------------------------------------------------------------
// fp32 FMA kernel (parity path): 64x64 tile, 16-deep, 4x4 outputs per thread
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm32_kernel(const pf_gemm_desc p, const GemmGrid g) {
  constexpr int TB = 64, TK = 16, PAD = 4;
  __shared__ float sA[TK][TB + PAD];
  __shared__ float sB[TK][TB + PAD];

  const int t = gemm_tile_id(g);
  if (t < 0) return;
  const int tm = t % g.tiles_m, tn = t / g.tiles_m;
  const int64_t m0 = (int64_t)tm * TB, n0 = (int64_t)tn * TB;
  const int64_t z = blockIdx.y, z1 = z / p.batch2, z2 = z % p.batch2;
  const float* A = (const float*)p.A + z1 * p.a_stride1 + z2 * p.a_stride2;
  const float* B = (const float*)p.B + z1 * p.b_stride1 + z2 * p.b_stride2;
  const int64_t c_base = z1 * p.c_stride1 + z2 * p.c_stride2;
  // element (m,k) of op(A) at A[m*sam + k*sak]; element (k,n) of op(B) at B[n*sbn + k*sbk]
  const int64_t sam = p.a_trans ? 1 : p.lda, sak = p.a_trans ? p.lda : 1;
  const int64_t sbn = p.b_trans ? 1 : p.ldb, sbk = p.b_trans ? p.ldb : 1;

  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int64_t k0 = 0; k0 < p.K; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + i * 256;
      int m, k;
      if (p.a_trans) { m = e & 63; k = e >> 6; } else { k = e & 15; m = e >> 4; }
      const int64_t gm = m0 + m, gk = k0 + k;
      sA[k][m] = (gm < p.M && gk < p.K) ? A[gm * sam + gk * sak] : 0.f;
      int n, kb;
      if (p.b_trans) { n = e & 63; kb = e >> 6; } else { kb = e & 15; n = e >> 4; }
      const int64_t gn = n0 + n, gkb = k0 + kb;
      sB[kb][n] = (gn < p.N && gkb < p.K) ? B[gn * sbn + gkb * sbk] : 0.f;
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
    if (row >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t col = n0 + tx * 4 + j;
      if (col < p.N) gemm_epilogue(p, c_base, row, col, acc[i][j]);
    }
  }
}

template <int DT, int BM, int BN>
int launch16(const pf_gemm_desc& d, hipStream_t st) {
  GemmGrid g;
  g.tiles_m = (int)((d.M + BM - 1) / BM);
  g.tiles_n = (int)((d.N + BN - 1) / BN);
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  g.per_xcd = (int)((total + 7) / 8);
  const dim3 grid((unsigned)(g.per_xcd * 8), (unsigned)(d.batch1 * d.batch2), 1);
  const size_t lds = 2 * (size_t)(BM + BN) * LDS_LD * sizeof(uint16_t);
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
