// Fused attention (forward, dQ, dK/dV) on gfx950 MFMA: softmax(Q K^T * scale [+ causal]) V
// without materialising the [B,H,Tq,Tk] score / probability matrices.
//
// All three kernels work in the "transposed world": score tiles are computed so that a
// lane owns ONE column of the tile (lane % 32) and 16 rows of it in registers.  The
// softmax statistics of that column are then a per-lane loop plus one exchange with
// lane ^ 32, and the probabilities can be fed straight back into the next MFMA as the
// B operand (the MFMA reduction index may be permuted freely as long as A and B agree),
// so P never goes through LDS.
//
//   forward / dQ kernel : tile = S^T[kv][q], column = query row   (workgroup = 128 queries)
//   dK/dV kernel        : tile = S[q][kv],   column = key row     (workgroup = 128 keys)
//
// Operands whose MFMA reduction index is NOT their contiguous dimension (V in forward,
// K in dQ, Q and dO in dK/dV) stay in their natural [token][hd] layout in LDS and are read
// with the transposing LDS read (ds_read_b64_tr_b16); no transposed copy exists anywhere.
//
// Q, K, V, O and their gradients are [B, H, T, hd] tensors addressed with element
// strides (batch, head, token) and unit stride along hd, so heads can live inside a
// packed qkv projection and the output can be token-major.
#include <mutex>
#include <set>
#include <utility>

#include "pf_common.h"

namespace {

constexpr int KT = 64;        // keys (forward/dQ) or queries (dK/dV) per LDS tile
constexpr float LOG2E = 1.4426950408889634f;

struct AttnArgs {
  const uint16_t* q; const uint16_t* k; const uint16_t* v; const uint16_t* o; const uint16_t* d_o;
  uint16_t* out; uint16_t* dq; uint16_t* dk; uint16_t* dv;
  float* lse; const float* delta;
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st, o_sb, o_sh, o_st;
  int64_t do_sb, do_sh, do_st, dq_sb, dq_sh, dq_st, dk_sb, dk_sh, dk_st, dv_sb, dv_sh, dv_st;
  int B, H, Tq, Tk, hd, causal;
  float scale;
};

template <int DT> struct M32;
template <> struct M32<PF_F16> {
  static __device__ __forceinline__ float16_t run(uint4 a, uint4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0,
                                                  0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pf_pack2_f16(lo, hi); }
};
template <> struct M32<PF_BF16> {
  static __device__ __forceinline__ float16_t run(uint4 a, uint4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pf_pack2_bf16(lo, hi); }
};

// registers r..r+7 of an accumulator tile -> one 16-byte MFMA operand (8 x 16-bit)
template <int DT>
__device__ __forceinline__ uint4 pack8(const float16_t& a, int r) {
  return make_uint4(M32<DT>::pack(a[r], a[r + 1]), M32<DT>::pack(a[r + 2], a[r + 3]),
                    M32<DT>::pack(a[r + 4], a[r + 5]), M32<DT>::pack(a[r + 6], a[r + 7]));
}

// row index inside a 32-row accumulator tile of register r for this lane
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// 16-byte global load of 8 consecutive hd elements of one token row; zero when the
// token or the hd chunk is out of range
__device__ __forceinline__ uint4 load_row8(const uint16_t* base, int64_t st, int t, int T, int h0, int hd) {
  if (t < T && h0 < hd) return *(const uint4*)(base + (int64_t)t * st + h0);
  return make_uint4(0, 0, 0, 0);
}

// One [ROWS tokens][HD] tile in flight: NV 16-byte vectors per thread, loaded from global into
// registers while the previous tile is being multiplied, stored to LDS ([KT][HD + 8]) afterwards.
template <int HD, int ROWS = KT> struct Tile {
  static constexpr int LD = HD + 8, VPR = HD / 8, NV = (ROWS * VPR + 255) / 256;
  uint4 v[NV];
  __device__ __forceinline__ void load(const uint16_t* base, int64_t st, int t0, int T, int hd, int tid) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + i * 256;
      v[i] = (e < ROWS * VPR) ? load_row8(base, st, t0 + e / VPR, T, (e % VPR) * 8, hd) : make_uint4(0, 0, 0, 0);
    }
  }
  __device__ __forceinline__ void store(uint16_t* s, int tid) const {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + i * 256;
      if (e < ROWS * VPR) *(uint4*)(s + (e / VPR) * LD + (e % VPR) * 8) = v[i];
    }
  }
};

#define PF_LDS16(T) __attribute__((address_space(3))) T*
typedef short short4v_t __attribute__((ext_vector_type(4)));

// Transposing LDS read.  The 16 lanes of a group each name an 8-byte chunk (4 elements);
// group lane j must point at row k0 + j/4, columns n0 + 4*(j%4); lane i of the group then
// receives the four elements (k0 .. k0+3, column n0 + i).
__device__ __forceinline__ uint2 lds_read_tr(const uint16_t* p) {
  const short4v_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PF_LDS16(short4v_t))(uintptr_t)p);
  return __builtin_bit_cast(uint2, r);
}

// A operand X^T[row = hd index][k = token] for the 16-token chunk starting at `t0` of a
// natural [token][LD] tile, hd rows o32 .. o32+31, with the token permutation of pack8():
// element i of the lane <-> token t0 + 8*(i/4) + 4*(lane/32) + (i%4)
template <int LD>
__device__ __forceinline__ uint4 frag_tr(const uint16_t* s, int t0, int o32, int lane) {
  const int g = lane >> 4, j = lane & 15;
  const uint16_t* p = s + (t0 + 4 * (g >> 1) + (j >> 2)) * LD + o32 + 16 * (g & 1) + 4 * (j & 3);
  const uint2 lo = lds_read_tr(p), hi = lds_read_tr(p + 8 * LD);
  return make_uint4(lo.x, lo.y, hi.x, hi.y);
}

// Workgroup -> (row block, batch*head).  The hardware starts workgroups in the order of their
// linear id (x fastest).  Under a causal mask the blocks of one head differ in work by up to the
// number of blocks (a query block sweeps the keys up to its diagonal, a key block the queries from
// its diagonal on): the heaviest blocks of EVERY head are started first, the lightest ones fill the
// tail.  Without a mask all blocks are alike and neighbours keep sharing a head's operands in L2.
__device__ __forceinline__ void attn_block(const AttnArgs& a, bool heavy_is_last, int& blk, int& bh) {
  blk = (int)blockIdx.x;
  bh = (int)blockIdx.y;
  if (a.causal) {
    const int id = (int)(blockIdx.y * gridDim.x + blockIdx.x), nbh = (int)gridDim.y;
    const int k = id / nbh;
    bh = id % nbh;
    blk = heavy_is_last ? (int)gridDim.x - 1 - k : k;
  }
}

// ---------------------------------------------------------------------------------
// forward: one workgroup = 128 queries of one (batch, head); wavefront w owns 32 of them
//
// Occupancy (second __launch_bounds__ argument) of the tiled kernels: a tile step is a chain of
// dependent MFMA -> softmax -> MFMA phases with LDS reads in between, so a SIMD that holds a single
// wavefront idles through every latency.  The register budget is set so that three (forward, head
// dim <= 64: 152 VGPRs) or two (dQ: 240, dK/dV: 247) wavefronts share a SIMD without spilling;
// measured on 2048 causal tokens x 64 heads: forward 76 -> 56 us, backward 280 -> 194 us.
// ---------------------------------------------------------------------------------
template <int DT, int HD>
__global__ __launch_bounds__(256, HD <= 64 ? 3 : 1) void attn_fwd_kernel(const AttnArgs a) {
  constexpr int NC = HD / 16, NO = HD / 32, KLD = HD + 8;
  __shared__ __align__(16) uint16_t sK[KT * KLD];
  __shared__ __align__(16) uint16_t sV[KT * KLD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int qb, bh;
  attn_block(a, true, qb, bh);
  const int b = bh / a.H, h = bh % a.H;
  const int q0 = qb * 128 + wave * 32;
  const int qi = q0 + (lane & 31);          // this lane's query row
  const uint16_t* Q = a.q + b * a.q_sb + h * a.q_sh;
  const uint16_t* K = a.k + b * a.k_sb + h * a.k_sh;
  const uint16_t* V = a.v + b * a.v_sb + h * a.v_sh;
  const float sc = a.scale * LOG2E;
  const int shift = a.Tk - a.Tq;            // causal: key j visible to query i iff j <= i + shift

  uint4 qf[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) qf[c] = load_row8(Q, a.q_st, qi, a.Tq, c * 16 + (lane >> 5) * 8, a.hd);

  float16_t oacc[NO];
#pragma unroll
  for (int o = 0; o < NO; ++o)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[o][r] = 0.f;
  float m = -INFINITY, l = 0.f;

  int k_end = a.Tk;
  if (a.causal) {
    const int last_q = min(qb * 128 + 127, a.Tq - 1);
    k_end = min(a.Tk, last_q + shift + 1);
  }
  Tile<HD> tk, tv;
  tk.load(K, a.k_st, 0, a.Tk, a.hd, tid);
  tv.load(V, a.v_st, 0, a.Tk, a.hd, tid);
  for (int k0 = 0; k0 < k_end; k0 += KT) {
    __syncthreads();                     // previous tile's LDS reads are done
    tk.store(sK, tid);
    tv.store(sV, tid);
    if (k0 + KT < k_end) {               // next tile's global loads fly during this tile's math
      tk.load(K, a.k_st, k0 + KT, a.Tk, a.hd, tid);
      tv.load(V, a.v_st, k0 + KT, a.Tk, a.hd, tid);
    }
    __syncthreads();
    float16_t s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[t][r] = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const uint4 kf = *(const uint4*)(sK + (t * 32 + (lane & 31)) * KLD + c * 16 + (lane >> 5) * 8);
        s[t] = M32<DT>::run(kf, qf[c], s[t]);
      }
    }
    // only the tile on the causal diagonal and the ragged last tile need per-element masks
    const bool masked = (k0 + KT > a.Tk) || (a.causal && k0 + KT - 1 > q0 + shift);
    float mx = m;   // running maximum of the RAW scores (scale > 0, so the ordering is the same)
    if (masked) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kj = k0 + t * 32 + acc_row(r, lane);
          const bool ok = kj < a.Tk && (!a.causal || kj <= qi + shift);
          s[t][r] = ok ? s[t][r] : -INFINITY;
          mx = fmaxf(mx, s[t][r]);
        }
    } else {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[t][r]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const bool dead = (mx == -INFINITY);
    const float moff = dead ? 0.f : -mx * sc;
    const float alpha = dead ? 1.f : __builtin_amdgcn_exp2f((m - mx) * sc);
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[t][r], sc, moff));   // masked entries: exp2(-inf) = 0
        s[t][r] = p;
        psum += p;
      }
    l = l * alpha + psum;
    m = mx;
    if (__any(alpha != 1.f)) {   // wavefront-uniform: once the maxima have settled nothing is rescaled
#pragma unroll
      for (int o = 0; o < NO; ++o)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[o][r] *= alpha;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint4 pf = pack8<DT>(s[j >> 1], 8 * (j & 1));
#pragma unroll
      for (int o = 0; o < NO; ++o) {
        oacc[o] = M32<DT>::run(frag_tr<KLD>(sV, 16 * j, o * 32, lane), pf, oacc[o]);
      }
    }
  }
  l += __shfl_xor(l, 32, 64);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (qi < a.Tq) {
    uint16_t* O = a.out + b * a.o_sb + h * a.o_sh + (int64_t)qi * a.o_st;
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int h0 = o * 32 + 8 * g + 4 * (lane >> 5);
        if (h0 < a.hd) {
          const uint2 w = make_uint2(M32<DT>::pack(oacc[o][4 * g] * inv, oacc[o][4 * g + 1] * inv),
                                     M32<DT>::pack(oacc[o][4 * g + 2] * inv, oacc[o][4 * g + 3] * inv));
          *(uint2*)(O + h0) = w;
        }
      }
    if ((lane >> 5) == 0) a.lse[((int64_t)bh) * a.Tq + qi] = (l > 0.f) ? (m * sc + log2f(l)) / LOG2E : -INFINITY;
  }
}

// delta[b,h,q] = sum_hd dO * O : 8 lanes per row (16-byte loads), 8 rows per wavefront
__global__ __launch_bounds__(256) void attn_delta_kernel(const AttnArgs a, float* delta) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t rows = (int64_t)a.B * a.H * a.Tq;
  const int64_t row = ((int64_t)blockIdx.x * 4 + wave) * 8 + (lane >> 3);
  const bool bf = (a.causal & 0x100) != 0;
  float s = 0.f;
  if (row < rows) {
    const int q = (int)(row % a.Tq);
    const int bh = (int)(row / a.Tq), b = bh / a.H, h = bh % a.H;
    const uint16_t* O = a.o + b * a.o_sb + h * a.o_sh + (int64_t)q * a.o_st;
    const uint16_t* D = a.d_o + b * a.do_sb + h * a.do_sh + (int64_t)q * a.do_st;
    for (int c = (lane & 7) * 8; c < a.hd; c += 64) {
      float x[8], y[8];
      if (bf) { Vec8<PF_BF16>::load(O, c, x); Vec8<PF_BF16>::load(D, c, y); }
      else { Vec8<PF_F16>::load(O, c, x); Vec8<PF_F16>::load(D, c, y); }
#pragma unroll
      for (int k = 0; k < 8; ++k) s += x[k] * y[k];
    }
  }
  s += __shfl_xor(s, 1, 64);
  s += __shfl_xor(s, 2, 64);
  s += __shfl_xor(s, 4, 64);
  if (row < rows && (lane & 7) == 0) delta[row] = s;
}

// ---------------------------------------------------------------------------------
// dQ: same tiling as forward (column = query); dQ^T[hd][q] += K^T[hd][kv] dS^T[kv][q]
// ---------------------------------------------------------------------------------
template <int DT, int HD>
__global__ __launch_bounds__(256, HD <= 64 ? 2 : 1) void attn_dq_kernel(const AttnArgs a) {
  constexpr int NC = HD / 16, NO = HD / 32, KLD = HD + 8;
  __shared__ __align__(16) uint16_t sK[KT * KLD];
  __shared__ __align__(16) uint16_t sV[KT * KLD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int qb, bh;
  attn_block(a, true, qb, bh);
  const int b = bh / a.H, h = bh % a.H;
  const int q0 = qb * 128 + wave * 32;
  const int qi = q0 + (lane & 31);
  const uint16_t* Q = a.q + b * a.q_sb + h * a.q_sh;
  const uint16_t* K = a.k + b * a.k_sb + h * a.k_sh;
  const uint16_t* V = a.v + b * a.v_sb + h * a.v_sh;
  const uint16_t* DO = a.d_o + b * a.do_sb + h * a.do_sh;
  const float sc = a.scale * LOG2E;
  const int shift = a.Tk - a.Tq;

  uint4 qf[NC], dof[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    qf[c] = load_row8(Q, a.q_st, qi, a.Tq, c * 16 + (lane >> 5) * 8, a.hd);
    dof[c] = load_row8(DO, a.do_st, qi, a.Tq, c * 16 + (lane >> 5) * 8, a.hd);
  }
  const bool qok = qi < a.Tq;
  // a query row past the end keeps lse = +inf so that its probabilities are exactly zero
  const float lse2 = qok ? a.lse[(int64_t)bh * a.Tq + qi] * LOG2E : INFINITY;
  const float dlt = qok ? a.delta[(int64_t)bh * a.Tq + qi] : 0.f;

  float16_t acc[NO];
#pragma unroll
  for (int o = 0; o < NO; ++o)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[o][r] = 0.f;

  int k_end = a.Tk;
  if (a.causal) {
    const int last_q = min(qb * 128 + 127, a.Tq - 1);
    k_end = min(a.Tk, last_q + shift + 1);
  }
  Tile<HD> tk, tv;
  tk.load(K, a.k_st, 0, a.Tk, a.hd, tid);
  tv.load(V, a.v_st, 0, a.Tk, a.hd, tid);
  for (int k0 = 0; k0 < k_end; k0 += KT) {
    __syncthreads();
    tk.store(sK, tid);
    tv.store(sV, tid);
    if (k0 + KT < k_end) {
      tk.load(K, a.k_st, k0 + KT, a.Tk, a.hd, tid);
      tv.load(V, a.v_st, k0 + KT, a.Tk, a.hd, tid);
    }
    __syncthreads();
    const bool masked = (k0 + KT > a.Tk) || (a.causal && k0 + KT - 1 > q0 + shift);
    float16_t s[2], dp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[t][r] = dp[t][r] = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int off = (t * 32 + (lane & 31)) * KLD + c * 16 + (lane >> 5) * 8;
        s[t] = M32<DT>::run(*(const uint4*)(sK + off), qf[c], s[t]);
        dp[t] = M32<DT>::run(*(const uint4*)(sV + off), dof[c], dp[t]);
      }
      if (masked) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kj = k0 + t * 32 + acc_row(r, lane);
          const bool ok = kj < a.Tk && (!a.causal || kj <= qi + shift);
          const float p = ok ? __builtin_amdgcn_exp2f(s[t][r] * sc - lse2) : 0.f;
          s[t][r] = p * (dp[t][r] - dlt);   // dS^T / scale (the scale is applied to dQ at the end)
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[t][r] = __builtin_amdgcn_exp2f(s[t][r] * sc - lse2) * (dp[t][r] - dlt);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint4 dsf = pack8<DT>(s[j >> 1], 8 * (j & 1));
#pragma unroll
      for (int o = 0; o < NO; ++o) {
        acc[o] = M32<DT>::run(frag_tr<KLD>(sK, 16 * j, o * 32, lane), dsf, acc[o]);
      }
    }
  }
  if (qok) {
    uint16_t* DQ = a.dq + b * a.dq_sb + h * a.dq_sh + (int64_t)qi * a.dq_st;
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int h0 = o * 32 + 8 * g + 4 * (lane >> 5);
        if (h0 < a.hd)
          *(uint2*)(DQ + h0) = make_uint2(M32<DT>::pack(acc[o][4 * g] * a.scale, acc[o][4 * g + 1] * a.scale),
                                          M32<DT>::pack(acc[o][4 * g + 2] * a.scale, acc[o][4 * g + 3] * a.scale));
      }
  }
}

// ---------------------------------------------------------------------------------
// dK/dV: column = key row; S[q][kv] = Q K^T, dV^T[hd][kv] += dO^T[hd][q] P[q][kv],
//        dK^T[hd][kv] += Q^T[hd][q] dS[q][kv]
// ---------------------------------------------------------------------------------
// SPLITQ (few keys, many queries: cross attention to a short context): a workgroup owns ONE 32-key
// tile, its four wavefronts each take a quarter of every staged block of 128 queries, and their
// accumulators are added at the end through LDS in wavefront order, so that a head's dK/dV come
// from 4 x ceil(Tk / 32) wavefronts instead of ceil(Tk / 32).
template <int DT, int HD, bool SPLITQ = false>
__global__ __launch_bounds__(256, SPLITQ ? 1 : 2) void attn_dkv_kernel(const AttnArgs a) {
  constexpr int NC = HD / 16, NO = HD / 32, QLD = HD + 8;
  constexpr int QT = SPLITQ ? 128 : KT;        // queries staged per iteration
  constexpr int NH = SPLITQ ? 1 : 2;           // 32-query halves per wavefront and iteration
  __shared__ __align__(16) uint16_t sQD[2 * QT * QLD];
  uint16_t* sQ = sQD;
  uint16_t* sDO = sQD + QT * QLD;
  __shared__ float sLse[QT], sDelta[QT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int kb, bh;
  attn_block(a, false, kb, bh);
  const int b = bh / a.H, h = bh % a.H;
  const int kw0 = SPLITQ ? kb * 32 : kb * 128 + wave * 32;     // this wavefront's first key row
  const int qoff = SPLITQ ? wave * 32 : 0;                     // its first query row inside a staged block
  const int kj = kw0 + (lane & 31);                            // this lane's key row
  const uint16_t* Q = a.q + b * a.q_sb + h * a.q_sh;
  const uint16_t* K = a.k + b * a.k_sb + h * a.k_sh;
  const uint16_t* V = a.v + b * a.v_sb + h * a.v_sh;
  const uint16_t* DO = a.d_o + b * a.do_sb + h * a.do_sh;
  const float sc = a.scale * LOG2E;
  const int shift = a.Tk - a.Tq;
  const bool kok = kj < a.Tk;

  uint4 kf[NC], vf[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    kf[c] = load_row8(K, a.k_st, kj, a.Tk, c * 16 + (lane >> 5) * 8, a.hd);
    vf[c] = load_row8(V, a.v_st, kj, a.Tk, c * 16 + (lane >> 5) * 8, a.hd);
  }
  float16_t dk[NO], dv[NO];
#pragma unroll
  for (int o = 0; o < NO; ++o)
#pragma unroll
    for (int r = 0; r < 16; ++r) dk[o][r] = dv[o][r] = 0.f;

  int q_begin = 0;
  if (a.causal) {  // queries i with i + shift >= first key of the block see it
    q_begin = max(0, (SPLITQ ? kb * 32 : kb * 128) - shift);
    q_begin = q_begin / QT * QT;
  }
  Tile<HD, QT> tq, tdo;
  float r_lse = 0.f, r_dlt = 0.f;
  auto prefetch = [&](int q0) {
    tq.load(Q, a.q_st, q0, a.Tq, a.hd, tid);
    tdo.load(DO, a.do_st, q0, a.Tq, a.hd, tid);
    if (tid < QT) {
      const int qi = q0 + tid;
      // rows past the end: Q and dO rows are zero, lse = +inf makes their P exactly zero
      r_lse = qi < a.Tq ? a.lse[(int64_t)bh * a.Tq + qi] * LOG2E : INFINITY;
      r_dlt = qi < a.Tq ? a.delta[(int64_t)bh * a.Tq + qi] : 0.f;
    }
  };
  if (q_begin < a.Tq) prefetch(q_begin);
  for (int q0 = q_begin; q0 < a.Tq; q0 += QT) {
    __syncthreads();
    tq.store(sQ, tid);
    tdo.store(sDO, tid);
    if (tid < QT) {
      sLse[tid] = r_lse;
      sDelta[tid] = r_dlt;
    }
    if (q0 + QT < a.Tq) prefetch(q0 + QT);
    __syncthreads();
    // causal: the tile needs element masks only where it crosses the diagonal
    const bool masked = a.causal && (kw0 + 31 > q0 + qoff + shift);
    float16_t s[NH], dp[NH];
#pragma unroll
    for (int t = 0; t < NH; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[t][r] = dp[t][r] = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int off = (qoff + t * 32 + (lane & 31)) * QLD + c * 16 + (lane >> 5) * 8;
        s[t] = M32<DT>::run(*(const uint4*)(sQ + off), kf[c], s[t]);
        dp[t] = M32<DT>::run(*(const uint4*)(sDO + off), vf[c], dp[t]);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int ql = qoff + t * 32 + acc_row(r, lane);
        float p = __builtin_amdgcn_exp2f(s[t][r] * sc - sLse[ql]);
        if (masked && kj > q0 + ql + shift) p = 0.f;
        s[t][r] = p;                                         // P
        dp[t][r] = p * (dp[t][r] - sDelta[ql]);              // dS / scale (applied to dK at the end)
      }
    }
#pragma unroll
    for (int j = 0; j < 2 * NH; ++j) {
      const uint4 pf = pack8<DT>(s[j >> 1], 8 * (j & 1));
      const uint4 dsf = pack8<DT>(dp[j >> 1], 8 * (j & 1));
#pragma unroll
      for (int o = 0; o < NO; ++o) {
        dv[o] = M32<DT>::run(frag_tr<QLD>(sDO, qoff + 16 * j, o * 32, lane), pf, dv[o]);
        dk[o] = M32<DT>::run(frag_tr<QLD>(sQ, qoff + 16 * j, o * 32, lane), dsf, dk[o]);
      }
    }
  }
  if constexpr (SPLITQ) {
    // wavefront 0 adds the other three's accumulators in wavefront order: dV, then dK
    float* red = (float*)sQD;
    static_assert(3 * NO * 16 * 64 * 4 <= 2 * QT * QLD * 2, "reduction patch exceeds the operand tiles");
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      __syncthreads();   // the tiles (or the previous pass's patch) are no longer read
      if (wave > 0) {
#pragma unroll
        for (int o = 0; o < NO; ++o)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            red[(((wave - 1) * NO + o) * 16 + r) * 64 + lane] = pass == 0 ? dv[o][r] : dk[o][r];
      }
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
          for (int o = 0; o < NO; ++o)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float x = red[((w * NO + o) * 16 + r) * 64 + lane];
              if (pass == 0) dv[o][r] += x; else dk[o][r] += x;
            }
      }
    }
    if (wave != 0) return;
  }
  if (kok) {
    uint16_t* DK = a.dk + b * a.dk_sb + h * a.dk_sh + (int64_t)kj * a.dk_st;
    uint16_t* DV = a.dv + b * a.dv_sb + h * a.dv_sh + (int64_t)kj * a.dv_st;
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int h0 = o * 32 + 8 * g + 4 * (lane >> 5);
        if (h0 < a.hd) {
          *(uint2*)(DK + h0) = make_uint2(M32<DT>::pack(dk[o][4 * g] * a.scale, dk[o][4 * g + 1] * a.scale),
                                          M32<DT>::pack(dk[o][4 * g + 2] * a.scale, dk[o][4 * g + 3] * a.scale));
          *(uint2*)(DV + h0) = make_uint2(M32<DT>::pack(dv[o][4 * g], dv[o][4 * g + 1]),
                                          M32<DT>::pack(dv[o][4 * g + 2], dv[o][4 * g + 3]));
        }
      }
  }
}


// =================================================================================
// Short sequences (Tq, Tk <= SHORT_T, e.g. ViT's 197 or 257 tokens): the two operands a workgroup
// sweeps over (K and V, or Q and dO) are loaded into LDS ONCE, whole, in their natural
// [token][hd] layout; after a single barrier every wavefront runs its tile loop without
// any further synchronisation.  Operands the MFMA needs transposed (V^T, K^T, Q^T, dO^T)
// are read from the natural layout with the transposing LDS read (ds_read_b64_tr_b16),
// so no transposed copy is made.
// =================================================================================
constexpr int SHORT_T = 288;   // 2 operands x 288 rows x (96 + 8) x 2 bytes = 117 KB of the 160 KB
template <int DT>
__device__ __forceinline__ void unpack8(const uint4& r, float (&v)[8]) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if constexpr (DT == PF_F16) {
      v[2 * k] = pf_f16_bits_to_f32((uint16_t)(w[k] & 0xffffu));
      v[2 * k + 1] = pf_f16_bits_to_f32((uint16_t)(w[k] >> 16));
    } else {
      v[2 * k] = __uint_as_float(w[k] << 16);
      v[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
    }
  }
}

// Two whole [T][hd] operands of one head -> LDS [rows][HD + 8] each (rows past T and hd
// chunks past hd are zero); NT threads, eight 16-byte loads in flight per thread
template <int HD, int NT>
__device__ __forceinline__ void load_heads(const uint16_t* x, int64_t x_st, const uint16_t* y, int64_t y_st, int T,
                                           int hd, int rows, uint16_t* sx, uint16_t* sy, int tid) {
  constexpr int VPR = HD / 8, LD = HD + 8;
  const int n = rows * VPR;
  for (int e0 = 0; e0 < n; e0 += NT * 4) {
    uint4 vx[4], vy[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = e0 + i * NT + tid;
      const int t = e / VPR, c = (e % VPR) * 8;
      vx[i] = e < n ? load_row8(x, x_st, t, T, c, hd) : make_uint4(0, 0, 0, 0);
      vy[i] = e < n ? load_row8(y, y_st, t, T, c, hd) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = e0 + i * NT + tid;
      if (e < n) {
        *(uint4*)(sx + (e / VPR) * LD + (e % VPR) * 8) = vx[i];
        *(uint4*)(sy + (e / VPR) * LD + (e % VPR) * 8) = vy[i];
      }
    }
  }
}

// forward: workgroup = NT / 2 queries of one (batch, head) at a time, wavefront = 32 of them; keys in
// steps of 32.  A wavefront whose tile lies past what the grid covers at once (gridDim.x * NT / 2
// queries) takes it in a second pass.  NT = 512 (eight wavefronts) lets ONE workgroup cover a whole head,
// so that the head's K and V are fetched once instead of once per 128 queries; NT = 256 otherwise.
template <int DT, int HD, int NT>
__global__ __launch_bounds__(NT) void attn_fwd_short_kernel(const AttnArgs a, int rows) {
  constexpr int NC = HD / 16, NO = HD / 32, LD = HD + 8;
  extern __shared__ __align__(16) uint16_t smem[];
  uint16_t* sK = smem;
  uint16_t* sV = smem + rows * LD;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const int q_step = (int)gridDim.x * (NT / 2);
  int q0 = blockIdx.x * (NT / 2) + wave * 32;
  const uint16_t* Q = a.q + b * a.q_sb + h * a.q_sh;
  const float sc = a.scale * LOG2E;
  const int shift = a.Tk - a.Tq;

  uint4 qf[NC];   // the first tile's queries are requested before the head is loaded
#pragma unroll
  for (int c = 0; c < NC; ++c) qf[c] = load_row8(Q, a.q_st, q0 + (lane & 31), a.Tq, c * 16 + (lane >> 5) * 8, a.hd);
  load_heads<HD, NT>(a.k + b * a.k_sb + h * a.k_sh, a.k_st, a.v + b * a.v_sb + h * a.v_sh, a.v_st, a.Tk, a.hd, rows, sK,
                 sV, tid);
  __syncthreads();
  // no barrier follows: a wavefront without a query tile leaves, one with several (the tiles past
  // what the grid covers at once, e.g. the 257th token of a 256-token-wide grid) loops
  for (; q0 < a.Tq; q0 += q_step) {
  const int qi = q0 + (lane & 31);
  float16_t oacc[NO];
#pragma unroll
  for (int o = 0; o < NO; ++o)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[o][r] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int k_end = a.causal ? min(a.Tk, min(q0 + 31, a.Tq - 1) + shift + 1) : a.Tk;
  for (int k0 = 0; k0 < k_end; k0 += 32) {
    float16_t s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const uint4 kf = *(const uint4*)(sK + (k0 + (lane & 31)) * LD + c * 16 + (lane >> 5) * 8);
      s = M32<DT>::run(kf, qf[c], s);
    }
    const bool masked = (k0 + 32 > a.Tk) || (a.causal && k0 + 31 > q0 + shift);
    float mx = m;
    if (masked) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kj = k0 + acc_row(r, lane);
        const bool ok = kj < a.Tk && (!a.causal || kj <= qi + shift);
        s[r] = ok ? s[r] : -INFINITY;
        mx = fmaxf(mx, s[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const bool dead = (mx == -INFINITY);
    const float moff = dead ? 0.f : -mx * sc;
    const float alpha = dead ? 1.f : __builtin_amdgcn_exp2f((m - mx) * sc);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float p = __builtin_amdgcn_exp2f(fmaf(s[r], sc, moff));
      s[r] = p;
      psum += p;
    }
    l = l * alpha + psum;
    m = mx;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int o = 0; o < NO; ++o)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[o][r] *= alpha;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint4 pf = pack8<DT>(s, 8 * j);
#pragma unroll
      for (int o = 0; o < NO; ++o) oacc[o] = M32<DT>::run(frag_tr<LD>(sV, k0 + 16 * j, o * 32, lane), pf, oacc[o]);
    }
  }
  l += __shfl_xor(l, 32, 64);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (qi < a.Tq) {
    uint16_t* O = a.out + b * a.o_sb + h * a.o_sh + (int64_t)qi * a.o_st;
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int h0 = o * 32 + 8 * g + 4 * (lane >> 5);
        if (h0 < a.hd)
          *(uint2*)(O + h0) = make_uint2(M32<DT>::pack(oacc[o][4 * g] * inv, oacc[o][4 * g + 1] * inv),
                                         M32<DT>::pack(oacc[o][4 * g + 2] * inv, oacc[o][4 * g + 3] * inv));
      }
    if ((lane >> 5) == 0) a.lse[((int64_t)bh) * a.Tq + qi] = (l > 0.f) ? (m * sc + log2f(l)) / LOG2E : -INFINITY;
  }
  if (q0 + q_step < a.Tq) {
#pragma unroll
    for (int c = 0; c < NC; ++c)
      qf[c] = load_row8(Q, a.q_st, q0 + q_step + (lane & 31), a.Tq, c * 16 + (lane >> 5) * 8, a.hd);
  }
  }
}

// dQ (and delta = rowsum(dO * O), which the dK/dV kernel launched after this one reads)
template <int DT, int HD, int NT>
__global__ __launch_bounds__(NT) void attn_dq_short_kernel(const AttnArgs a, float* delta_out, int rows) {
  constexpr int NC = HD / 16, NO = HD / 32, LD = HD + 8;
  extern __shared__ __align__(16) uint16_t smem[];
  uint16_t* sK = smem;
  uint16_t* sV = smem + rows * LD;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const int q_step = (int)gridDim.x * (NT / 2);
  int q0 = blockIdx.x * (NT / 2) + wave * 32;
  const uint16_t* Q = a.q + b * a.q_sb + h * a.q_sh;
  const uint16_t* DO = a.d_o + b * a.do_sb + h * a.do_sh;
  const uint16_t* OO = a.o + b * a.o_sb + h * a.o_sh;
  const float sc = a.scale * LOG2E;
  const int shift = a.Tk - a.Tq;

  uint4 qf[NC], dof[NC];
  float dlt, lse2;
  // this lane's query row of the tile at `qs`: Q, dO, delta (also written out) and the row's lse
  auto load_rows = [&](int qs) {
    const int qr = qs + (lane & 31);
    dlt = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int h0 = c * 16 + (lane >> 5) * 8;
      qf[c] = load_row8(Q, a.q_st, qr, a.Tq, h0, a.hd);
      dof[c] = load_row8(DO, a.do_st, qr, a.Tq, h0, a.hd);
      const uint4 of = load_row8(OO, a.o_st, qr, a.Tq, h0, a.hd);
      float x[8], y[8];
      unpack8<DT>(dof[c], x);
      unpack8<DT>(of, y);
#pragma unroll
      for (int k = 0; k < 8; ++k) dlt += x[k] * y[k];
    }
    dlt += __shfl_xor(dlt, 32, 64);
    if (qr < a.Tq && (lane >> 5) == 0) delta_out[(int64_t)bh * a.Tq + qr] = dlt;
    lse2 = qr < a.Tq ? a.lse[(int64_t)bh * a.Tq + qr] * LOG2E : INFINITY;
  };
  load_rows(q0);   // the first tile's rows are requested before the head is loaded
  load_heads<HD, NT>(a.k + b * a.k_sb + h * a.k_sh, a.k_st, a.v + b * a.v_sb + h * a.v_sh, a.v_st, a.Tk, a.hd, rows, sK,
                 sV, tid);
  __syncthreads();
  // no barrier follows: a wavefront without a query tile leaves, one with several loops
  for (; q0 < a.Tq; q0 += q_step) {
  const int qi = q0 + (lane & 31);
  const bool qok = qi < a.Tq;
  float16_t acc[NO];
#pragma unroll
  for (int o = 0; o < NO; ++o)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[o][r] = 0.f;
  const int k_end = a.causal ? min(a.Tk, min(q0 + 31, a.Tq - 1) + shift + 1) : a.Tk;
  for (int k0 = 0; k0 < k_end; k0 += 32) {
    float16_t s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int off = (k0 + (lane & 31)) * LD + c * 16 + (lane >> 5) * 8;
      s = M32<DT>::run(*(const uint4*)(sK + off), qf[c], s);
      dp = M32<DT>::run(*(const uint4*)(sV + off), dof[c], dp);
    }
    const bool masked = (k0 + 32 > a.Tk) || (a.causal && k0 + 31 > q0 + shift);
    if (masked) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kj = k0 + acc_row(r, lane);
        const bool ok = kj < a.Tk && (!a.causal || kj <= qi + shift);
        const float p = ok ? __builtin_amdgcn_exp2f(s[r] * sc - lse2) : 0.f;
        s[r] = p * (dp[r] - dlt);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = __builtin_amdgcn_exp2f(s[r] * sc - lse2) * (dp[r] - dlt);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint4 dsf = pack8<DT>(s, 8 * j);
#pragma unroll
      for (int o = 0; o < NO; ++o) acc[o] = M32<DT>::run(frag_tr<LD>(sK, k0 + 16 * j, o * 32, lane), dsf, acc[o]);
    }
  }
  if (qok) {
    uint16_t* DQ = a.dq + b * a.dq_sb + h * a.dq_sh + (int64_t)qi * a.dq_st;
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int h0 = o * 32 + 8 * g + 4 * (lane >> 5);
        if (h0 < a.hd)
          *(uint2*)(DQ + h0) = make_uint2(M32<DT>::pack(acc[o][4 * g] * a.scale, acc[o][4 * g + 1] * a.scale),
                                          M32<DT>::pack(acc[o][4 * g + 2] * a.scale, acc[o][4 * g + 3] * a.scale));
      }
  }
  if (q0 + q_step < a.Tq) load_rows(q0 + q_step);
  }
}

// dK/dV: workgroup = NT / 2 keys, wavefront = 32 of them; queries in steps of 32
template <int DT, int HD, int NT>
__global__ __launch_bounds__(NT) void attn_dkv_short_kernel(const AttnArgs a, int rows) {
  constexpr int NC = HD / 16, NO = HD / 32, LD = HD + 8;
  extern __shared__ __align__(16) uint16_t smem[];
  uint16_t* sQ = smem;
  uint16_t* sDO = smem + rows * LD;
  float* sLse = (float*)(smem + 2 * rows * LD);
  float* sDelta = sLse + rows;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const int k_step = (int)gridDim.x * (NT / 2);
  int kw0 = blockIdx.x * (NT / 2) + wave * 32;
  const uint16_t* K = a.k + b * a.k_sb + h * a.k_sh;
  const uint16_t* V = a.v + b * a.v_sb + h * a.v_sh;
  const float sc = a.scale * LOG2E;
  const int shift = a.Tk - a.Tq;

  uint4 kf[NC], vf[NC];
  auto load_rows = [&](int ks) {   // this lane's key row of the tile at `ks`
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      kf[c] = load_row8(K, a.k_st, ks + (lane & 31), a.Tk, c * 16 + (lane >> 5) * 8, a.hd);
      vf[c] = load_row8(V, a.v_st, ks + (lane & 31), a.Tk, c * 16 + (lane >> 5) * 8, a.hd);
    }
  };
  load_rows(kw0);   // the first tile's rows are requested before the head is loaded
  for (int i = tid; i < rows; i += NT) {
    // rows past the end: Q and dO rows are zero, lse = +inf makes their P exactly zero
    sLse[i] = i < a.Tq ? a.lse[(int64_t)bh * a.Tq + i] * LOG2E : INFINITY;
    sDelta[i] = i < a.Tq ? a.delta[(int64_t)bh * a.Tq + i] : 0.f;
  }
  load_heads<HD, NT>(a.q + b * a.q_sb + h * a.q_sh, a.q_st, a.d_o + b * a.do_sb + h * a.do_sh, a.do_st, a.Tq, a.hd, rows,
                 sQ, sDO, tid);
  __syncthreads();
  // no barrier follows: a wavefront without a key tile leaves, one with several loops
  for (; kw0 < a.Tk; kw0 += k_step) {
  const int kj = kw0 + (lane & 31);
  const bool kok = kj < a.Tk;
  float16_t dk[NO], dv[NO];
#pragma unroll
  for (int o = 0; o < NO; ++o)
#pragma unroll
    for (int r = 0; r < 16; ++r) dk[o][r] = dv[o][r] = 0.f;
  int q_begin = 0;
  if (a.causal) q_begin = max(0, kw0 - shift) / 32 * 32;   // queries i with i + shift >= kw0 see this wavefront's keys
  for (int q0 = q_begin; q0 < a.Tq; q0 += 32) {
    const bool masked = a.causal && (kw0 + 31 > q0 + shift);
    float16_t s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int off = (q0 + (lane & 31)) * LD + c * 16 + (lane >> 5) * 8;
      s = M32<DT>::run(*(const uint4*)(sQ + off), kf[c], s);
      dp = M32<DT>::run(*(const uint4*)(sDO + off), vf[c], dp);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int ql = q0 + acc_row(r, lane);
      float p = __builtin_amdgcn_exp2f(s[r] * sc - sLse[ql]);
      if (masked && kj > ql + shift) p = 0.f;
      s[r] = p;
      dp[r] = p * (dp[r] - sDelta[ql]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint4 pf = pack8<DT>(s, 8 * j);
      const uint4 dsf = pack8<DT>(dp, 8 * j);
#pragma unroll
      for (int o = 0; o < NO; ++o) {
        dv[o] = M32<DT>::run(frag_tr<LD>(sDO, q0 + 16 * j, o * 32, lane), pf, dv[o]);
        dk[o] = M32<DT>::run(frag_tr<LD>(sQ, q0 + 16 * j, o * 32, lane), dsf, dk[o]);
      }
    }
  }
  if (kok) {
    uint16_t* DK = a.dk + b * a.dk_sb + h * a.dk_sh + (int64_t)kj * a.dk_st;
    uint16_t* DV = a.dv + b * a.dv_sb + h * a.dv_sh + (int64_t)kj * a.dv_st;
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int h0 = o * 32 + 8 * g + 4 * (lane >> 5);
        if (h0 < a.hd) {
          *(uint2*)(DK + h0) = make_uint2(M32<DT>::pack(dk[o][4 * g] * a.scale, dk[o][4 * g + 1] * a.scale),
                                          M32<DT>::pack(dk[o][4 * g + 2] * a.scale, dk[o][4 * g + 3] * a.scale));
          *(uint2*)(DV + h0) = make_uint2(M32<DT>::pack(dv[o][4 * g], dv[o][4 * g + 1]),
                                          M32<DT>::pack(dv[o][4 * g + 2], dv[o][4 * g + 3]));
        }
      }
  }
  if (kw0 + k_step < a.Tk) load_rows(kw0 + k_step);
  }
}

// dQ, dK and dV of one head in ONE workgroup of eight wavefronts (heads of up to 256 queries and 256
// keys, head dim <= 64): Q, dO, K and V are loaded into LDS once (4 x 32 KB at 197 tokens), every
// wavefront first forms delta and dQ for its 32 queries (sweeping the keys), then, after one barrier,
// dK and dV for its 32 keys (sweeping the queries); against the two-kernel form this saves a launch and
// one load of the head.  Same arithmetic, in the same order, as attn_dq_short_kernel and
// attn_dkv_short_kernel.
template <int DT, int HD>
__global__ __launch_bounds__(512) void attn_bwd_short_fused_kernel(const AttnArgs a, float* delta_out, int rows_q, int rows_k) {
  constexpr int NC = HD / 16, NO = HD / 32, LD = HD + 8, NT = 512;
  extern __shared__ __align__(16) uint16_t smem[];
  uint16_t* sK = smem;
  uint16_t* sV = sK + rows_k * LD;
  uint16_t* sQ = sV + rows_k * LD;
  uint16_t* sDO = sQ + rows_q * LD;
  float* sLse = (float*)(sDO + rows_q * LD);
  float* sDelta = sLse + rows_q;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const uint16_t* OO = a.o + b * a.o_sb + h * a.o_sh;
  const float sc = a.scale * LOG2E;
  const int shift = a.Tk - a.Tq;

  // delta = rowsum(dO * O) and lse of this lane's query row: requested before the head is loaded
  const int q0 = wave * 32, qi = q0 + (lane & 31);
  const bool qok = qi < a.Tq;
  const uint16_t* DOg = a.d_o + b * a.do_sb + h * a.do_sh;
  float dlt = 0.f;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int h0 = c * 16 + (lane >> 5) * 8;
    const uint4 dof = load_row8(DOg, a.do_st, qi, a.Tq, h0, a.hd);
    const uint4 of = load_row8(OO, a.o_st, qi, a.Tq, h0, a.hd);
    float x[8], y[8];
    unpack8<DT>(dof, x);
    unpack8<DT>(of, y);
#pragma unroll
    for (int k = 0; k < 8; ++k) dlt += x[k] * y[k];
  }
  dlt += __shfl_xor(dlt, 32, 64);
  const float lse2 = qok ? a.lse[(int64_t)bh * a.Tq + qi] * LOG2E : INFINITY;
  load_heads<HD, NT>(a.k + b * a.k_sb + h * a.k_sh, a.k_st, a.v + b * a.v_sb + h * a.v_sh, a.v_st, a.Tk, a.hd, rows_k, sK,
                     sV, tid);
  load_heads<HD, NT>(a.q + b * a.q_sb + h * a.q_sh, a.q_st, DOg, a.do_st, a.Tq, a.hd, rows_q, sQ, sDO, tid);
  if (q0 < rows_q && (lane >> 5) == 0) {
    // rows past the end: Q and dO rows are zero, lse = +inf makes their P exactly zero
    sLse[qi] = lse2;
    sDelta[qi] = qok ? dlt : 0.f;
    if (qok) delta_out[(int64_t)bh * a.Tq + qi] = dlt;
  }
  __syncthreads();

  // ---- dQ for queries q0 .. q0+31
  if (q0 < a.Tq) {
    uint4 qf[NC], dof[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int off = qi * LD + c * 16 + (lane >> 5) * 8;
      qf[c] = *(const uint4*)(sQ + off);
      dof[c] = *(const uint4*)(sDO + off);
    }
    float16_t acc[NO];
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[o][r] = 0.f;
    const int k_end = a.causal ? min(a.Tk, min(q0 + 31, a.Tq - 1) + shift + 1) : a.Tk;
    for (int k0 = 0; k0 < k_end; k0 += 32) {
      float16_t s, dp;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int off = (k0 + (lane & 31)) * LD + c * 16 + (lane >> 5) * 8;
        s = M32<DT>::run(*(const uint4*)(sK + off), qf[c], s);
        dp = M32<DT>::run(*(const uint4*)(sV + off), dof[c], dp);
      }
      const bool masked = (k0 + 32 > a.Tk) || (a.causal && k0 + 31 > q0 + shift);
      if (masked) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kj = k0 + acc_row(r, lane);
          const bool ok = kj < a.Tk && (!a.causal || kj <= qi + shift);
          const float p = ok ? __builtin_amdgcn_exp2f(s[r] * sc - lse2) : 0.f;
          s[r] = p * (dp[r] - dlt);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = __builtin_amdgcn_exp2f(s[r] * sc - lse2) * (dp[r] - dlt);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint4 dsf = pack8<DT>(s, 8 * j);
#pragma unroll
        for (int o = 0; o < NO; ++o) acc[o] = M32<DT>::run(frag_tr<LD>(sK, k0 + 16 * j, o * 32, lane), dsf, acc[o]);
      }
    }
    if (qok) {
      uint16_t* DQ = a.dq + b * a.dq_sb + h * a.dq_sh + (int64_t)qi * a.dq_st;
#pragma unroll
      for (int o = 0; o < NO; ++o)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int h0 = o * 32 + 8 * g + 4 * (lane >> 5);
          if (h0 < a.hd)
            *(uint2*)(DQ + h0) = make_uint2(M32<DT>::pack(acc[o][4 * g] * a.scale, acc[o][4 * g + 1] * a.scale),
                                            M32<DT>::pack(acc[o][4 * g + 2] * a.scale, acc[o][4 * g + 3] * a.scale));
        }
    }
  }

  // ---- dK, dV for keys kw0 .. kw0+31 (sLse / sDelta were complete at the barrier above)
  const int kw0 = wave * 32, kj = kw0 + (lane & 31);
  if (kw0 >= a.Tk) return;
  const bool kok = kj < a.Tk;
  uint4 kf[NC], vf[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int off = kj * LD + c * 16 + (lane >> 5) * 8;   // rows up to rows_k are in LDS (zero past Tk)
    kf[c] = *(const uint4*)(sK + off);
    vf[c] = *(const uint4*)(sV + off);
  }
  float16_t dk[NO], dv[NO];
#pragma unroll
  for (int o = 0; o < NO; ++o)
#pragma unroll
    for (int r = 0; r < 16; ++r) dk[o][r] = dv[o][r] = 0.f;
  int q_begin = 0;
  if (a.causal) q_begin = max(0, kw0 - shift) / 32 * 32;
  for (int qs = q_begin; qs < a.Tq; qs += 32) {
    const bool masked = a.causal && (kw0 + 31 > qs + shift);
    float16_t s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int off = (qs + (lane & 31)) * LD + c * 16 + (lane >> 5) * 8;
      s = M32<DT>::run(*(const uint4*)(sQ + off), kf[c], s);
      dp = M32<DT>::run(*(const uint4*)(sDO + off), vf[c], dp);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int ql = qs + acc_row(r, lane);
      float p = __builtin_amdgcn_exp2f(s[r] * sc - sLse[ql]);
      if (masked && kj > ql + shift) p = 0.f;
      s[r] = p;
      dp[r] = p * (dp[r] - sDelta[ql]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint4 pf = pack8<DT>(s, 8 * j);
      const uint4 dsf = pack8<DT>(dp, 8 * j);
#pragma unroll
      for (int o = 0; o < NO; ++o) {
        dv[o] = M32<DT>::run(frag_tr<LD>(sDO, qs + 16 * j, o * 32, lane), pf, dv[o]);
        dk[o] = M32<DT>::run(frag_tr<LD>(sQ, qs + 16 * j, o * 32, lane), dsf, dk[o]);
      }
    }
  }
  if (kok) {
    uint16_t* DK = a.dk + b * a.dk_sb + h * a.dk_sh + (int64_t)kj * a.dk_st;
    uint16_t* DV = a.dv + b * a.dv_sb + h * a.dv_sh + (int64_t)kj * a.dv_st;
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int h0 = o * 32 + 8 * g + 4 * (lane >> 5);
        if (h0 < a.hd) {
          *(uint2*)(DK + h0) = make_uint2(M32<DT>::pack(dk[o][4 * g] * a.scale, dk[o][4 * g + 1] * a.scale),
                                          M32<DT>::pack(dk[o][4 * g + 2] * a.scale, dk[o][4 * g + 3] * a.scale));
          *(uint2*)(DV + h0) = make_uint2(M32<DT>::pack(dv[o][4 * g], dv[o][4 * g + 1]),
                                          M32<DT>::pack(dv[o][4 * g + 2], dv[o][4 * g + 3]));
        }
      }
  }
}

bool strides_ok(const void* p, int64_t sb, int64_t sh, int64_t st) {
  return pf_aligned(p, 16) && sb % 8 == 0 && sh % 8 == 0 && st % 8 == 0;
}

int check_common(const pf_attn_desc* d, const char* name) {
  PF_REQUIRE(d != nullptr, "%s: null descriptor", name);
  PF_REQUIRE(d->dtype == PF_F16 || d->dtype == PF_BF16, "%s: dtype must be fp16 or bf16", name);
  PF_REQUIRE(d->B > 0 && d->H > 0 && d->Tq > 0 && d->Tk > 0 && d->hd > 0, "%s: bad shape", name);
  if (d->hd % 8 != 0 || d->hd > 96) {
    pf_set_error("%s: head dim %d is not supported by the fused kernels (multiple of 8, <= 96)", name, d->hd);
    return PF_ERR_UNSUPPORTED;
  }
  PF_REQUIRE((int64_t)d->B * d->H <= 65535, "%s: B*H exceeds 65535", name);
  PF_REQUIRE(d->q && d->k && d->v && d->lse, "%s: null operand", name);
  PF_REQUIRE(strides_ok(d->q, d->q_sb, d->q_sh, d->q_st) && strides_ok(d->k, d->k_sb, d->k_sh, d->k_st) &&
                 strides_ok(d->v, d->v_sb, d->v_sh, d->v_st),
             "%s: q/k/v must be 16-byte aligned with strides that are multiples of 8", name);
  if (d->causal) PF_REQUIRE(d->Tk >= d->Tq, "%s: causal attention needs Tk >= Tq", name);
  return PF_OK;
}

AttnArgs make_args(const pf_attn_desc* d) {
  AttnArgs a;
  a.q = (const uint16_t*)d->q; a.k = (const uint16_t*)d->k; a.v = (const uint16_t*)d->v;
  a.o = (const uint16_t*)d->o; a.d_o = (const uint16_t*)d->d_o; a.out = (uint16_t*)d->o;
  a.dq = (uint16_t*)d->dq; a.dk = (uint16_t*)d->dk; a.dv = (uint16_t*)d->dv;
  a.lse = d->lse; a.delta = d->delta;
  a.q_sb = d->q_sb; a.q_sh = d->q_sh; a.q_st = d->q_st; a.k_sb = d->k_sb; a.k_sh = d->k_sh; a.k_st = d->k_st;
  a.v_sb = d->v_sb; a.v_sh = d->v_sh; a.v_st = d->v_st; a.o_sb = d->o_sb; a.o_sh = d->o_sh; a.o_st = d->o_st;
  a.do_sb = d->do_sb; a.do_sh = d->do_sh; a.do_st = d->do_st; a.dq_sb = d->dq_sb; a.dq_sh = d->dq_sh;
  a.dq_st = d->dq_st; a.dk_sb = d->dk_sb; a.dk_sh = d->dk_sh; a.dk_st = d->dk_st; a.dv_sb = d->dv_sb;
  a.dv_sh = d->dv_sh; a.dv_st = d->dv_st;
  a.B = d->B; a.H = d->H; a.Tq = d->Tq; a.Tk = d->Tk; a.hd = d->hd; a.causal = d->causal ? 1 : 0;
  a.scale = d->scale;
  return a;
}

}  // namespace

// Launch of a short-sequence kernel with `lds` bytes of dynamic LDS (above 64 KB the kernel is
// opted in once per kernel and device).
template <typename K, typename... Args>
int launch_short(K kern, dim3 grid, int threads, size_t lds, hipStream_t st, Args... args) {
  if (lds > 64 * 1024) {
    static std::mutex mu;
    static std::set<std::pair<const void*, int>> raised;   // instantiations share this function's type
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    std::lock_guard<std::mutex> lock(mu);
    if (!raised.count({(const void*)kern, dev})) {
      const hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (e != hipSuccess) {
        pf_set_error("pf_attention: cannot raise dynamic LDS: %s", hipGetErrorString(e));
        return PF_ERR_HIP;
      }
      raised.insert({(const void*)kern, dev});
    }
  }
  hipLaunchKernelGGL(kern, grid, dim3((unsigned)threads), lds, st, args...);
  return PF_OK;
}

// T: tokens along the axis the workgroups divide (queries, or keys for dK/dV), in tiles of 32 per
// wavefront.  A head of more than 128 tokens takes ONE workgroup of eight wavefronts (its two LDS
// operands are fetched once; the tiles past the eighth, e.g. the 257th token's, are a second pass of
// the first wavefronts).  NT96: workgroup size for head dims above 64, 512 where the kernel's
// registers allow two wavefronts per SIMD (forward, dQ), else 256: then every workgroup takes four
// tiles and a remainder of one or two tiles becomes a second pass instead of a workgroup (and a
// load of the whole head) of its own.
#define PF_ATTN_SHORT(KERNEL, NT96, rc, T, BH, lds, st, dt, hd, ...)                                            \
  do {                                                                                                         \
    const int tiles_ = ((T) + 31) / 32;                                                                        \
    const bool w64_ = (hd) <= 64 && (T) > 128, w96_ = (hd) > 64 && (NT96) == 512 && (T) > 128;                  \
    const int gx_ = (w64_ || w96_) ? 1 : ((tiles_ + 1) / 4 > 1 ? (tiles_ + 1) / 4 : 1);                         \
    const dim3 grid_((unsigned)gx_, (unsigned)(BH));                                                           \
    if (dt == PF_F16) {                                                                                        \
      if (w64_) rc = launch_short(KERNEL<PF_F16, 64, 512>, grid_, 512, (lds)(64), st, __VA_ARGS__);             \
      else if (hd <= 64) rc = launch_short(KERNEL<PF_F16, 64, 256>, grid_, 256, (lds)(64), st, __VA_ARGS__);    \
      else if (w96_) rc = launch_short(KERNEL<PF_F16, 96, NT96>, grid_, NT96, (lds)(96), st, __VA_ARGS__);      \
      else rc = launch_short(KERNEL<PF_F16, 96, 256>, grid_, 256, (lds)(96), st, __VA_ARGS__);                  \
    } else {                                                                                                   \
      if (w64_) rc = launch_short(KERNEL<PF_BF16, 64, 512>, grid_, 512, (lds)(64), st, __VA_ARGS__);            \
      else if (hd <= 64) rc = launch_short(KERNEL<PF_BF16, 64, 256>, grid_, 256, (lds)(64), st, __VA_ARGS__);   \
      else if (w96_) rc = launch_short(KERNEL<PF_BF16, 96, NT96>, grid_, NT96, (lds)(96), st, __VA_ARGS__);     \
      else rc = launch_short(KERNEL<PF_BF16, 96, 256>, grid_, 256, (lds)(96), st, __VA_ARGS__);                 \
    }                                                                                                          \
  } while (0)

#define PF_ATTN_DISPATCH(KERNEL, grid, st, a, dt, hd)                                          \
  do {                                                                                         \
    if (dt == PF_F16) {                                                                        \
      if (hd <= 64) hipLaunchKernelGGL((KERNEL<PF_F16, 64>), grid, dim3(256), 0, st, a);       \
      else hipLaunchKernelGGL((KERNEL<PF_F16, 96>), grid, dim3(256), 0, st, a);                \
    } else {                                                                                   \
      if (hd <= 64) hipLaunchKernelGGL((KERNEL<PF_BF16, 64>), grid, dim3(256), 0, st, a);      \
      else hipLaunchKernelGGL((KERNEL<PF_BF16, 96>), grid, dim3(256), 0, st, a);               \
    }                                                                                          \
  } while (0)

extern "C" int pf_attention_fwd(const pf_attn_desc* d, void* stream) {
  int rc = check_common(d, "pf_attention_fwd");
  if (rc != PF_OK) return rc;
  PF_REQUIRE(d->o && strides_ok(d->o, d->o_sb, d->o_sh, d->o_st) && d->o_st % 4 == 0,
             "pf_attention_fwd: bad output operand");
  AttnArgs a = make_args(d);
  const dim3 grid((unsigned)((d->Tq + 127) / 128), (unsigned)(d->B * d->H));
  if (d->Tq <= SHORT_T && d->Tk <= SHORT_T) {
    const int rows = (d->Tk + 31) / 32 * 32;
    auto lds = [rows](int HD) { return (size_t)2 * rows * (HD + 8) * 2; };
    PF_ATTN_SHORT(attn_fwd_short_kernel, 512, rc, d->Tq, d->B * d->H, lds, (hipStream_t)stream, d->dtype, d->hd, a, rows);
    if (rc != PF_OK) return rc;
  } else {
    PF_ATTN_DISPATCH(attn_fwd_kernel, grid, (hipStream_t)stream, a, d->dtype, d->hd);
  }
  PF_CHECK_LAUNCH("pf_attention_fwd");
  return PF_OK;
}

extern "C" int pf_attention_bwd(const pf_attn_desc* d, void* stream) {
  int rc = check_common(d, "pf_attention_bwd");
  if (rc != PF_OK) return rc;
  PF_REQUIRE(d->o && d->d_o && d->dq && d->dk && d->dv && d->delta, "pf_attention_bwd: null operand");
  PF_REQUIRE(strides_ok(d->o, d->o_sb, d->o_sh, d->o_st) && strides_ok(d->d_o, d->do_sb, d->do_sh, d->do_st),
             "pf_attention_bwd: o/dO must be 16-byte aligned with strides that are multiples of 8");
  PF_REQUIRE(pf_aligned(d->dq, 8) && pf_aligned(d->dk, 8) && pf_aligned(d->dv, 8) && d->dq_sb % 4 == 0 &&
                 d->dq_sh % 4 == 0 && d->dq_st % 4 == 0 && d->dk_sb % 4 == 0 && d->dk_sh % 4 == 0 &&
                 d->dk_st % 4 == 0 && d->dv_sb % 4 == 0 && d->dv_sh % 4 == 0 && d->dv_st % 4 == 0,
             "pf_attention_bwd: gradient operands must be 8-byte aligned with strides that are multiples of 4");
  AttnArgs a = make_args(d);
  hipStream_t st = (hipStream_t)stream;
  AttnArgs ad = a;
  if (d->dtype == PF_BF16) ad.causal |= 0x100;  // dtype flag for the delta kernel
  const dim3 gq((unsigned)((d->Tq + 127) / 128), (unsigned)(d->B * d->H));
  const dim3 gk((unsigned)((d->Tk + 127) / 128), (unsigned)(d->B * d->H));
  if (d->Tq <= SHORT_T && d->Tk <= SHORT_T) {
    const int rows_k = (d->Tk + 31) / 32 * 32, rows_q = (d->Tq + 31) / 32 * 32;
    if (d->hd <= 64 && d->Tq <= 256 && d->Tk <= 256 && (d->Tq > 128 || d->Tk > 128)) {
      // one workgroup per head forms dQ, dK and dV from a single load of the head
      const size_t lds = (size_t)2 * (rows_k + rows_q) * (64 + 8) * 2 + (size_t)rows_q * 8;
      const dim3 gf(1, (unsigned)(d->B * d->H));
      if (d->dtype == PF_F16) rc = launch_short(attn_bwd_short_fused_kernel<PF_F16, 64>, gf, 512, lds, st, a, d->delta, rows_q, rows_k);
      else rc = launch_short(attn_bwd_short_fused_kernel<PF_BF16, 64>, gf, 512, lds, st, a, d->delta, rows_q, rows_k);
      if (rc != PF_OK) return rc;
      PF_CHECK_LAUNCH("pf_attention_bwd");
      return PF_OK;
    }
    // dQ first: it also leaves delta = rowsum(dO * O) for the dK/dV kernel
    auto lds_q = [rows_k](int HD) { return (size_t)2 * rows_k * (HD + 8) * 2; };
    auto lds_k = [rows_q](int HD) { return (size_t)2 * rows_q * (HD + 8) * 2 + (size_t)rows_q * 8; };
    PF_ATTN_SHORT(attn_dq_short_kernel, 512, rc, d->Tq, d->B * d->H, lds_q, st, d->dtype, d->hd, a, d->delta, rows_k);
    if (rc != PF_OK) return rc;
    PF_ATTN_SHORT(attn_dkv_short_kernel, 256, rc, d->Tk, d->B * d->H, lds_k, st, d->dtype, d->hd, a, rows_q);
    if (rc != PF_OK) return rc;
    PF_CHECK_LAUNCH("pf_attention_bwd");
    return PF_OK;
  }
  const int64_t rows = (int64_t)d->B * d->H * d->Tq;
  hipLaunchKernelGGL(attn_delta_kernel, dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, st, ad, d->delta);
  // few keys, many queries (cross attention to a short context): split each key tile's query sweep
  // over the four wavefronts of a workgroup
  if ((int64_t)gk.x * gk.y < 200 && d->Tq >= 256) {
    const dim3 gs((unsigned)((d->Tk + 31) / 32), (unsigned)(d->B * d->H));
    if (d->dtype == PF_F16) {
      if (d->hd <= 64) hipLaunchKernelGGL((attn_dkv_kernel<PF_F16, 64, true>), gs, dim3(256), 0, st, a);
      else hipLaunchKernelGGL((attn_dkv_kernel<PF_F16, 96, true>), gs, dim3(256), 0, st, a);
    } else {
      if (d->hd <= 64) hipLaunchKernelGGL((attn_dkv_kernel<PF_BF16, 64, true>), gs, dim3(256), 0, st, a);
      else hipLaunchKernelGGL((attn_dkv_kernel<PF_BF16, 96, true>), gs, dim3(256), 0, st, a);
    }
  } else {
    PF_ATTN_DISPATCH(attn_dkv_kernel, gk, st, a, d->dtype, d->hd);
  }
  PF_ATTN_DISPATCH(attn_dq_kernel, gq, st, a, d->dtype, d->hd);
  PF_CHECK_LAUNCH("pf_attention_bwd");
  return PF_OK;
}
