// Pieces shared by the GEMM translation units: launch geometry, the runtime-configured
// epilogue, the XCD-aware workgroup -> tile order, MFMA wrappers, raw buffer access.
#pragma once
#include <cstdlib>
#include <mutex>
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
  float* colsum_ws;
  float* nonfinite;
};

__device__ __forceinline__ Epi make_epi(const pf_gemm_desc& p) {
  Epi e;
  // (a loss scale kept on the device divides the product: read here, once per workgroup)
  e.alpha = p.unscale_by != nullptr ? p.alpha / p.unscale_by[0] : p.alpha;
  e.beta = p.beta; e.round_mid = p.round_mid; e.act = p.act; e.dact = p.dact;
  e.in_dtype = p.in_dtype; e.c_dtype = p.c_dtype; e.bias_dtype = p.bias_dtype; e.res_dtype = p.res_dtype;
  e.bias = p.bias; e.aux_out = p.aux_out; e.aux_in = p.aux_in; e.residual = p.residual; e.C = p.C;
  e.ldc = p.ldc; e.ld_aux_out = p.ld_aux_out; e.ld_aux_in = p.ld_aux_in; e.ld_res = p.ld_res;
  e.colsum_ws = p.colsum_ws;
  e.nonfinite = p.nonfinite_flag;
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
  if (e.act == PF_ACT_GELU) {   // the common case without a per-element switch
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = pf_gelu_erf(v[k]);
  } else if (e.act != PF_ACT_NONE) {
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = pf_act(e.act, v[k]);
  }
  if (e.dact != PF_ACT_NONE) {
    ld_vec<8>(e.aux_in, row * e.ld_aux_in + col, e.in_dtype, t);
    if (e.dact == PF_ACT_GELU) {
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] *= pf_gelu_erf_grad(t[k]);
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] *= pf_act_grad(e.dact, t[k]);
    }
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
__device__ __forceinline__ int gemm_tile_id(int pid, int tiles, int per_xcd) {
  const int t = (pid & 7) * per_xcd + (pid >> 3);
  return t < tiles ? t : -1;
}

// Tile id -> (tile row, tile column) in grouped order: ids walk down GROUP_M tile
// rows before moving to the next tile column, so the ~32-64 workgroups an XCD runs
// at the same time cover a compact patch of C and share their A rows and B columns
// through that XCD's L2 instead of streaming whole operands from HBM.
constexpr int GROUP_M = 8;
__device__ __forceinline__ void gemm_tile_rc(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int per_group = GROUP_M * tiles_n;
  const int group = t / per_group;
  const int first_m = group * GROUP_M;
  const int gm = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
  const int r = t - group * per_group;
  tm = first_m + r % gm;
  tn = r / gm;
}

// ---------------------------------------------------------------------------
// 16-bit MFMA kernel
// ---------------------------------------------------------------------------
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
  static __device__ __forceinline__ float16_t run8(short __attribute__((ext_vector_type(8))) a, short __attribute__((ext_vector_type(8))) b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float16_t run(uint4 a, uint4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0,
                                                  0, 0);
  }
};
template <> struct Mfma<PF_BF16> {
  static __device__ __forceinline__ float16_t run8(short __attribute__((ext_vector_type(8))) a, short __attribute__((ext_vector_type(8))) b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float16_t run(uint4 a, uint4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  }
};

inline bool epi_ptr_ok(const void* p, int64_t ld) { return p == nullptr || (pf_aligned(p, 16) && ld % 8 == 0); }
inline int epi_vec_ok(const pf_gemm_desc& d) {
  return epi_ptr_ok(d.C, d.ldc) && d.c_stride1 % 8 == 0 && d.c_stride2 % 8 == 0 &&
         (d.bias == nullptr || pf_aligned(d.bias, 16)) && epi_ptr_ok(d.aux_out, d.ld_aux_out) &&
         epi_ptr_ok(d.aux_in, d.ld_aux_in) && epi_ptr_ok(d.residual, d.ld_res);
}

// raw buffer access: a descriptor whose extent is the operand's valid byte range makes the
// hardware return zeros for (and drop stores to) anything past it
typedef int v4i_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
  const v4i_t x = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0);
  return make_uint4((uint32_t)x.x, (uint32_t)x.y, (uint32_t)x.z, (uint32_t)x.w);
}

// Tile shapes of the direct-to-LDS kernel (BM x BN; reduction depth per stage, stages; wavefronts):
//   256x256 (32 deep, 5 stages): one 128x128 block per wavefront, the least operand traffic per FLOP
//   256x128 (64 deep, 3 stages), 128x128 (64 deep, 3 stages): more workgroups for smaller outputs
//   192x256 (32 deep, 5 stages): for outputs that 256-row blocks cover badly
//   ids 1-4: four wavefronts (2 x 2); ids 7-9: the same tiles shared by EIGHT wavefronts (2 x 4,
//   two per SIMD); ids 5, 6: 128x128 and 256x128 with eight wavefronts as TWO 2 x 2 grids that
//   split every tile's reduction depth between them ("k2")
enum { PF_XT_256x256 = 1, PF_XT_256x128 = 2, PF_XT_128x128 = 3, PF_XT_192x256 = 4, PF_XT_128x128k2 = 5,
       PF_XT_256x128k2 = 6, PF_XT_256x256w8 = 7, PF_XT_128x128w8 = 8, PF_XT_256x128w8 = 9, PF_XT_COUNT = 10 };
// BM, BN, reduction depth per stage, stages, wavefront grid (rows x columns x reduction split) of each tile id
template <int XT> struct XTile;
template <> struct XTile<PF_XT_256x256> { static constexpr int BM = 256, BN = 256, BK = 32, ST = 5, WGM = 2, WGN = 2, KS = 1; };
template <> struct XTile<PF_XT_256x128> { static constexpr int BM = 256, BN = 128, BK = 64, ST = 3, WGM = 2, WGN = 2, KS = 1; };
template <> struct XTile<PF_XT_128x128> { static constexpr int BM = 128, BN = 128, BK = 64, ST = 3, WGM = 2, WGN = 2, KS = 1; };
template <> struct XTile<PF_XT_192x256> { static constexpr int BM = 192, BN = 256, BK = 32, ST = 5, WGM = 2, WGN = 2, KS = 1; };
template <> struct XTile<PF_XT_128x128k2> { static constexpr int BM = 128, BN = 128, BK = 64, ST = 3, WGM = 2, WGN = 2, KS = 2; };
template <> struct XTile<PF_XT_256x128k2> { static constexpr int BM = 256, BN = 128, BK = 64, ST = 3, WGM = 2, WGN = 2, KS = 2; };
template <> struct XTile<PF_XT_256x256w8> { static constexpr int BM = 256, BN = 256, BK = 32, ST = 5, WGM = 2, WGN = 4, KS = 1; };
template <> struct XTile<PF_XT_128x128w8> { static constexpr int BM = 128, BN = 128, BK = 64, ST = 3, WGM = 2, WGN = 4, KS = 1; };
template <> struct XTile<PF_XT_256x128w8> { static constexpr int BM = 256, BN = 128, BK = 64, ST = 3, WGM = 4, WGN = 2, KS = 1; };
inline int x_tile_bk(int xt) { return (xt == PF_XT_256x256 || xt == PF_XT_192x256 || xt == PF_XT_256x256w8) ? 32 : 64; }

// Epilogue classes with straight-line code (which operands exist, and their dtypes, fixed at
// compile time).  Everything else takes EC_GENERIC: one rolled loop with runtime switches.
enum {
  EC_GENERIC = -1,
  EC_STORE16 = 0,  // C 16-bit
  EC_STORE32 = 1,  // C fp32
  EC_ACT16 = 2,    // C 16-bit, pre-activation saved (aux_out), GELU
  EC_RES32 = 3,    // C fp32, fp32 residual added
  EC_ACC32 = 4,    // C fp32 accumulated in place (beta = 1)
  EC_DACT16 = 5,   // C 16-bit, multiplied by GELU'(aux_in)
  EC_ACC16 = 6,    // C 16-bit accumulated in place (beta = 1)
  EC_RES16 = 7,    // C 16-bit, residual of the same 16-bit dtype added (a 16-bit residual stream)
};
// Epilogue class of a problem (see the EC_* list): the straight-line classes need 16-byte
// vector access to every epilogue operand, whole 8-column groups, and 32-bit byte offsets.
inline int epi_class(const pf_gemm_desc& d, int vec_ok) {
  if (!vec_ok || d.N % 8 != 0) return EC_GENERIC;
  const int64_t lim = (1ll << 31) - 64;
  if (d.M * d.ldc * 4 >= lim) return EC_GENERIC;
  if (d.aux_out && d.M * d.ld_aux_out * 2 >= lim) return EC_GENERIC;
  if (d.aux_in && d.M * d.ld_aux_in * 2 >= lim) return EC_GENERIC;
  if (d.residual && d.M * d.ld_res * 4 >= lim) return EC_GENERIC;   // (bounds the 16-bit case too)
  const bool c16 = d.c_dtype == d.in_dtype, c32 = d.c_dtype == PF_F32;
  if (!c16 && !c32) return EC_GENERIC;
  const bool act = d.act != PF_ACT_NONE, dact = d.dact != PF_ACT_NONE, res = d.residual != nullptr, beta = d.beta != 0;
  if (act != (d.aux_out != nullptr)) return EC_GENERIC;
  const int n = (act ? 1 : 0) + (dact ? 1 : 0) + (res ? 1 : 0) + (beta ? 1 : 0);
  if (n == 0) return c16 ? EC_STORE16 : EC_STORE32;
  if (n > 1) return EC_GENERIC;
  if (act) return (c16 && d.act == PF_ACT_GELU) ? EC_ACT16 : EC_GENERIC;
  if (dact) return (c16 && d.dact == PF_ACT_GELU) ? EC_DACT16 : EC_GENERIC;
  if (res) return (c32 && d.res_dtype == PF_F32) ? EC_RES32 : ((c16 && d.res_dtype == d.in_dtype) ? EC_RES16 : EC_GENERIC);
  return c32 ? EC_ACC32 : EC_ACC16;
}

}  // namespace
