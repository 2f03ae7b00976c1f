// Shared device/host helpers for the pfeife_amd HIP kernels (gfx950 / CDNA4 only).
//
// Every kernel in this library is launched on a caller-supplied stream, never
// allocates, never synchronises the host, and returns an int status through the
// C ABI (0 = ok, negative = error, text via pf_last_error()).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/pfeife_hip.h"

#define PF_WAVE 64

typedef _Float16 pf_half;
typedef __bf16 pf_bf16;

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------------------
// host-side error plumbing
// ---------------------------------------------------------------------------
void pf_set_error(const char* fmt, ...);

#define PF_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      pf_set_error(__VA_ARGS__);         \
      return PF_ERR_INVALID;             \
    }                                    \
  } while (0)

#define PF_CHECK_LAUNCH(name)                                            \
  do {                                                                   \
    hipError_t e__ = hipGetLastError();                                  \
    if (e__ != hipSuccess) {                                             \
      pf_set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
      return PF_ERR_HIP;                                                 \
    }                                                                    \
  } while (0)

static inline int pf_dtype_size(int dt) {
  switch (dt) {
    case PF_F32: return 4;
    case PF_F16: return 2;
    case PF_BF16: return 2;
    case PF_I64: return 8;
    case PF_I32: return 4;
    case PF_U8: return 1;
    default: return 0;
  }
}

static inline bool pf_is_float_dtype(int dt) { return dt == PF_F32 || dt == PF_F16 || dt == PF_BF16; }
static inline bool pf_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// ---------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------
#ifdef __HIPCC__

// bf16 <-> f32 with round-to-nearest-even (matches torch's .to(torch.bfloat16))
__device__ __forceinline__ float pf_bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ __forceinline__ uint16_t pf_f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float pf_f16_bits_to_f32(uint16_t b) {
  union { uint16_t u; _Float16 h; } c;
  c.u = b;
  return (float)c.h;
}
__device__ __forceinline__ uint16_t pf_f32_to_f16_bits(float f) {
  union { uint16_t u; _Float16 h; } c;
  c.h = (_Float16)f;  // v_cvt_f16_f32: round-to-nearest-even
  return c.u;
}

// two fp32 -> one packed pair of 16-bit values (low half = first argument), round to nearest
// even: single v_cvt_pk_{bf16,f16}_f32 instructions on gfx950
typedef __bf16 pf_bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 pf_f16x2_t __attribute__((ext_vector_type(2)));
typedef float pf_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pf_pack2_bf16(float lo, float hi) {
  const pf_f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, pf_bf16x2_t));
}
__device__ __forceinline__ uint32_t pf_pack2_f16(float lo, float hi) {
  const pf_f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, pf_f16x2_t));
}

// Element codecs: T is float, pf_half tag or pf_bf16 tag. Storage of the 16-bit
// kinds is always handled as uint16_t so that no implicit arithmetic sneaks in.
template <int DT> struct Codec;
template <> struct Codec<PF_F32> {
  typedef float storage;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Codec<PF_F16> {
  typedef uint16_t storage;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return pf_f16_bits_to_f32(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = pf_f32_to_f16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return pf_f16_bits_to_f32(pf_f32_to_f16_bits(v)); }
};
template <> struct Codec<PF_BF16> {
  typedef uint16_t storage;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return pf_bf16_bits_to_f32(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = pf_f32_to_bf16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return pf_bf16_bits_to_f32(pf_f32_to_bf16_bits(v)); }
};

// runtime-dtype scalar access (used in epilogues where the branch is wave-uniform)
__device__ __forceinline__ float pf_load_as_f32(const void* p, int64_t i, int dt) {
  if (dt == PF_F32) return ((const float*)p)[i];
  if (dt == PF_F16) return pf_f16_bits_to_f32(((const uint16_t*)p)[i]);
  return pf_bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
__device__ __forceinline__ void pf_store_from_f32(void* p, int64_t i, int dt, float v) {
  if (dt == PF_F32) ((float*)p)[i] = v;
  else if (dt == PF_F16) ((uint16_t*)p)[i] = pf_f32_to_f16_bits(v);
  else ((uint16_t*)p)[i] = pf_f32_to_bf16_bits(v);
}
__device__ __forceinline__ float pf_round_to(int dt, float v) {
  if (dt == PF_F16) return pf_f16_bits_to_f32(pf_f32_to_f16_bits(v));
  if (dt == PF_BF16) return pf_bf16_bits_to_f32(pf_f32_to_bf16_bits(v));
  return v;
}

// 8-wide / 4-wide vector access: 8 consecutive elements starting at element i
// (i must be a multiple of 8 and the base 16-byte aligned for the 16-bit kinds;
// for f32 the 8 values are two 16-byte loads).
template <int DT> struct Vec8;
template <> struct Vec8<PF_F32> {
  static __device__ __forceinline__ void load(const void* p, int64_t i, float (&v)[8]) {
    const float4* q = (const float4*)((const float*)p + i);
    float4 a = q[0], b = q[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void store(void* p, int64_t i, const float (&v)[8]) {
    float4* q = (float4*)((float*)p + i);
    q[0] = make_float4(v[0], v[1], v[2], v[3]);
    q[1] = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <> struct Vec8<PF_F16> {
  static __device__ __forceinline__ void load(const void* p, int64_t i, float (&v)[8]) {
    uint4 r = *(const uint4*)((const uint16_t*)p + i);
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = pf_f16_bits_to_f32((uint16_t)(w[k] & 0xffffu));
      v[2 * k + 1] = pf_f16_bits_to_f32((uint16_t)(w[k] >> 16));
    }
  }
  static __device__ __forceinline__ void store(void* p, int64_t i, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = pf_pack2_f16(v[2 * k], v[2 * k + 1]);
    *(uint4*)((uint16_t*)p + i) = make_uint4(w[0], w[1], w[2], w[3]);
  }
};
template <> struct Vec8<PF_BF16> {
  static __device__ __forceinline__ void load(const void* p, int64_t i, float (&v)[8]) {
    uint4 r = *(const uint4*)((const uint16_t*)p + i);
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = __uint_as_float(w[k] << 16);
      v[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(void* p, int64_t i, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = pf_pack2_bf16(v[2 * k], v[2 * k + 1]);
    *(uint4*)((uint16_t*)p + i) = make_uint4(w[0], w[1], w[2], w[3]);
  }
};

// runtime-dtype W-wide access: W == 8 takes the 16-byte vector path (index a
// multiple of 8, base 16-byte aligned), W == 1 the scalar path.
template <int W>
__device__ __forceinline__ void ld_vec(const void* p, int64_t i, int dt, float (&v)[W]) {
  if constexpr (W == 8) {
    if (dt == PF_F32) Vec8<PF_F32>::load(p, i, v);
    else if (dt == PF_F16) Vec8<PF_F16>::load(p, i, v);
    else Vec8<PF_BF16>::load(p, i, v);
  } else {
#pragma unroll
    for (int k = 0; k < W; ++k) v[k] = pf_load_as_f32(p, i + k, dt);
  }
}
template <int W>
__device__ __forceinline__ void st_vec(void* p, int64_t i, int dt, const float (&v)[W]) {
  if constexpr (W == 8) {
    if (dt == PF_F32) Vec8<PF_F32>::store(p, i, v);
    else if (dt == PF_F16) Vec8<PF_F16>::store(p, i, v);
    else Vec8<PF_BF16>::store(p, i, v);
  } else {
#pragma unroll
    for (int k = 0; k < W; ++k) pf_store_from_f32(p, i + k, dt, v[k]);
  }
}

// The same with the dtype known at compile time when DT >= 0 (W == 8): no branch around the
// access, so several of them issue back to back and wait once.  (A runtime dtype switch puts
// every access into a control-flow region of its own, and the compiler drains the memory
// counter where regions join: one memory round trip per access.)
template <int W, int DT>
__device__ __forceinline__ void ld_vec_c(const void* p, int64_t i, int dt, float (&v)[W]) {
  if constexpr (W == 8 && DT >= 0) Vec8<DT>::load(p, i, v);
  else ld_vec<W>(p, i, dt, v);
}
template <int W, int DT>
__device__ __forceinline__ void st_vec_c(void* p, int64_t i, int dt, const float (&v)[W]) {
  if constexpr (W == 8 && DT >= 0) Vec8<DT>::store(p, i, v);
  else st_vec<W>(p, i, dt, v);
}

// 64-lane wavefront reductions (butterfly; every lane ends with the result)
__device__ __forceinline__ float pf_wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, PF_WAVE);
  return v;
}
__device__ __forceinline__ float pf_wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, PF_WAVE));
  return v;
}

// Block-wide reductions for blocks of NW wavefronts; `sm` holds >= NW floats.
template <int NW>
__device__ __forceinline__ float pf_block_sum(float v, float* sm) {
  v = pf_wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) sm[w] = v;
  __syncthreads();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) r += sm[i];
  return r;
}
template <int NW>
__device__ __forceinline__ float pf_block_max(float v, float* sm) {
  v = pf_wave_max(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) sm[w] = v;
  __syncthreads();
  float r = sm[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = fmaxf(r, sm[i]);
  return r;
}

// activation math (fp32)
// erf by Abramowitz & Stegun 7.1.26 (|error| <= 1.5e-7, far below fp16/bf16 resolution and
// below what a 1e-5 relative loss tolerance can see): one reciprocal, one v_exp_f32, five FMAs.
// e2 returns exp(-u*u) for reuse by the GELU derivative.
__device__ __forceinline__ float pf_erf_fast(float u, float& e2) {
  const float au = fabsf(u);
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, au, 1.f));
  e2 = __builtin_amdgcn_exp2f(-1.4426950408889634f * au * au);
  float p = fmaf(1.061405429f, t, -1.453152027f);
  p = fmaf(p, t, 1.421413741f);
  p = fmaf(p, t, -0.284496736f);
  p = fmaf(p, t, 0.254829592f);
  const float y = 1.f - p * t * e2;
  return copysignf(y, u);
}
// GELU (erf form) without the reciprocal: the upper tail of the normal distribution is
// 1 - Phi(a) = 2^-g(a) with g a degree-5 polynomial on [0, 5.5] (weighted minimax fit; beyond 5.5 the
// tail is below 2e-8), and x * Phi(x) = x - x * tail(|x|) for x >= 0, x * tail(|x|) for x < 0.
// |error| <= 9e-7 in fp32 arithmetic over [-8, 8]: five FMAs, one v_exp_f32, a multiply, a subtract, a select.
__device__ __forceinline__ float pf_gelu_erf(float x) {
  const float a = fminf(fabsf(x), 5.5f);
  float g = fmaf(0.00049698935f, a, -0.007244379f);
  g = fmaf(g, a, 0.05221166f);
  g = fmaf(g, a, 0.45959195f);
  g = fmaf(g, a, 1.1509614f);
  g = fmaf(g, a, 1.0000144f);
  const float xq = x * __builtin_amdgcn_exp2f(-g);
  return x >= 0.f ? x - xq : xq;
}
__device__ __forceinline__ float pf_gelu_erf_grad(float x) {
  float e2;   // = exp(-x*x/2)
  const float cdf = 0.5f * (1.f + pf_erf_fast(x * 0.70710678118654752440f, e2));
  return fmaf(x * 0.39894228040143267794f, e2, cdf);
}
__device__ __forceinline__ float pf_gelu_tanh(float x) {
  const float k = 0.79788456080286535588f, c = 0.044715f;
  return 0.5f * x * (1.f + tanhf(k * (x + c * x * x * x)));
}
__device__ __forceinline__ float pf_gelu_tanh_grad(float x) {
  const float k = 0.79788456080286535588f, c = 0.044715f;
  const float u = k * (x + c * x * x * x);
  const float t = tanhf(u);
  const float du = k * (1.f + 3.f * c * x * x);
  return 0.5f * (1.f + t) + 0.5f * x * (1.f - t * t) * du;
}
__device__ __forceinline__ float pf_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float pf_silu(float x) { return x * pf_sigmoid(x); }
__device__ __forceinline__ float pf_silu_grad(float x) {
  const float s = pf_sigmoid(x);
  return s * (1.f + x * (1.f - s));
}
__device__ __forceinline__ float pf_act(int act, float x) {
  switch (act) {
    case PF_ACT_GELU: return pf_gelu_erf(x);
    case PF_ACT_GELU_TANH: return pf_gelu_tanh(x);
    case PF_ACT_SILU: return pf_silu(x);
    case PF_ACT_RELU: return x > 0.f ? x : 0.f;
    default: return x;
  }
}
__device__ __forceinline__ float pf_act_grad(int act, float x) {
  switch (act) {
    case PF_ACT_GELU: return pf_gelu_erf_grad(x);
    case PF_ACT_GELU_TANH: return pf_gelu_tanh_grad(x);
    case PF_ACT_SILU: return pf_silu_grad(x);
    case PF_ACT_RELU: return x > 0.f ? 1.f : 0.f;
    default: return 1.f;
  }
}

#endif  // __HIPCC__
