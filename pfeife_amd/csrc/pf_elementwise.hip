// HBM-bound streaming kernels: activations, gated MLP, axpby, bias add, casts,
// fills, strided copies, rotary embedding and the fp32 gradient accumulation.
// All of them move 16 bytes (8 x 16-bit) or 32 bytes (8 x fp32) per lane per
// step in a grid-stride loop sized to keep every CU busy.
#include <math.h>

#include "pf_common.h"

namespace {

constexpr int EW_BLOCK = 256;
constexpr int EW_MAX_BLOCKS = 256 * 16;  // 16 workgroups per CU is plenty of bytes in flight

inline dim3 ew_grid(int64_t work_items) {
  int64_t b = (work_items + EW_BLOCK - 1) / EW_BLOCK;
  if (b < 1) b = 1;
  if (b > EW_MAX_BLOCKS) b = EW_MAX_BLOCKS;
  return dim3((unsigned)b);
}

// F provides:  void run<W>(int64_t i)  processing W elements starting at i
template <class F>
__global__ __launch_bounds__(EW_BLOCK) void ew_kernel(F f, int64_t n, int vec) {
  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  const int64_t nv = vec ? n / 8 : 0;
  for (int64_t i = gtid; i < nv; i += gsz) f.template run<8>(i * 8);
  for (int64_t i = nv * 8 + gtid; i < n; i += gsz) f.template run<1>(i);
}

template <class F>
int ew_launch(const F& f, int64_t n, bool vec, hipStream_t st, const char* name) {
  if (n <= 0) return PF_OK;
  hipLaunchKernelGGL(ew_kernel<F>, ew_grid(vec ? (n + 7) / 8 : n), dim3(EW_BLOCK), 0, st, f, n, vec ? 1 : 0);
  PF_CHECK_LAUNCH(name);
  return PF_OK;
}

inline bool al16(const void* p) { return pf_aligned(p, 16); }

struct ActFwd {
  const void* x; void* y; int dt, act;
  template <int W> __device__ void run(int64_t i) const {
    float v[W];
    ld_vec<W>(x, i, dt, v);
#pragma unroll
    for (int k = 0; k < W; ++k) v[k] = pf_act(act, v[k]);
    st_vec<W>(y, i, dt, v);
  }
};
struct ActBwd {
  const void* dy; const void* x; void* dx; int dt, act;
  template <int W> __device__ void run(int64_t i) const {
    float g[W], v[W];
    ld_vec<W>(dy, i, dt, g);
    ld_vec<W>(x, i, dt, v);
#pragma unroll
    for (int k = 0; k < W; ++k) g[k] *= pf_act_grad(act, v[k]);
    st_vec<W>(dx, i, dt, g);
  }
};
struct Axpby {
  const void* a; const void* b; void* o; int adt, bdt, odt; float alpha, beta;
  template <int W> __device__ void run(int64_t i) const {
    float x[W], y[W];
    ld_vec<W>(a, i, adt, x);
    ld_vec<W>(b, i, bdt, y);
#pragma unroll
    for (int k = 0; k < W; ++k) x[k] = alpha * x[k] + beta * y[k];
    st_vec<W>(o, i, odt, x);
  }
};
struct Scale {  // out = alpha * a (b absent)
  const void* a; void* o; int adt, odt; float alpha;
  template <int W> __device__ void run(int64_t i) const {
    float x[W];
    ld_vec<W>(a, i, adt, x);
#pragma unroll
    for (int k = 0; k < W; ++k) x[k] *= alpha;
    st_vec<W>(o, i, odt, x);
  }
};
struct Cast {
  const void* s; void* d; int sdt, ddt;
  template <int W> __device__ void run(int64_t i) const {
    float x[W];
    ld_vec<W>(s, i, sdt, x);
    st_vec<W>(d, i, ddt, x);
  }
};
struct Fill {
  void* d; int dt; float value;
  template <int W> __device__ void run(int64_t i) const {
    float x[W];
#pragma unroll
    for (int k = 0; k < W; ++k) x[k] = value;
    st_vec<W>(d, i, dt, x);
  }
};
struct GradAcc {
  float* acc; const void* g; int gdt;
  template <int W> __device__ void run(int64_t i) const {
    float a[W], x[W];
    ld_vec<W>(acc, i, PF_F32, a);
    ld_vec<W>(g, i, gdt, x);
#pragma unroll
    for (int k = 0; k < W; ++k) a[k] += x[k];
    st_vec<W>(acc, i, PF_F32, a);
  }
};
struct BiasAdd {  // bias_len is a multiple of 8 on the vector path
  const void* x; const void* bias; void* y; int xdt, bdt, ydt; int64_t bias_len, span;
  template <int W> __device__ void run(int64_t i) const {
    float v[W], b[W];
    ld_vec<W>(x, i, xdt, v);
    // span = elements of x that share one bias row (0: every row uses bias row 0)
    ld_vec<W>(bias, (span ? (i / span) * bias_len : 0) + i % bias_len, bdt, b);
#pragma unroll
    for (int k = 0; k < W; ++k) v[k] += b[k];
    st_vec<W>(y, i, ydt, v);
  }
};

// gated MLP: rows x cols with independent row strides; index space is rows*cols
// DT: the operands' dtype when fixed at compile time (-1: read `dt` at run time).  With a fixed
// dtype the two or three loads of an element group issue back to back and wait once.
template <int DT = -1>
struct GluFwd {
  const void* gate; const void* up; void* y; int64_t ldg, ldu, ldy, cols; int dt, act;
  template <int W> __device__ void run(int64_t i) const {
    const int64_t r = i / cols, c = i % cols;
    const int edt = DT >= 0 ? DT : dt;
    float g[W], u[W];
    ld_vec_c<W, DT>(gate, r * ldg + c, dt, g);
    ld_vec_c<W, DT>(up, r * ldu + c, dt, u);
#pragma unroll
    for (int k = 0; k < W; ++k) g[k] = pf_round_to(edt, pf_act(act, g[k])) * u[k];
    st_vec_c<W, DT>(y, r * ldy + c, dt, g);
  }
};
template <int DT = -1>
struct GluBwd {
  const void* dy; const void* gate; const void* up; void* dgate; void* dup;
  int64_t lddy, ldg, ldu, lddg, lddu, cols; int dt, act;
  template <int W> __device__ void run(int64_t i) const {
    const int64_t r = i / cols, c = i % cols;
    const int edt = DT >= 0 ? DT : dt;
    float d[W], g[W], u[W], dg[W], du[W];
    ld_vec_c<W, DT>(dy, r * lddy + c, dt, d);
    ld_vec_c<W, DT>(gate, r * ldg + c, dt, g);
    ld_vec_c<W, DT>(up, r * ldu + c, dt, u);
#pragma unroll
    for (int k = 0; k < W; ++k) {
      du[k] = d[k] * pf_round_to(edt, pf_act(act, g[k]));
      dg[k] = d[k] * u[k] * pf_act_grad(act, g[k]);
    }
    st_vec_c<W, DT>(dgate, r * lddg + c, dt, dg);
    st_vec_c<W, DT>(dup, r * lddu + c, dt, du);
  }
};

// ---- strided copy (<= 6 dims) ----------------------------------------------
struct CopyDesc {
  int64_t size[6], ss[6], ds[6];  // innermost dimension last; size of the innermost already divided by W
  int ndim;
};
template <int W>
__global__ __launch_bounds__(EW_BLOCK) void copy_strided_kernel(const void* src, int sdt, void* dst, int ddt,
                                                                CopyDesc cd, int64_t total, int accumulate) {
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gsz) {
    int64_t rem = i, so = 0, dof = 0;
#pragma unroll
    for (int k = 5; k >= 0; --k) {
      if (k < cd.ndim) {
        const int64_t idx = rem % cd.size[k];
        rem /= cd.size[k];
        const int64_t mul = (k == cd.ndim - 1) ? W : 1;
        so += idx * cd.ss[k] * mul;
        dof += idx * cd.ds[k] * mul;
      }
    }
    float v[W];
    ld_vec<W>(src, so, sdt, v);
    if (accumulate) {
      float o[W];
      ld_vec<W>(dst, dof, ddt, o);
#pragma unroll
      for (int k = 0; k < W; ++k) v[k] += o[k];
    }
    st_vec<W>(dst, dof, ddt, v);
  }
}

// same-dtype copy of non-float element types (token ids, masks): moves raw elements
template <typename U>
__global__ __launch_bounds__(EW_BLOCK) void copy_strided_raw_kernel(const U* src, U* dst, CopyDesc cd, int64_t total) {
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gsz) {
    int64_t rem = i, so = 0, dof = 0;
#pragma unroll
    for (int k = 5; k >= 0; --k) {
      if (k < cd.ndim) {
        const int64_t idx = rem % cd.size[k];
        rem /= cd.size[k];
        so += idx * cd.ss[k];
        dof += idx * cd.ds[k];
      }
    }
    dst[dof] = src[so];
  }
}

// Strided copy in which the source is contiguous along one dimension (`j`) and the destination
// along another (`l`): a batched transpose (NCHW <-> NHWC, [B, C, T] <-> [B, T, C], a convolution
// weight [out, in, 9] <-> [out, 9, in]).  64x64 tiles over (j, l) go through LDS so that reads run
// along j and writes along l, both in runs of up to 64 elements; the remaining dimensions are the
// batch (blockIdx.z).
struct TransposeDesc {
  int64_t nj, nl;            // extents of dimensions j and l
  int64_t s_l, d_j;          // source stride along l, destination stride along j
  int64_t bsize[4], bss[4], bds[4];
  int nb;
};
__global__ __launch_bounds__(256) void copy_transpose_kernel(const void* src, int sdt, void* dst, int ddt,
                                                             TransposeDesc td, int accumulate) {
  __shared__ float tile[64][65];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  int64_t rem = blockIdx.z, so = 0, dof = 0;
#pragma unroll
  for (int k = 3; k >= 0; --k) {
    if (k < td.nb) {
      const int64_t idx = rem % td.bsize[k];
      rem /= td.bsize[k];
      so += idx * td.bss[k];
      dof += idx * td.bds[k];
    }
  }
  const int64_t j0 = (int64_t)blockIdx.x * 64, l0 = (int64_t)blockIdx.y * 64;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t l = l0 + ty + i * 4, j = j0 + tx;
    tile[ty + i * 4][tx] = (l < td.nl && j < td.nj) ? pf_load_as_f32(src, so + l * td.s_l + j, sdt) : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t j = j0 + ty + i * 4, l = l0 + tx;
    if (j < td.nj && l < td.nl) {
      const int64_t o = dof + j * td.d_j + l;
      float v = tile[tx][ty + i * 4];
      if (accumulate) v += pf_load_as_f32(dst, o, ddt);
      pf_store_from_f32(dst, o, ddt, v);
    }
  }
}

// The same when one of the two dimensions is short (a 3x3 convolution's 9 taps) and the block of
// (long, short) elements is contiguous on the side where the short dimension is the contiguous one:
// that side is streamed linearly, 256 x n elements per workgroup, the other side in runs of 256.
//   SRC_NARROW: source element (l, j) at l * nj + j (nj <= 32), destination at j * d_j + l
//   else:       source at l * s_l + j, destination element (j, l) at j * nl + l (nl <= 32)
template <bool SRC_NARROW>
__global__ __launch_bounds__(256) void copy_transpose_narrow_kernel(const void* src, int sdt, void* dst, int ddt,
                                                                    TransposeDesc td, int accumulate) {
  __shared__ float buf[256 * 33];
  const int t = threadIdx.x;
  int64_t rem = blockIdx.z, so = 0, dof = 0;
#pragma unroll
  for (int k = 3; k >= 0; --k) {
    if (k < td.nb) {
      const int64_t idx = rem % td.bsize[k];
      rem /= td.bsize[k];
      so += idx * td.bss[k];
      dof += idx * td.bds[k];
    }
  }
  if (SRC_NARROW) {
    const int n = (int)td.nj, np = n | 1;
    const int64_t l0 = (int64_t)blockIdx.x * 256;
    const int cnt = (int)((td.nl - l0 < 256 ? td.nl - l0 : 256) * n);
    for (int i = t; i < cnt; i += 256) buf[(i / n) * np + (i % n)] = pf_load_as_f32(src, so + l0 * n + i, sdt);
    __syncthreads();
    if (l0 + t < td.nl) {
      for (int j = 0; j < n; ++j) {
        const int64_t o = dof + j * td.d_j + l0 + t;
        float v = buf[t * np + j];
        if (accumulate) v += pf_load_as_f32(dst, o, ddt);
        pf_store_from_f32(dst, o, ddt, v);
      }
    }
  } else {
    const int n = (int)td.nl, np = n | 1;
    const int64_t j0 = (int64_t)blockIdx.x * 256;
    if (j0 + t < td.nj)
      for (int l = 0; l < n; ++l) buf[t * np + l] = pf_load_as_f32(src, so + l * td.s_l + j0 + t, sdt);
    __syncthreads();
    const int cnt = (int)((td.nj - j0 < 256 ? td.nj - j0 : 256) * n);
    for (int i = t; i < cnt; i += 256) {
      const int64_t o = dof + j0 * n + i;
      float v = buf[(i / n) * np + (i % n)];
      if (accumulate) v += pf_load_as_f32(dst, o, ddt);
      pf_store_from_f32(dst, o, ddt, v);
    }
  }
}

// dst[c, r] = src[r, c] with dtype conversion, 64x64 tiles through LDS so that both
// the reads and the writes are contiguous runs of 64 elements
__global__ __launch_bounds__(256) void transpose_cast_kernel(const void* src, int sdt, int64_t ld_src, void* dst,
                                                             int ddt, int64_t ld_dst, int64_t rows, int64_t cols) {
  __shared__ float tile[64][65];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t r = r0 + ty + i * 4, c = c0 + tx;
    tile[ty + i * 4][tx] = (r < rows && c < cols) ? pf_load_as_f32(src, r * ld_src + c, sdt) : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t c = c0 + ty + i * 4, r = r0 + tx;
    if (c < cols && r < rows) pf_store_from_f32(dst, c * ld_dst + r, ddt, tile[tx][ty + i * 4]);
  }
}

// 16-bit -> 16-bit transpose without LDS: a wavefront owns a 64x64 tile, lane (lr, lc) the
// 8x8 block (lr, lc); eight 16-byte loads, an in-register 8x8 transpose, eight 16-byte stores.
// Eight lanes cover 128 contiguous bytes on both the read and the write side.
__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t* src, int64_t ld_src, uint16_t* dst,
                                                          int64_t ld_dst, int64_t rows, int64_t cols) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane >> 3, lc = lane & 7;
  const int64_t r0 = ((int64_t)blockIdx.y * 4 + wave) * 64 + lr * 8, c0 = (int64_t)blockIdx.x * 64 + lc * 8;
  if (r0 >= rows || c0 >= cols) return;
  uint32_t in[8][4];
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    uint4 x = make_uint4(0, 0, 0, 0);
    if (r0 + r < rows) x = *(const uint4*)(src + (r0 + r) * ld_src + c0);
    in[r][0] = x.x; in[r][1] = x.y; in[r][2] = x.z; in[r][3] = x.w;
  }
#pragma unroll
  for (int J = 0; J < 4; ++J) {
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int I = 0; I < 4; ++I) {
      const uint32_t a = in[2 * I][J], c = in[2 * I + 1][J];
      lo[I] = (a & 0xffffu) | (c << 16);
      hi[I] = (a >> 16) | (c & 0xffff0000u);
    }
    if (c0 + 2 * J < cols) *(uint4*)(dst + (c0 + 2 * J) * ld_dst + r0) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    if (c0 + 2 * J + 1 < cols) *(uint4*)(dst + (c0 + 2 * J + 1) * ld_dst + r0) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
  }
}

// ---- multi-tensor cast: the per-step refresh of every 16-bit weight shadow in one launch ----
__global__ __launch_bounds__(256) void cast_batch_kernel(const pf_cast_item* items) {
  const pf_cast_item it = items[blockIdx.y];
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nv = it.vec ? it.n / 8 : 0;
  for (int64_t i = gtid; i < nv; i += gsz) {
    float x[8];
    ld_vec<8>(it.src, i * 8, it.src_dtype, x);
    st_vec<8>(it.dst, i * 8, it.dst_dtype, x);
  }
  for (int64_t i = nv * 8 + gtid; i < it.n; i += gsz)
    pf_store_from_f32(it.dst, i, it.dst_dtype, pf_load_as_f32(it.src, i, it.src_dtype));
}

// ---- both 16-bit shadows of every weight matrix in one launch -------------------------------
// Block (x, y) converts the 64x64 tile x of item y: the fp32 master is read once (float4 per
// lane, 256-byte runs), the plain shadow is written from registers (8 bytes per lane), the
// transposed shadow through a 16-bit LDS tile (8 bytes per lane, 128-byte runs).
__global__ __launch_bounds__(256) void shadow_batch_kernel(const pf_shadow_item* items) {
  __shared__ uint16_t tile[64][64 + 2];
  const pf_shadow_item it = items[blockIdx.y];
  const int64_t tiles_c = (it.cols + 63) / 64, tiles_r = (it.rows + 63) / 64;
  if ((int64_t)blockIdx.x >= tiles_c * tiles_r) return;   // uniform over the block
  const int64_t r0 = ((int64_t)blockIdx.x / tiles_c) * 64, c0 = ((int64_t)blockIdx.x % tiles_c) * 64;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const bool bf = it.dtype == PF_BF16;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int lr = ty + 16 * i;
    const int64_t r = r0 + lr, c = c0 + tx * 4;
    uint16_t h[4] = {0, 0, 0, 0};
    if (r < it.rows && c < it.cols) {       // rows and cols are multiples of 4
      const float4 v = *(const float4*)(it.src + r * it.cols + c);
      const float f[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) h[k] = bf ? pf_f32_to_bf16_bits(f[k]) : pf_f32_to_f16_bits(f[k]);
      if (it.plain)
        *(uint2*)((uint16_t*)it.plain + r * it.cols + c) =
            make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) tile[lr][tx * 4 + k] = h[k];
  }
  __syncthreads();
  if (!it.transposed) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int lc = ty + 16 * i;             // source column = row of the transposed shadow
    const int64_t c = c0 + lc, r = r0 + tx * 4;
    if (c < it.cols && r < it.rows) {
      const uint32_t lo = (uint32_t)tile[tx * 4][lc] | ((uint32_t)tile[tx * 4 + 1][lc] << 16);
      const uint32_t hi = (uint32_t)tile[tx * 4 + 2][lc] | ((uint32_t)tile[tx * 4 + 3][lc] << 16);
      *(uint2*)((uint16_t*)it.transposed + c * it.rows + r) = make_uint2(lo, hi);
    }
  }
}

// ---- multi-tensor Adam / AdamW ---------------------------------------------------------
// One launch updates every parameter of a param group.  Items live in device memory;
// block y walks item y in a grid-stride loop.  The arithmetic follows torch.optim.Adam's
// single-tensor formulation operation by operation (lerp for the first moment, mul + addcmul
// for the second, sqrt / bias_correction2_sqrt + eps, addcdiv).
// With a loss-scaler state (float[8] = scale, growth tracker, found_inf, completed steps,
// step_size, bias_c2_sqrt, 2 unused) the launch does nothing when found_inf is set
// (GradScaler.step skipping the optimizer), and the bias corrections use the device-side count
// of completed steps, which the host cannot know without a synchronisation: a one-thread launch
// ahead of this one forms them in double and leaves them in state[4..5].
__global__ void adam_coefficients_kernel(float* state, double lr, double beta1, double beta2) {
  const double t = (double)state[3] + 1.0;
  state[4] = (float)(lr / (1.0 - pow(beta1, t)));
  state[5] = (float)sqrt(1.0 - pow(beta2, t));
}

__global__ __launch_bounds__(256) void adam_kernel(const pf_adam_item* items, float lr, float omb1, float beta2,
                                                   float omb2, float eps, float weight_decay, float step_size,
                                                   float bias_c2_sqrt, int adamw, const float* scaler_state) {
  // omb1 = 1 - beta1, omb2 = 1 - beta2, step_size = lr / (1 - beta1^t): formed in double
  // like torch does, then rounded once
  if (scaler_state != nullptr) {
    if (scaler_state[2] != 0.f) return;   // uniform over the grid
    step_size = scaler_state[4];
    bias_c2_sqrt = scaler_state[5];
  }
  const pf_adam_item it = items[blockIdx.y];
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x * 4;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < it.n; i += gsz) {
    if (i + 4 <= it.n) {
      float4 p = *(float4*)(it.param + i), g = *(const float4*)(it.grad + i);
      float4 m = *(float4*)(it.exp_avg + i), v = *(float4*)(it.exp_avg_sq + i);
      float pp[4] = {p.x, p.y, p.z, p.w}, gg[4] = {g.x, g.y, g.z, g.w};
      float mm[4] = {m.x, m.y, m.z, m.w}, vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (adamw) pp[k] *= 1.f - lr * weight_decay;
        else if (weight_decay != 0.f) gg[k] += weight_decay * pp[k];
        mm[k] = mm[k] + omb1 * (gg[k] - mm[k]);
        vv[k] = vv[k] * beta2 + omb2 * gg[k] * gg[k];
        const float denom = sqrtf(vv[k]) / bias_c2_sqrt + eps;
        pp[k] = pp[k] - step_size * (mm[k] / denom);
      }
      *(float4*)(it.param + i) = make_float4(pp[0], pp[1], pp[2], pp[3]);
      *(float4*)(it.exp_avg + i) = make_float4(mm[0], mm[1], mm[2], mm[3]);
      *(float4*)(it.exp_avg_sq + i) = make_float4(vv[0], vv[1], vv[2], vv[3]);
    } else {
      for (int64_t j = i; j < it.n; ++j) {
        float pv = it.param[j], gv = it.grad[j], mv = it.exp_avg[j], vv = it.exp_avg_sq[j];
        if (adamw) pv *= 1.f - lr * weight_decay;
        else if (weight_decay != 0.f) gv += weight_decay * pv;
        mv = mv + omb1 * (gv - mv);
        vv = vv * beta2 + omb2 * gv * gv;
        const float denom = sqrtf(vv) / bias_c2_sqrt + eps;
        pv = pv - step_size * (mv / denom);
        it.param[j] = pv; it.exp_avg[j] = mv; it.exp_avg_sq[j] = vv;
      }
    }
  }
}

// ---- rotary embedding --------------------------------------------------------
// one thread per (b, t, h, i) pair index i < D/2
__global__ __launch_bounds__(EW_BLOCK) void rope_kernel(const void* x, void* y, int dt, const float* cos_t,
                                                        const float* sin_t, int64_t tab_ld, int64_t B, int64_t T,
                                                        int64_t H, int64_t D, int64_t xsb, int64_t xst, int64_t xsh,
                                                        int64_t ysb, int64_t yst, int64_t ysh, int inverse) {
  const int64_t half = D / 2;
  const int64_t total = B * T * H * half;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gsz) {
    const int64_t i = idx % half;
    int64_t r = idx / half;
    const int64_t h = r % H;
    r /= H;
    const int64_t t = r % T, b = r / T;
    const int64_t xo = b * xsb + t * xst + h * xsh, yo = b * ysb + t * yst + h * ysh;
    const float x1 = pf_load_as_f32(x, xo + i, dt), x2 = pf_load_as_f32(x, xo + i + half, dt);
    const float c = cos_t[t * tab_ld + i];
    const float s = inverse ? -sin_t[t * tab_ld + i] : sin_t[t * tab_ld + i];
    pf_store_from_f32(y, yo + i, dt, x1 * c - x2 * s);
    pf_store_from_f32(y, yo + i + half, dt, x2 * c + x1 * s);
  }
}

}  // namespace

extern "C" int pf_act_fwd(const void* x, void* y, int dtype, int act, int64_t n, void* stream) {
  PF_REQUIRE(n >= 0 && pf_is_float_dtype(dtype), "pf_act_fwd: bad arguments");
  if (n == 0) return PF_OK;
  PF_REQUIRE(x && y, "pf_act_fwd: null pointer");
  ActFwd f{x, y, dtype, act};
  return ew_launch(f, n, al16(x) && al16(y), (hipStream_t)stream, "pf_act_fwd");
}

extern "C" int pf_act_bwd(const void* dy, const void* x, void* dx, int dtype, int act, int64_t n, void* stream) {
  PF_REQUIRE(n >= 0 && pf_is_float_dtype(dtype), "pf_act_bwd: bad arguments");
  if (n == 0) return PF_OK;
  PF_REQUIRE(dy && x && dx, "pf_act_bwd: null pointer");
  ActBwd f{dy, x, dx, dtype, act};
  return ew_launch(f, n, al16(dy) && al16(x) && al16(dx), (hipStream_t)stream, "pf_act_bwd");
}

extern "C" int pf_glu_fwd(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* y, int64_t ld_y,
                          int dtype, int act, int64_t rows, int64_t cols, void* stream) {
  PF_REQUIRE(rows >= 0 && cols >= 0 && pf_is_float_dtype(dtype), "pf_glu_fwd: bad arguments");
  if (rows == 0 || cols == 0) return PF_OK;
  PF_REQUIRE(gate && up && y, "pf_glu_fwd: null pointer");
  PF_REQUIRE(ld_gate >= cols && ld_up >= cols && ld_y >= cols, "pf_glu_fwd: leading dimension too small");
  const bool vec = al16(gate) && al16(up) && al16(y) && cols % 8 == 0 && ld_gate % 8 == 0 && ld_up % 8 == 0 &&
                   ld_y % 8 == 0;
  if (vec && dtype == PF_BF16)
    return ew_launch(GluFwd<PF_BF16>{gate, up, y, ld_gate, ld_up, ld_y, cols, dtype, act}, rows * cols, vec,
                     (hipStream_t)stream, "pf_glu_fwd");
  if (vec && dtype == PF_F16)
    return ew_launch(GluFwd<PF_F16>{gate, up, y, ld_gate, ld_up, ld_y, cols, dtype, act}, rows * cols, vec,
                     (hipStream_t)stream, "pf_glu_fwd");
  GluFwd<> f{gate, up, y, ld_gate, ld_up, ld_y, cols, dtype, act};
  return ew_launch(f, rows * cols, vec, (hipStream_t)stream, "pf_glu_fwd");
}

extern "C" int pf_glu_bwd(const void* dy, int64_t ld_dy, const void* gate, int64_t ld_gate, const void* up,
                          int64_t ld_up, void* dgate, int64_t ld_dgate, void* dup, int64_t ld_dup, int dtype, int act,
                          int64_t rows, int64_t cols, void* stream) {
  PF_REQUIRE(rows >= 0 && cols >= 0 && pf_is_float_dtype(dtype), "pf_glu_bwd: bad arguments");
  if (rows == 0 || cols == 0) return PF_OK;
  PF_REQUIRE(dy && gate && up && dgate && dup, "pf_glu_bwd: null pointer");
  PF_REQUIRE(ld_dy >= cols && ld_gate >= cols && ld_up >= cols && ld_dgate >= cols && ld_dup >= cols,
             "pf_glu_bwd: leading dimension too small");
  const bool vec = al16(dy) && al16(gate) && al16(up) && al16(dgate) && al16(dup) && cols % 8 == 0 &&
                   ld_dy % 8 == 0 && ld_gate % 8 == 0 && ld_up % 8 == 0 && ld_dgate % 8 == 0 && ld_dup % 8 == 0;
  if (vec && dtype == PF_BF16)
    return ew_launch(GluBwd<PF_BF16>{dy, gate, up, dgate, dup, ld_dy, ld_gate, ld_up, ld_dgate, ld_dup, cols, dtype, act},
                     rows * cols, vec, (hipStream_t)stream, "pf_glu_bwd");
  if (vec && dtype == PF_F16)
    return ew_launch(GluBwd<PF_F16>{dy, gate, up, dgate, dup, ld_dy, ld_gate, ld_up, ld_dgate, ld_dup, cols, dtype, act},
                     rows * cols, vec, (hipStream_t)stream, "pf_glu_bwd");
  GluBwd<> f{dy, gate, up, dgate, dup, ld_dy, ld_gate, ld_up, ld_dgate, ld_dup, cols, dtype, act};
  return ew_launch(f, rows * cols, vec, (hipStream_t)stream, "pf_glu_bwd");
}

extern "C" int pf_axpby(const void* a, int a_dtype, float alpha, const void* b, int b_dtype, float beta, void* out,
                        int out_dtype, int64_t n, void* stream) {
  PF_REQUIRE(n >= 0 && pf_is_float_dtype(a_dtype) && pf_is_float_dtype(out_dtype), "pf_axpby: bad arguments");
  if (n == 0) return PF_OK;
  PF_REQUIRE(a && out, "pf_axpby: null pointer");
  if (!b) {
    Scale f{a, out, a_dtype, out_dtype, alpha};
    return ew_launch(f, n, al16(a) && al16(out), (hipStream_t)stream, "pf_axpby");
  }
  PF_REQUIRE(pf_is_float_dtype(b_dtype), "pf_axpby: bad b dtype");
  Axpby f{a, b, out, a_dtype, b_dtype, out_dtype, alpha, beta};
  return ew_launch(f, n, al16(a) && al16(b) && al16(out), (hipStream_t)stream, "pf_axpby");
}

extern "C" int pf_bias_add(const void* x, int x_dtype, const void* bias, int bias_dtype, void* y, int y_dtype,
                           int64_t n, int64_t bias_len, int64_t rows_per_bias, void* stream) {
  PF_REQUIRE(n >= 0 && bias_len > 0 && pf_is_float_dtype(x_dtype) && pf_is_float_dtype(bias_dtype) &&
                 pf_is_float_dtype(y_dtype),
             "pf_bias_add: bad arguments");
  if (n == 0) return PF_OK;
  PF_REQUIRE(x && bias && y, "pf_bias_add: null pointer");
  PF_REQUIRE(n % bias_len == 0, "pf_bias_add: n must be a multiple of bias_len");
  PF_REQUIRE(rows_per_bias >= 0, "pf_bias_add: negative rows_per_bias");
  BiasAdd f{x, bias, y, x_dtype, bias_dtype, y_dtype, bias_len, rows_per_bias * bias_len};
  return ew_launch(f, n, al16(x) && al16(bias) && al16(y) && bias_len % 8 == 0, (hipStream_t)stream, "pf_bias_add");
}

extern "C" int pf_cast(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n, void* stream) {
  PF_REQUIRE(n >= 0 && pf_is_float_dtype(src_dtype) && pf_is_float_dtype(dst_dtype), "pf_cast: bad arguments");
  if (n == 0) return PF_OK;
  PF_REQUIRE(src && dst, "pf_cast: null pointer");
  Cast f{src, dst, src_dtype, dst_dtype};
  return ew_launch(f, n, al16(src) && al16(dst), (hipStream_t)stream, "pf_cast");
}

extern "C" int pf_transpose_cast(const void* src, int src_dtype, int64_t ld_src, void* dst, int dst_dtype,
                                 int64_t ld_dst, int64_t rows, int64_t cols, void* stream) {
  PF_REQUIRE(rows >= 0 && cols >= 0 && pf_is_float_dtype(src_dtype) && pf_is_float_dtype(dst_dtype),
             "pf_transpose_cast: bad arguments");
  if (rows == 0 || cols == 0) return PF_OK;
  PF_REQUIRE(src && dst && ld_src >= cols && ld_dst >= rows, "pf_transpose_cast: bad operands");
  // same 16-bit dtype, everything 16-byte granular (the destination rows are `rows` long and
  // written 8 at a time: ld_dst >= ceil8(rows)): register-transpose path
  if (src_dtype == dst_dtype && src_dtype != PF_F32 && cols % 8 == 0 && ld_src % 8 == 0 && ld_dst % 8 == 0 &&
      ld_dst >= (rows + 7) / 8 * 8 && pf_aligned(src, 16) && pf_aligned(dst, 16)) {
    const dim3 g16((unsigned)((cols + 63) / 64), (unsigned)((rows + 255) / 256));
    PF_REQUIRE(g16.y <= 65535, "pf_transpose_cast: too many rows");
    hipLaunchKernelGGL(transpose16_kernel, g16, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)src, ld_src,
                       (uint16_t*)dst, ld_dst, rows, cols);
    PF_CHECK_LAUNCH("pf_transpose_cast");
    return PF_OK;
  }
  const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  PF_REQUIRE(grid.y <= 65535, "pf_transpose_cast: too many rows");
  hipLaunchKernelGGL(transpose_cast_kernel, grid, dim3(256), 0, (hipStream_t)stream, src, src_dtype, ld_src, dst,
                     dst_dtype, ld_dst, rows, cols);
  PF_CHECK_LAUNCH("pf_transpose_cast");
  return PF_OK;
}

extern "C" int pf_fill(void* dst, int dtype, float value, int64_t n, void* stream) {
  PF_REQUIRE(n >= 0 && pf_is_float_dtype(dtype), "pf_fill: bad arguments");
  if (n == 0) return PF_OK;
  PF_REQUIRE(dst, "pf_fill: null pointer");
  Fill f{dst, dtype, value};
  return ew_launch(f, n, al16(dst), (hipStream_t)stream, "pf_fill");
}

extern "C" int pf_grad_accumulate_f32(float* acc, const void* g, int g_dtype, int64_t n, void* stream) {
  PF_REQUIRE(n >= 0 && pf_is_float_dtype(g_dtype), "pf_grad_accumulate_f32: bad arguments");
  if (n == 0) return PF_OK;
  PF_REQUIRE(acc && g, "pf_grad_accumulate_f32: null pointer");
  GradAcc f{acc, g, g_dtype};
  return ew_launch(f, n, al16(acc) && al16(g), (hipStream_t)stream, "pf_grad_accumulate_f32");
}

extern "C" int pf_copy_strided(const void* src, int src_dtype, const int64_t* src_strides, void* dst, int dst_dtype,
                               const int64_t* dst_strides, const int64_t* sizes, int ndim, int accumulate,
                               void* stream) {
  PF_REQUIRE(ndim >= 1 && ndim <= 6, "pf_copy_strided: ndim %d outside 1..6", ndim);
  PF_REQUIRE(src_strides && dst_strides && sizes, "pf_copy_strided: null shape");
  const bool raw = !pf_is_float_dtype(src_dtype);
  if (raw) PF_REQUIRE(src_dtype == dst_dtype && pf_dtype_size(src_dtype) > 0 && !accumulate,
                      "pf_copy_strided: integer tensors can only be copied to the same dtype");
  else PF_REQUIRE(pf_is_float_dtype(dst_dtype), "pf_copy_strided: bad dtype");
  CopyDesc cd;
  cd.ndim = ndim;
  int64_t total = 1;
  bool vec = pf_aligned(src, 16) && pf_aligned(dst, 16);
  for (int k = 0; k < 6; ++k) {
    cd.size[k] = k < ndim ? sizes[k] : 1;
    cd.ss[k] = k < ndim ? src_strides[k] : 0;
    cd.ds[k] = k < ndim ? dst_strides[k] : 0;
    if (k < ndim) {
      PF_REQUIRE(sizes[k] >= 0, "pf_copy_strided: negative size");
      PF_REQUIRE(dst_strides[k] >= 0 && src_strides[k] >= 0, "pf_copy_strided: negative stride");
      total *= sizes[k];
      if (k < ndim - 1) vec = vec && src_strides[k] % 8 == 0 && dst_strides[k] % 8 == 0;
    }
  }
  if (total == 0) return PF_OK;
  PF_REQUIRE(src && dst, "pf_copy_strided: null pointer");
  vec = vec && src_strides[ndim - 1] == 1 && dst_strides[ndim - 1] == 1 && sizes[ndim - 1] % 8 == 0;
  hipStream_t st = (hipStream_t)stream;
  if (raw) {
    switch (pf_dtype_size(src_dtype)) {
      case 8: hipLaunchKernelGGL(copy_strided_raw_kernel<uint64_t>, ew_grid(total), dim3(EW_BLOCK), 0, st, (const uint64_t*)src, (uint64_t*)dst, cd, total); break;
      case 4: hipLaunchKernelGGL(copy_strided_raw_kernel<uint32_t>, ew_grid(total), dim3(EW_BLOCK), 0, st, (const uint32_t*)src, (uint32_t*)dst, cd, total); break;
      default: hipLaunchKernelGGL(copy_strided_raw_kernel<uint8_t>, ew_grid(total), dim3(EW_BLOCK), 0, st, (const uint8_t*)src, (uint8_t*)dst, cd, total); break;
    }
  } else if (vec) {
    cd.size[ndim - 1] /= 8;
    total /= 8;
    hipLaunchKernelGGL(copy_strided_kernel<8>, ew_grid(total), dim3(EW_BLOCK), 0, st, src, src_dtype, dst, dst_dtype,
                       cd, total, accumulate);
  } else {
    // batched transpose: the source is contiguous along one dimension (p), the destination along another (q)
    int pdim = -1, qdim = -1;
    if (ndim >= 2 && ndim <= 6) {
      for (int k = ndim - 1; k >= 0; --k) {
        if (pdim < 0 && src_strides[k] == 1 && sizes[k] >= 2) pdim = k;
        if (qdim < 0 && dst_strides[k] == 1 && sizes[k] >= 2) qdim = k;
      }
    }
    if (pdim >= 0 && qdim >= 0 && pdim != qdim && ndim - 2 <= 4) {
      TransposeDesc td;
      td.nj = sizes[pdim]; td.nl = sizes[qdim];
      td.s_l = src_strides[qdim]; td.d_j = dst_strides[pdim];
      td.nb = 0;
      int64_t batch = 1;
      for (int k = 0; k < ndim; ++k) {
        if (k == pdim || k == qdim) continue;
        td.bsize[td.nb] = sizes[k]; td.bss[td.nb] = src_strides[k]; td.bds[td.nb] = dst_strides[k];
        ++td.nb;
        batch *= sizes[k];
      }
      for (int k = td.nb; k < 4; ++k) { td.bsize[k] = 1; td.bss[k] = 0; td.bds[k] = 0; }
      const int64_t gx = (td.nj + 63) / 64, gy = (td.nl + 63) / 64;
      if (batch <= 65535 && td.nj <= 32 && td.s_l == td.nj) {
        hipLaunchKernelGGL(copy_transpose_narrow_kernel<true>, dim3((unsigned)((td.nl + 255) / 256), 1, (unsigned)batch),
                           dim3(256), 0, st, src, src_dtype, dst, dst_dtype, td, accumulate);
        PF_CHECK_LAUNCH("pf_copy_strided");
        return PF_OK;
      }
      if (batch <= 65535 && td.nl <= 32 && td.d_j == td.nl) {
        hipLaunchKernelGGL(copy_transpose_narrow_kernel<false>, dim3((unsigned)((td.nj + 255) / 256), 1, (unsigned)batch),
                           dim3(256), 0, st, src, src_dtype, dst, dst_dtype, td, accumulate);
        PF_CHECK_LAUNCH("pf_copy_strided");
        return PF_OK;
      }
      if (batch <= 65535 && gy <= 65535) {
        hipLaunchKernelGGL(copy_transpose_kernel, dim3((unsigned)gx, (unsigned)gy, (unsigned)batch), dim3(256), 0, st, src,
                           src_dtype, dst, dst_dtype, td, accumulate);
        PF_CHECK_LAUNCH("pf_copy_strided");
        return PF_OK;
      }
    }
    hipLaunchKernelGGL(copy_strided_kernel<1>, ew_grid(total), dim3(EW_BLOCK), 0, st, src, src_dtype, dst, dst_dtype,
                       cd, total, accumulate);
  }
  PF_CHECK_LAUNCH("pf_copy_strided");
  return PF_OK;
}

namespace {
// 16-bit rotary embedding, one thread per 8 consecutive pair indices: two 16-byte loads, two
// 16-byte stores, 8 cos / sin values each (requires D/2 % 8 == 0 and 16-byte aligned rows)
template <int DT>
__global__ __launch_bounds__(EW_BLOCK) void rope_vec_kernel(const uint16_t* x, uint16_t* y, const float* cos_t,
                                                            const float* sin_t, int64_t tab_ld, int64_t B, int64_t T,
                                                            int64_t H, int64_t D, int64_t xsb, int64_t xst, int64_t xsh,
                                                            int64_t ysb, int64_t yst, int64_t ysh, int inverse) {
  const int64_t half = D / 2, hv = half / 8;
  const int64_t total = B * T * H * hv;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gsz) {
    const int64_t i = (idx % hv) * 8;
    int64_t r = idx / hv;
    const int64_t h = r % H;
    r /= H;
    const int64_t t = r % T, b = r / T;
    const int64_t xo = b * xsb + t * xst + h * xsh + i, yo = b * ysb + t * yst + h * ysh + i;
    float x1[8], x2[8], c[8], sn[8], o1[8], o2[8];
    Vec8<DT>::load(x, xo, x1);
    Vec8<DT>::load(x, xo + half, x2);
    Vec8<PF_F32>::load(cos_t, t * tab_ld + i, c);
    Vec8<PF_F32>::load(sin_t, t * tab_ld + i, sn);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float s = inverse ? -sn[k] : sn[k];
      o1[k] = x1[k] * c[k] - x2[k] * s;
      o2[k] = x2[k] * c[k] + x1[k] * s;
    }
    Vec8<DT>::store(y, yo, o1);
    Vec8<DT>::store(y, yo + half, o2);
  }
}
}  // namespace

extern "C" int pf_rope(const void* x, void* y, int dtype, const float* cos_t, const float* sin_t, int64_t tab_ld,
                       int64_t B, int64_t T, int64_t H, int64_t D, int64_t x_sb, int64_t x_st, int64_t x_sh,
                       int64_t y_sb, int64_t y_st, int64_t y_sh, int inverse, void* stream) {
  PF_REQUIRE(B >= 0 && T >= 0 && H >= 0 && D >= 0 && D % 2 == 0 && pf_is_float_dtype(dtype), "pf_rope: bad arguments");
  PF_REQUIRE(tab_ld >= D / 2, "pf_rope: table row stride %lld < D/2", (long long)tab_ld);
  const int64_t total = B * T * H * (D / 2);
  if (total == 0) return PF_OK;
  PF_REQUIRE(x && y && cos_t && sin_t, "pf_rope: null pointer");
  const bool vec = dtype != PF_F32 && (D / 2) % 8 == 0 && tab_ld % 4 == 0 && al16(x) && al16(y) && al16(cos_t) &&
                   al16(sin_t) && x_sb % 8 == 0 && x_st % 8 == 0 && x_sh % 8 == 0 && y_sb % 8 == 0 && y_st % 8 == 0 &&
                   y_sh % 8 == 0;
  if (vec) {
    const dim3 grid = ew_grid(total / 8);
    if (dtype == PF_F16)
      hipLaunchKernelGGL(rope_vec_kernel<PF_F16>, grid, dim3(EW_BLOCK), 0, (hipStream_t)stream, (const uint16_t*)x,
                         (uint16_t*)y, cos_t, sin_t, tab_ld, B, T, H, D, x_sb, x_st, x_sh, y_sb, y_st, y_sh, inverse);
    else
      hipLaunchKernelGGL(rope_vec_kernel<PF_BF16>, grid, dim3(EW_BLOCK), 0, (hipStream_t)stream, (const uint16_t*)x,
                         (uint16_t*)y, cos_t, sin_t, tab_ld, B, T, H, D, x_sb, x_st, x_sh, y_sb, y_st, y_sh, inverse);
    PF_CHECK_LAUNCH("pf_rope");
    return PF_OK;
  }
  hipLaunchKernelGGL(rope_kernel, ew_grid(total), dim3(EW_BLOCK), 0, (hipStream_t)stream, x, y, dtype, cos_t, sin_t,
                     tab_ld, B, T, H, D, x_sb, x_st, x_sh, y_sb, y_st, y_sh, inverse);
  PF_CHECK_LAUNCH("pf_rope");
  return PF_OK;
}

namespace {
int adam_launch(const pf_adam_item* items_dev, int n_items, int64_t max_n, double lr, double beta1, double beta2,
                double eps, double weight_decay, int64_t step, int adamw, float* scaler_state, void* stream,
                const char* name);
}

extern "C" int pf_adam_step(const pf_adam_item* items_dev, int n_items, int64_t max_n, double lr, double beta1,
                            double beta2, double eps, double weight_decay, int64_t step, int adamw, void* stream) {
  PF_REQUIRE(step >= 1, "pf_adam_step: bad step");
  return adam_launch(items_dev, n_items, max_n, lr, beta1, beta2, eps, weight_decay, step, adamw, nullptr, stream,
                     "pf_adam_step");
}

extern "C" int pf_adam_step_scaled(const pf_adam_item* items_dev, int n_items, int64_t max_n, double lr, double beta1,
                                   double beta2, double eps, double weight_decay, int adamw, float* scaler_state,
                                   void* stream) {
  PF_REQUIRE(scaler_state != nullptr, "pf_adam_step_scaled: null scaler state");
  return adam_launch(items_dev, n_items, max_n, lr, beta1, beta2, eps, weight_decay, 1, adamw, scaler_state, stream,
                     "pf_adam_step_scaled");
}

// ---- dynamic loss scaling (torch.amp.GradScaler's rule, on the device) -------------------
namespace {
// g *= 1/scale in place; found_inf = 1 when any element is not finite (plain store of the same
// value from every block that sees one: no atomic needed, and deterministic)
__device__ __forceinline__ unsigned nonfinite(float v) {   // all exponent bits set: inf or NaN
  return (__float_as_uint(v) & 0x7f800000u) == 0x7f800000u ? 1u : 0u;
}

__global__ __launch_bounds__(256) void scaler_unscale_kernel(float* g, int64_t n, float* state) {
  const float inv = 1.0f / state[0];
  unsigned bad = 0;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x * 4;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < n; i += gsz) {
    if (i + 4 <= n) {
      float4 v = *(float4*)(g + i);
      v.x *= inv; v.y *= inv; v.z *= inv; v.w *= inv;
      bad |= nonfinite(v.x) | nonfinite(v.y) | nonfinite(v.z) | nonfinite(v.w);
      *(float4*)(g + i) = v;
    } else {
      for (int64_t j = i; j < n; ++j) {
        const float v = g[j] * inv;
        bad |= nonfinite(v);
        g[j] = v;
      }
    }
  }
  if (bad) state[2] = 1.0f;
}

__global__ void scaler_update_kernel(float* state, float growth, float backoff, int interval) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  float scale = state[0], tracker = state[1];
  if (state[2] != 0.f) {
    scale *= backoff;
    tracker = 0.f;
  } else {
    tracker += 1.f;
    state[3] += 1.f;
    if (tracker >= (float)interval) {
      scale *= growth;
      tracker = 0.f;
    }
  }
  state[0] = scale;
  state[1] = tracker;
  state[2] = 0.f;
}

struct ScaleByState {
  const void* src; int src_dt; const float* state; void* dst; int dst_dt;
  __device__ __forceinline__ void apply8(int64_t i) const {
    float v[8];
    ld_vec<8>(src, i, src_dt, v);
    const float s = state[0];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] *= s;
    st_vec<8>(dst, i, dst_dt, v);
  }
  __device__ __forceinline__ void apply1(int64_t i) const {
    pf_store_from_f32(dst, i, dst_dt, pf_load_as_f32(src, i, src_dt) * state[0]);
  }
};

__global__ __launch_bounds__(256) void scale_by_state_kernel(ScaleByState f, int64_t n, int vec) {
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nv = vec ? n / 8 : 0;
  for (int64_t i = gtid; i < nv; i += gsz) f.apply8(i * 8);
  for (int64_t i = nv * 8 + gtid; i < n; i += gsz) f.apply1(i);
}
}  // namespace

extern "C" int pf_scaler_unscale(float* grads, int64_t n, float* state, void* stream) {
  PF_REQUIRE(n >= 0, "pf_scaler_unscale: negative size");
  if (n == 0) return PF_OK;
  PF_REQUIRE(grads && state && pf_aligned(grads, 16), "pf_scaler_unscale: null or unaligned pointer");
  int64_t blocks = (n / 4 + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(scaler_unscale_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, grads, n, state);
  PF_CHECK_LAUNCH("pf_scaler_unscale");
  return PF_OK;
}

extern "C" int pf_scaler_update(float* state, double growth_factor, double backoff_factor, int growth_interval,
                                void* stream) {
  PF_REQUIRE(state && growth_factor >= 1.0 && backoff_factor > 0.0 && backoff_factor <= 1.0 && growth_interval >= 1,
             "pf_scaler_update: bad arguments");
  hipLaunchKernelGGL(scaler_update_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, state, (float)growth_factor,
                     (float)backoff_factor, growth_interval);
  PF_CHECK_LAUNCH("pf_scaler_update");
  return PF_OK;
}

extern "C" int pf_scale_by_state(const void* src, int src_dtype, const float* state, void* dst, int dst_dtype, int64_t n,
                                 void* stream) {
  PF_REQUIRE(n >= 0, "pf_scale_by_state: negative size");
  if (n == 0) return PF_OK;
  PF_REQUIRE(src && dst && state, "pf_scale_by_state: null pointer");
  PF_REQUIRE(pf_is_float_dtype(src_dtype) && pf_is_float_dtype(dst_dtype), "pf_scale_by_state: bad dtype");
  ScaleByState f{src, src_dtype, state, dst, dst_dtype};
  const int vec = pf_aligned(src, 16) && pf_aligned(dst, 16);
  int64_t blocks = ((vec ? n / 8 : n) + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(scale_by_state_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, f, n, vec);
  PF_CHECK_LAUNCH("pf_scale_by_state");
  return PF_OK;
}

namespace {
int adam_launch(const pf_adam_item* items_dev, int n_items, int64_t max_n, double lr, double beta1, double beta2,
                double eps, double weight_decay, int64_t step, int adamw, float* scaler_state, void* stream,
                const char* name) {
  PF_REQUIRE(n_items >= 0 && max_n >= 0, "%s: bad arguments", name);
  if (n_items == 0 || max_n == 0) return PF_OK;
  PF_REQUIRE(items_dev != nullptr && n_items <= 65535, "%s: bad item list", name);
  const double bc1 = 1.0 - pow(beta1, (double)step);
  const double bc2 = 1.0 - pow(beta2, (double)step);
  int64_t bx = (max_n / 4 + 255) / 256;
  if (bx > 64) bx = 64;   // enough blocks per tensor; small tensors leave most of them idle at once
  if (bx < 1) bx = 1;
  if (scaler_state != nullptr)
    hipLaunchKernelGGL(adam_coefficients_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, scaler_state, lr, beta1,
                       beta2);
  hipLaunchKernelGGL(adam_kernel, dim3((unsigned)bx, (unsigned)n_items), dim3(256), 0, (hipStream_t)stream, items_dev,
                     (float)lr, (float)(1.0 - beta1), (float)beta2, (float)(1.0 - beta2), (float)eps, (float)weight_decay,
                     (float)(lr / bc1), (float)sqrt(bc2), adamw, scaler_state);
  PF_CHECK_LAUNCH(name);
  return PF_OK;
}
}  // namespace

extern "C" int pf_shadow_batch(const pf_shadow_item* items_dev, int n_items, int64_t max_tiles, void* stream) {
  PF_REQUIRE(n_items >= 0 && max_tiles >= 0, "pf_shadow_batch: bad arguments");
  if (n_items == 0 || max_tiles == 0) return PF_OK;
  PF_REQUIRE(items_dev != nullptr && n_items <= 65535 && max_tiles < (1ll << 31), "pf_shadow_batch: bad item list");
  hipLaunchKernelGGL(shadow_batch_kernel, dim3((unsigned)max_tiles, (unsigned)n_items), dim3(256), 0,
                     (hipStream_t)stream, items_dev);
  PF_CHECK_LAUNCH("pf_shadow_batch");
  return PF_OK;
}

extern "C" int pf_cast_batch(const pf_cast_item* items_dev, int n_items, int64_t max_n, void* stream) {
  PF_REQUIRE(n_items >= 0 && max_n >= 0, "pf_cast_batch: bad arguments");
  if (n_items == 0 || max_n == 0) return PF_OK;
  PF_REQUIRE(items_dev != nullptr && n_items <= 65535, "pf_cast_batch: bad item list");
  int64_t bx = (max_n / 8 + 255) / 256;
  if (bx > 64) bx = 64;
  if (bx < 1) bx = 1;
  hipLaunchKernelGGL(cast_batch_kernel, dim3((unsigned)bx, (unsigned)n_items), dim3(256), 0, (hipStream_t)stream,
                     items_dev);
  PF_CHECK_LAUNCH("pf_cast_batch");
  return PF_OK;
}
