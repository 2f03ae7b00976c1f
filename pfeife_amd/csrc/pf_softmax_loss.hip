// Row softmax (attention probabilities), cross-entropy, MSE and sum losses.
// Row-wise kernels: one wavefront per attention row, one workgroup per
// cross-entropy row (vocabulary-sized rows); reductions are wavefront
// butterflies plus a 4-entry LDS exchange, never atomics, so results are
// reproducible run to run.
#include "pf_common.h"

namespace {

// ---- softmax forward: fp32 scores -> probabilities --------------------------
__global__ __launch_bounds__(256) void softmax_fwd_kernel(const float* s, int64_t ld_s, void* p, int p_dt, int64_t ld_p,
                                                          int64_t rows, int64_t cols, int64_t q_len, int causal) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  const float* sr = s + row * ld_s;
  int64_t lim = cols;  // columns [0, lim) are visible
  if (causal) {
    lim = (row % q_len) + (cols - q_len) + 1;
    if (lim > cols) lim = cols;
    if (lim < 0) lim = 0;
  }
  float m = -INFINITY;
  for (int64_t c = lane; c < lim; c += 64) m = fmaxf(m, sr[c]);
  m = pf_wave_max(m);
  float z = 0.f;
  for (int64_t c = lane; c < lim; c += 64) z += expf(sr[c] - m);
  z = pf_wave_sum(z);
  const float inv = z > 0.f ? 1.f / z : 0.f;
  const int64_t pb = row * ld_p;
  for (int64_t c = lane; c < ld_p; c += 64) {
    const float v = c < lim ? expf(sr[c] - m) * inv : 0.f;
    pf_store_from_f32(p, pb + c, p_dt, v);
  }
}

// ds = scale * p * (dp - sum(dp * p))
__global__ __launch_bounds__(256) void softmax_bwd_kernel(const float* dp, int64_t ld_dp, const void* p, int p_dt,
                                                          int64_t ld_p, void* ds, int ds_dt, int64_t ld_ds,
                                                          int64_t rows, int64_t cols, float scale) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  const float* dr = dp + row * ld_dp;
  const int64_t pb = row * ld_p;
  float acc = 0.f;
  for (int64_t c = lane; c < cols; c += 64) acc += dr[c] * pf_load_as_f32(p, pb + c, p_dt);
  acc = pf_wave_sum(acc);
  const int64_t ob = row * ld_ds;
  for (int64_t c = lane; c < ld_ds; c += 64) {
    float v = 0.f;
    if (c < cols) v = scale * pf_load_as_f32(p, pb + c, p_dt) * (dr[c] - acc);
    pf_store_from_f32(ds, ob + c, ds_dt, v);
  }
}

// ---- cross entropy -------------------------------------------------------------
__global__ __launch_bounds__(256) void ce_fwd_kernel(const void* logits, int l_dt, const int64_t* targets,
                                                     float* row_loss, float* row_lse, int64_t classes,
                                                     int64_t ignore_index) {
  __shared__ float sm[4];
  const int64_t row = blockIdx.x;
  const int64_t base = row * classes;
  float m = -INFINITY;
  for (int64_t c = threadIdx.x; c < classes; c += 256) m = fmaxf(m, pf_load_as_f32(logits, base + c, l_dt));
  m = pf_block_max<4>(m, sm);
  float z = 0.f;
  for (int64_t c = threadIdx.x; c < classes; c += 256) z += expf(pf_load_as_f32(logits, base + c, l_dt) - m);
  z = pf_block_sum<4>(z, sm);
  if (threadIdx.x == 0) {
    const float lse = m + logf(z);
    const int64_t t = targets[row];
    row_lse[row] = lse;
    // out-of-range targets other than ignore_index are treated as ignored and
    // flagged with NaN so that the caller sees them
    float l = 0.f;
    if (t != ignore_index) l = (t >= 0 && t < classes) ? lse - pf_load_as_f32(logits, base + t, l_dt) : NAN;
    row_loss[row] = l;
  }
}

// loss[0] = sum(row_loss over valid rows) / n_valid ; loss[1] = n_valid
__global__ __launch_bounds__(256) void ce_mean_kernel(const float* row_loss, const int64_t* targets, float* loss,
                                                      int64_t rows, int64_t ignore_index) {
  __shared__ float sm[4];
  float s = 0.f, n = 0.f;
  for (int64_t r = threadIdx.x; r < rows; r += 256) {
    if (targets[r] != ignore_index) {
      s += row_loss[r];
      n += 1.f;
    }
  }
  s = pf_block_sum<4>(s, sm);
  n = pf_block_sum<4>(n, sm);
  if (threadIdx.x == 0) {
    loss[0] = n > 0.f ? s / n : NAN;  // torch returns nan for an all-ignored batch
    loss[1] = n;
  }
}

__global__ __launch_bounds__(256) void ce_bwd_kernel(const void* logits, int l_dt, const int64_t* targets,
                                                     const float* row_lse, const float* dloss, const float* n_valid,
                                                     void* dlogits, int dl_dt, int64_t classes,
                                                     int64_t ignore_index) {
  const int64_t row = blockIdx.x;
  const int64_t base = row * classes;
  const int64_t t = targets[row];
  const float g = (dloss ? dloss[0] : 1.f) / n_valid[0];
  const float lse = row_lse[row];
  const bool ignored = (t == ignore_index);
  for (int64_t c = threadIdx.x; c < classes; c += 256) {
    float v = 0.f;
    if (!ignored) {
      v = expf(pf_load_as_f32(logits, base + c, l_dt) - lse);
      if (c == t) v -= 1.f;
      v *= g;
    }
    pf_store_from_f32(dlogits, base + c, dl_dt, v);
  }
}

// Vectorised variants (classes % 8 == 0, 16-byte aligned rows, dtype fixed at compile time):
// eight classes per lane and access, several accesses in flight; same two passes over the row
// (maximum, then sum of exponentials; the second pass is served by the caches).
template <int DT>
__global__ __launch_bounds__(256) void ce_fwd_vec_kernel(const void* logits, const int64_t* targets, float* row_loss,
                                                         float* row_lse, int64_t classes, int64_t ignore_index) {
  __shared__ float sm[4];
  const int64_t row = blockIdx.x;
  const int64_t base = row * classes;
  float m = -INFINITY;
#pragma unroll 4
  for (int64_t c = (int64_t)threadIdx.x * 8; c < classes; c += 2048) {
    float v[8];
    Vec8<DT>::load(logits, base + c, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) m = fmaxf(m, v[k]);
  }
  m = pf_block_max<4>(m, sm);
  float z = 0.f;
#pragma unroll 4
  for (int64_t c = (int64_t)threadIdx.x * 8; c < classes; c += 2048) {
    float v[8];
    Vec8<DT>::load(logits, base + c, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) z += expf(v[k] - m);
  }
  z = pf_block_sum<4>(z, sm);
  if (threadIdx.x == 0) {
    const float lse = m + logf(z);
    const int64_t t = targets[row];
    row_lse[row] = lse;
    float l = 0.f;
    if (t != ignore_index) l = (t >= 0 && t < classes) ? lse - pf_load_as_f32(logits, base + t, DT) : NAN;
    row_loss[row] = l;
  }
}

template <int DT, int ODT>
__global__ __launch_bounds__(256) void ce_bwd_vec_kernel(const void* logits, const int64_t* targets,
                                                         const float* row_lse, const float* dloss,
                                                         const float* n_valid, void* dlogits, int64_t classes,
                                                         int64_t ignore_index) {
  const int64_t row = blockIdx.x;
  const int64_t base = row * classes;
  const int64_t t = targets[row];
  const float g = (dloss ? dloss[0] : 1.f) / n_valid[0];
  const float lse = row_lse[row];
  const bool ignored = (t == ignore_index);
#pragma unroll 4
  for (int64_t c = (int64_t)threadIdx.x * 8; c < classes; c += 2048) {
    float v[8];
    Vec8<DT>::load(logits, base + c, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      float o = 0.f;
      if (!ignored) {
        o = expf(v[k] - lse);
        if (c + k == t) o -= 1.f;
        o *= g;
      }
      v[k] = o;
    }
    Vec8<ODT>::store(dlogits, base + c, v);
  }
}

// ---- scalar reductions (MSE, sum) ---------------------------------------------
constexpr int RED_MAX_BLOCKS = 1024;

// mode 0: sum(a) ; mode 1: sum((a-b)^2)
__global__ __launch_bounds__(256) void reduce_partial_kernel(const void* a, int a_dt, const void* b, int b_dt,
                                                             float* partial, int64_t n, int mode) {
  __shared__ float sm[4];
  float s = 0.f;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gsz) {
    float v = pf_load_as_f32(a, i, a_dt);
    if (mode == 1) {
      v -= pf_load_as_f32(b, i, b_dt);
      v *= v;
    }
    s += v;
  }
  s = pf_block_sum<4>(s, sm);
  if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
__global__ __launch_bounds__(256) void reduce_final_kernel(const float* partial, int np, float* out, float scale) {
  __shared__ float sm[4];
  float s = 0.f;
  for (int i = threadIdx.x; i < np; i += 256) s += partial[i];
  s = pf_block_sum<4>(s, sm);
  if (threadIdx.x == 0) out[0] = s * scale;
}

__global__ __launch_bounds__(256) void mse_bwd_kernel(const void* a, int a_dt, const void* b, int b_dt,
                                                      const float* dloss, void* da, int da_dt, int64_t n) {
  const float g = 2.f * (dloss ? dloss[0] : 1.f) / (float)n;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gsz)
    pf_store_from_f32(da, i, da_dt, g * (pf_load_as_f32(a, i, a_dt) - pf_load_as_f32(b, i, b_dt)));
}

inline int red_blocks(int64_t n) {
  int64_t b = (n + 256 * 8 - 1) / (256 * 8);
  if (b < 1) b = 1;
  if (b > RED_MAX_BLOCKS) b = RED_MAX_BLOCKS;
  return (int)b;
}

}  // namespace

extern "C" int pf_softmax_fwd(const float* s, int64_t ld_s, void* p, int p_dtype, int64_t ld_p, int64_t rows,
                              int64_t cols, int64_t q_len, int causal, void* stream) {
  PF_REQUIRE(rows >= 0 && cols >= 0 && ld_s >= cols && ld_p >= cols && pf_is_float_dtype(p_dtype),
             "pf_softmax_fwd: bad arguments");
  if (rows == 0) return PF_OK;
  PF_REQUIRE(s && p, "pf_softmax_fwd: null pointer");
  if (causal) PF_REQUIRE(q_len > 0 && rows % q_len == 0, "pf_softmax_fwd: rows must be a multiple of q_len");
  else q_len = 1;
  hipLaunchKernelGGL(softmax_fwd_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream, s, ld_s,
                     p, p_dtype, ld_p, rows, cols, q_len, causal);
  PF_CHECK_LAUNCH("pf_softmax_fwd");
  return PF_OK;
}

extern "C" int pf_softmax_bwd(const float* dp, int64_t ld_dp, const void* p, int p_dtype, int64_t ld_p, void* ds,
                              int ds_dtype, int64_t ld_ds, int64_t rows, int64_t cols, float scale, void* stream) {
  PF_REQUIRE(rows >= 0 && cols >= 0 && ld_dp >= cols && ld_p >= cols && ld_ds >= cols && pf_is_float_dtype(p_dtype) &&
                 pf_is_float_dtype(ds_dtype),
             "pf_softmax_bwd: bad arguments");
  if (rows == 0) return PF_OK;
  PF_REQUIRE(dp && p && ds, "pf_softmax_bwd: null pointer");
  hipLaunchKernelGGL(softmax_bwd_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream, dp,
                     ld_dp, p, p_dtype, ld_p, ds, ds_dtype, ld_ds, rows, cols, scale);
  PF_CHECK_LAUNCH("pf_softmax_bwd");
  return PF_OK;
}

extern "C" int pf_cross_entropy_fwd(const void* logits, int l_dtype, const int64_t* targets, float* row_loss,
                                    float* row_lse, float* loss, int64_t rows, int64_t classes, int64_t ignore_index,
                                    void* stream) {
  PF_REQUIRE(rows >= 0 && classes > 0 && pf_is_float_dtype(l_dtype), "pf_cross_entropy_fwd: bad arguments");
  PF_REQUIRE(loss, "pf_cross_entropy_fwd: null loss");
  PF_REQUIRE(rows < (1ll << 31), "pf_cross_entropy_fwd: too many rows");
  hipStream_t st = (hipStream_t)stream;
  if (rows > 0) {
    PF_REQUIRE(logits && targets && row_loss && row_lse, "pf_cross_entropy_fwd: null pointer");
    const bool vec = classes % 8 == 0 && pf_aligned(logits, 16);
#define PF_CEF(DT) \
  hipLaunchKernelGGL(ce_fwd_vec_kernel<DT>, dim3((unsigned)rows), dim3(256), 0, st, logits, targets, row_loss, row_lse, classes, ignore_index)
    if (vec && l_dtype == PF_F32) PF_CEF(PF_F32);
    else if (vec && l_dtype == PF_F16) PF_CEF(PF_F16);
    else if (vec && l_dtype == PF_BF16) PF_CEF(PF_BF16);
    else
      hipLaunchKernelGGL(ce_fwd_kernel, dim3((unsigned)rows), dim3(256), 0, st, logits, l_dtype, targets, row_loss,
                         row_lse, classes, ignore_index);
#undef PF_CEF
  }
  hipLaunchKernelGGL(ce_mean_kernel, dim3(1), dim3(256), 0, st, row_loss, targets, loss, rows, ignore_index);
  PF_CHECK_LAUNCH("pf_cross_entropy_fwd");
  return PF_OK;
}

extern "C" int pf_cross_entropy_bwd(const void* logits, int l_dtype, const int64_t* targets, const float* row_lse,
                                    const float* dloss, const float* n_valid, void* dlogits, int dl_dtype,
                                    int64_t rows, int64_t classes, int64_t ignore_index, void* stream) {
  PF_REQUIRE(rows >= 0 && classes > 0 && pf_is_float_dtype(l_dtype) && pf_is_float_dtype(dl_dtype),
             "pf_cross_entropy_bwd: bad arguments");
  if (rows == 0) return PF_OK;
  PF_REQUIRE(logits && targets && row_lse && n_valid && dlogits, "pf_cross_entropy_bwd: null pointer");
  PF_REQUIRE(rows < (1ll << 31), "pf_cross_entropy_bwd: too many rows");
  const bool vec = classes % 8 == 0 && pf_aligned(logits, 16) && pf_aligned(dlogits, 16);
#define PF_CEB(DT, ODT)                                                                                         \
  hipLaunchKernelGGL((ce_bwd_vec_kernel<DT, ODT>), dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, logits, \
                     targets, row_lse, dloss, n_valid, dlogits, classes, ignore_index)
  if (vec && l_dtype == PF_F32 && dl_dtype == PF_F32) PF_CEB(PF_F32, PF_F32);
  else if (vec && l_dtype == PF_F16 && dl_dtype == PF_F16) PF_CEB(PF_F16, PF_F16);
  else if (vec && l_dtype == PF_BF16 && dl_dtype == PF_BF16) PF_CEB(PF_BF16, PF_BF16);
  else if (vec && l_dtype == PF_F32 && dl_dtype == PF_F16) PF_CEB(PF_F32, PF_F16);
  else if (vec && l_dtype == PF_F32 && dl_dtype == PF_BF16) PF_CEB(PF_F32, PF_BF16);
  else
    hipLaunchKernelGGL(ce_bwd_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, logits, l_dtype, targets,
                       row_lse, dloss, n_valid, dlogits, dl_dtype, classes, ignore_index);
#undef PF_CEB
  PF_CHECK_LAUNCH("pf_cross_entropy_bwd");
  return PF_OK;
}

extern "C" int64_t pf_reduce_workspace(int64_t n) {
  (void)n;
  return RED_MAX_BLOCKS;
}

extern "C" int pf_mse_fwd(const void* a, int a_dtype, const void* b, int b_dtype, float* partial, float* loss,
                          int64_t n, void* stream) {
  PF_REQUIRE(n > 0 && pf_is_float_dtype(a_dtype) && pf_is_float_dtype(b_dtype), "pf_mse_fwd: bad arguments");
  PF_REQUIRE(a && b && partial && loss, "pf_mse_fwd: null pointer");
  const int nb = red_blocks(n);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(reduce_partial_kernel, dim3(nb), dim3(256), 0, st, a, a_dtype, b, b_dtype, partial, n, 1);
  hipLaunchKernelGGL(reduce_final_kernel, dim3(1), dim3(256), 0, st, partial, nb, loss, 1.0f / (float)n);
  PF_CHECK_LAUNCH("pf_mse_fwd");
  return PF_OK;
}

extern "C" int pf_mse_bwd(const void* a, int a_dtype, const void* b, int b_dtype, const float* dloss, void* da,
                          int da_dtype, int64_t n, void* stream) {
  PF_REQUIRE(n > 0 && pf_is_float_dtype(a_dtype) && pf_is_float_dtype(b_dtype) && pf_is_float_dtype(da_dtype),
             "pf_mse_bwd: bad arguments");
  PF_REQUIRE(a && b && da, "pf_mse_bwd: null pointer");
  int64_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(mse_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a, a_dtype, b, b_dtype,
                     dloss, da, da_dtype, n);
  PF_CHECK_LAUNCH("pf_mse_bwd");
  return PF_OK;
}

extern "C" int pf_sum_fwd(const void* x, int x_dtype, float* partial, float* loss, int64_t n, void* stream) {
  PF_REQUIRE(n >= 0 && pf_is_float_dtype(x_dtype), "pf_sum_fwd: bad arguments");
  PF_REQUIRE(partial && loss && (x || n == 0), "pf_sum_fwd: null pointer");
  const int nb = red_blocks(n);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(reduce_partial_kernel, dim3(nb), dim3(256), 0, st, x, x_dtype, (const void*)nullptr, 0, partial,
                     n, 0);
  hipLaunchKernelGGL(reduce_final_kernel, dim3(1), dim3(256), 0, st, partial, nb, loss, 1.0f);
  PF_CHECK_LAUNCH("pf_sum_fwd");
  return PF_OK;
}
