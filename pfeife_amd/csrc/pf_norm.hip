// LayerNorm / RMSNorm forward+backward and column reductions (HBM-bound).
//
// One 64-lane wavefront owns one row; row statistics are butterfly reductions
// inside the wavefront (no LDS, no atomics).  A row is re-read from L2 for the
// second/third pass, so HBM sees it once.  Parameter gradients (dgamma, dbeta,
// bias gradients) are reduced deterministically in two stages: per-workgroup
// column partials in a caller-supplied workspace, then one thread per column.
#include <mutex>

#include "pf_common.h"

namespace {

constexpr int COLRED_MAX_BLOCKS = 1024;

// ---- forward ---------------------------------------------------------------
// NV > 0: the row (d <= 64*W*NV) is loaded ONCE into registers, all loads in flight together;
// mean, then the sum of squared deviations, then the output come from the registers: one memory
// round trip per row instead of three dependent ones (the kernel is latency-bound, a row is
// 2-8 KB).  NV == 0: any d, three sweeps over the row (the second and third hit L2).
// XDT / YDT: dtypes of x and y when known at compile time (-1: read x_dt / y_dt at run time).
template <int W, int NV, int XDT = -1, int YDT = -1>
__global__ __launch_bounds__(256) void norm_fwd_kernel(const void* x, int x_dt, const float* gamma, const float* beta,
                                                       void* y, int y_dt, float* mean, float* rstd, int64_t rows,
                                                       int64_t d, float eps, int rms) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  const int64_t base = row * d;
  if constexpr (NV > 0) {
    // nothing around the loads branches: out-of-range lanes read column 0 and are masked out of
    // the sums and the stores; a missing beta reads gamma instead and is not added
    float v[NV][W], g[NV][W], b[NV][W];
    bool ok[NV];
    int64_t col[NV];
    const bool has_beta = beta != nullptr;
    const float* bsrc = has_beta ? beta : gamma;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int64_t c = ((int64_t)lane + i * 64) * W;
      ok[i] = c < d;
      col[i] = ok[i] ? c : 0;
      ld_vec_c<W, XDT>(x, base + col[i], x_dt, v[i]);
      ld_vec_c<W, PF_F32>(gamma, col[i], PF_F32, g[i]);
      ld_vec_c<W, PF_F32>(bsrc, col[i], PF_F32, b[i]);
    }
    float mu = 0.f;
    if (!rms) {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int k = 0; k < W; ++k) s += ok[i] ? v[i][k] : 0.f;
      mu = pf_wave_sum(s) / (float)d;
    }
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
#pragma unroll
      for (int k = 0; k < W; ++k) {
        const float t = v[i][k] - mu;
        q += ok[i] ? t * t : 0.f;
      }
    }
    const float var = pf_wave_sum(q) / (float)d;
    const float rs = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      float o[W];
#pragma unroll
      for (int k = 0; k < W; ++k) {
        const float t = (v[i][k] - mu) * rs * g[i][k];
        o[k] = has_beta ? t + b[i][k] : t;
      }
      if (ok[i]) st_vec_c<W, YDT>(y, base + col[i], y_dt, o);
    }
    if (lane == 0) {
      if (mean) mean[row] = mu;
      rstd[row] = rs;
    }
    return;
  }
  float mu = 0.f;
  if (!rms) {
    float s = 0.f;
    for (int64_t c = (int64_t)lane * W; c < d; c += 64 * W) {
      float v[W];
      ld_vec<W>(x, base + c, x_dt, v);
#pragma unroll
      for (int k = 0; k < W; ++k) s += v[k];
    }
    mu = pf_wave_sum(s) / (float)d;
  }
  float q = 0.f;
  for (int64_t c = (int64_t)lane * W; c < d; c += 64 * W) {
    float v[W];
    ld_vec<W>(x, base + c, x_dt, v);
#pragma unroll
    for (int k = 0; k < W; ++k) {
      const float t = v[k] - mu;
      q += t * t;
    }
  }
  const float var = pf_wave_sum(q) / (float)d;
  const float rs = 1.0f / sqrtf(var + eps);
  for (int64_t c = (int64_t)lane * W; c < d; c += 64 * W) {
    float v[W], g[W], o[W];
    ld_vec<W>(x, base + c, x_dt, v);
    ld_vec<W>(gamma, c, PF_F32, g);
    if (beta) {
      float b[W];
      ld_vec<W>(beta, c, PF_F32, b);
#pragma unroll
      for (int k = 0; k < W; ++k) o[k] = (v[k] - mu) * rs * g[k] + b[k];
    } else {
#pragma unroll
      for (int k = 0; k < W; ++k) o[k] = (v[k] - mu) * rs * g[k];
    }
    st_vec<W>(y, base + c, y_dt, o);
  }
  if (lane == 0) {
    if (mean) mean[row] = mu;
    rstd[row] = rs;
  }
}

// ---- backward ----------------------------------------------------------------
// NV = column groups a lane owns (d <= 64 * W * NV).  Column partials for
// dgamma/dbeta stay in registers across the rows a wavefront processes.
// IODT: dtype of x, dx_add and dx when they all share one known at compile time (-1: run time);
// LPDT: dtype of dx_lp likewise; DYDT: dtype of dy likewise.
template <int W, int NV, int IODT = -1, int LPDT = -1, int DYDT = -1>
__global__ __launch_bounds__(256) void norm_bwd_kernel(const void* dy, int dy_dt, const void* x, int x_dt,
                                                       const float* gamma, const float* mean, const float* rstd,
                                                       const void* dx_add, int add_dt, void* dx, int dx_dt,
                                                       float* ws, int64_t rows, int64_t d, int rms, int want_wgrad,
                                                       void* dx_lp, int lp_dt, int want_colsum) {
  // dx_lp: optional second copy of dx in a 16-bit dtype (what the next matrix product reads);
  // want_colsum: also leave the column sums of that copy's values (the bias gradient of the
  // layer that produced x) as a third partial row.  Partial rows per block: [dgamma, dbeta]
  // or, with want_colsum, [dgamma, dbeta, colsum].
  __shared__ float red[4][64 * W];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr int NS = (NV * W <= 32) ? NV : 1;   // column sums only exist on the register-cached variants
  float pg[NV][W], pb[NV][W], ps[NS][W];
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int k = 0; k < W; ++k) pg[i][k] = pb[i][k] = 0.f;
#pragma unroll
  for (int i = 0; i < NS; ++i)
#pragma unroll
    for (int k = 0; k < W; ++k) ps[i][k] = 0.f;

  constexpr bool CACHE = (NV * W <= 32);   // keep the row's dy and x in registers between the two passes
  // Straight-line variants with at most two column groups per lane: the operands of the wavefront's
  // NEXT row are requested before the current row is reduced and stored, so a wavefront that
  // owns two rows pays one memory round trip, not two.  Nothing around the loads branches (row and
  // column indices are clamped, out-of-range lanes contribute zeros and store nothing).
  constexpr bool PIPE = CACHE && NV <= 4 && IODT >= 0 && DYDT >= 0 && W == 8;
  if constexpr (PIPE) {
    const int64_t stride = (int64_t)gridDim.x * 4;
    int64_t row = (int64_t)blockIdx.x * 4 + wave;
    const bool has_add = dx_add != nullptr;
    bool ok[NV];
    int64_t col[NV];
    float g[NV][W];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int64_t c = ((int64_t)lane + i * 64) * W;
      ok[i] = c < d;
      col[i] = ok[i] ? c : 0;
      ld_vec_c<W, PF_F32>(gamma, col[i], PF_F32, g[i]);
    }
    float ndy[NV][W], nx[NV][W], nadd[NV][W], nmu, nrs;
    auto fetch = [&](int64_t r) {
      const int64_t rr = r < rows ? r : rows - 1;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        ld_vec_c<W, DYDT>(dy, rr * d + col[i], dy_dt, ndy[i]);
        ld_vec_c<W, IODT>(x, rr * d + col[i], x_dt, nx[i]);
        if (has_add) ld_vec_c<W, IODT>(dx_add, rr * d + col[i], add_dt, nadd[i]);
      }
      nmu = rms ? 0.f : mean[rr];
      nrs = rstd[rr];
    };
    if (row < rows) fetch(row);
    while (row < rows) {
      float cdy[NV][W], cx[NV][W], cadd[NV][W];
      const float mu = nmu, rs = nrs;
#pragma unroll
      for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int k = 0; k < W; ++k) {
          cdy[i][k] = ok[i] ? ndy[i][k] : 0.f;
          cx[i][k] = nx[i][k];
          cadd[i][k] = has_add ? nadd[i][k] : 0.f;
        }
      fetch(row + stride);
      float c1 = 0.f, c2 = 0.f;
      float xh[NV][W], gg[NV][W];
#pragma unroll
      for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int k = 0; k < W; ++k) {
          gg[i][k] = cdy[i][k] * g[i][k];
          xh[i][k] = ok[i] ? (cx[i][k] - mu) * rs : 0.f;
          c1 += gg[i][k];
          c2 += gg[i][k] * xh[i][k];
        }
      c1 = rms ? 0.f : pf_wave_sum(c1) / (float)d;
      c2 = pf_wave_sum(c2) / (float)d;
      const int64_t base = row * d;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        float o[W];
#pragma unroll
        for (int k = 0; k < W; ++k) {
          o[k] = rs * (gg[i][k] - c1 - xh[i][k] * c2) + cadd[i][k];
          pg[i][k] += cdy[i][k] * xh[i][k];
          pb[i][k] += cdy[i][k];
        }
        if (ok[i]) {
          st_vec_c<W, IODT>(dx, base + col[i], dx_dt, o);
          if (dx_lp) {
            st_vec_c<W, LPDT>(dx_lp, base + col[i], lp_dt, o);
            if (want_colsum) {
#pragma unroll
              for (int k = 0; k < W; ++k) ps[i][k] += pf_round_to(LPDT >= 0 ? LPDT : lp_dt, o[k]);
            }
          }
        }
      }
      row += stride;
    }
  } else
  for (int64_t row = (int64_t)blockIdx.x * 4 + wave; row < rows; row += (int64_t)gridDim.x * 4) {
    const int64_t base = row * d;
    const float mu = rms ? 0.f : mean[row];
    const float rs = rstd[row];
    float c1 = 0.f, c2 = 0.f;
    float cdy[CACHE ? NV : 1][W], cxh[CACHE ? NV : 1][W], cg[CACHE ? NV : 1][W], cadd[CACHE ? NV : 1][W];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int64_t c = ((int64_t)lane + i * 64) * W;
      if (c < d) {
        float vdy[W], vx[W], g[W];
        ld_vec_c<W, DYDT>(dy, base + c, dy_dt, vdy);
        ld_vec_c<W, IODT>(x, base + c, x_dt, vx);
        ld_vec_c<W, PF_F32>(gamma, c, PF_F32, g);
        // the gradient already accumulated on x: requested with the other operands, so that the
        // row costs one memory round trip, not a second one after the reductions
        if constexpr (CACHE) {
          if (dx_add) ld_vec_c<W, IODT>(dx_add, base + c, add_dt, cadd[i]);
        }
#pragma unroll
        for (int k = 0; k < W; ++k) {
          const float gg = vdy[k] * g[k];
          const float xh = (vx[k] - mu) * rs;
          c1 += gg;
          c2 += gg * xh;
          if constexpr (CACHE) {
            cdy[i][k] = vdy[k];
            cxh[i][k] = xh;
            cg[i][k] = gg;
          }
        }
      }
    }
    c1 = rms ? 0.f : pf_wave_sum(c1) / (float)d;
    c2 = pf_wave_sum(c2) / (float)d;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int64_t c = ((int64_t)lane + i * 64) * W;
      if (c < d) {
        float vdy[W], xhv[W], ggv[W], o[W];
        if constexpr (CACHE) {
#pragma unroll
          for (int k = 0; k < W; ++k) {
            vdy[k] = cdy[i][k];
            xhv[k] = cxh[i][k];
            ggv[k] = cg[i][k];
          }
        } else {
          float vx[W], g[W];
          ld_vec_c<W, DYDT>(dy, base + c, dy_dt, vdy);
          ld_vec_c<W, IODT>(x, base + c, x_dt, vx);
          ld_vec_c<W, PF_F32>(gamma, c, PF_F32, g);
#pragma unroll
          for (int k = 0; k < W; ++k) {
            ggv[k] = vdy[k] * g[k];
            xhv[k] = (vx[k] - mu) * rs;
          }
        }
#pragma unroll
        for (int k = 0; k < W; ++k) {
          o[k] = rs * (ggv[k] - c1 - xhv[k] * c2);
          pg[i][k] += vdy[k] * xhv[k];
          pb[i][k] += vdy[k];
        }
        if (dx_add) {
          if constexpr (CACHE) {
#pragma unroll
            for (int k = 0; k < W; ++k) o[k] += cadd[i][k];
          } else {
            float a[W];
            ld_vec_c<W, IODT>(dx_add, base + c, add_dt, a);
#pragma unroll
            for (int k = 0; k < W; ++k) o[k] += a[k];
          }
        }
        st_vec_c<W, IODT>(dx, base + c, dx_dt, o);
        if (dx_lp) {
          st_vec_c<W, LPDT>(dx_lp, base + c, lp_dt, o);
          if constexpr (NS == NV) {
            if (want_colsum) {
#pragma unroll
              for (int k = 0; k < W; ++k) ps[i][k] += pf_round_to(LPDT >= 0 ? LPDT : lp_dt, o[k]);
            }
          }
        }
      }
    }
  }
  if (!want_wgrad && !want_colsum) return;  // uniform over the block
  // reduce the 4 wavefronts through LDS, then one partial row per block:
  // ws layout [gridDim.x][2 or 3][d]
  const int nrows = want_colsum ? 3 : 2;
  float* wrow = ws + (int64_t)blockIdx.x * nrows * d;
#pragma unroll
  for (int which = 0; which < 3; ++which) {
    if (which < 2 ? !want_wgrad : !want_colsum) continue;   // uniform over the block
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      __syncthreads();
#pragma unroll
      // value k of lane l sits at [k * 64 + l]: consecutive lanes hit consecutive banks
      for (int k = 0; k < W; ++k) red[wave][k * 64 + lane] = which == 0 ? pg[i][k] : (which == 1 ? pb[i][k] : ps[i < NS ? i : 0][k]);
      __syncthreads();
      if (wave == 0) {
        const int64_t c = ((int64_t)lane + i * 64) * W;
        if (c < d) {
#pragma unroll
          for (int k = 0; k < W; ++k) {
            const float s = red[0][k * 64 + lane] + red[1][k * 64 + lane] + red[2][k * 64 + lane] + red[3][k * 64 + lane];
            wrow[which * d + c + k] = s;
          }
        }
      }
    }
  }
}

// acc[c] += sum_p ws[p*stride + c].  A block owns 32 columns; its 8 groups of 32
// threads split the partials, then combine through LDS in a fixed order.
__global__ __launch_bounds__(256) void colreduce_finalize_kernel(const float* ws, int n_partials, int64_t stride,
                                                                 int64_t cols, float* acc) {
  __shared__ float red[8][32];
  const int cl = threadIdx.x & 31, part = threadIdx.x >> 5;
  const int64_t c = (int64_t)blockIdx.x * 32 + cl;
  float s = 0.f;
  if (c < cols)
    for (int p = part; p < n_partials; p += 8) s += ws[(int64_t)p * stride + c];
  red[part][cl] = s;
  __syncthreads();
  if (part == 0 && c < cols) {
    float t = 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) t += red[q][cl];
    acc[c] += t;
  }
}

// column sums of x[rows, cols]: block = 4 wavefronts sharing one 64*W column
// strip, wavefront w takes rows w, w+4, ... of its row chunk.
// XDT: dtype of x when fixed at compile time (-1: run time).
template <int W, int XDT = -1>
__global__ __launch_bounds__(256) void colsum_kernel(const void* x, int x_dt, int64_t rows, int64_t cols, int64_t ld,
                                                     float* ws, int64_t rows_per_chunk) {
  __shared__ float red[4][64 * W];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t c = ((int64_t)blockIdx.x * 64 + lane) * W;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < rows ? r0 + rows_per_chunk : rows;
  float s[W];
#pragma unroll
  for (int k = 0; k < W; ++k) s[k] = 0.f;
  if (c < cols) {
    // 8 rows requested together (the loop is short and latency-bound), summed in row order; rows
    // past the chunk are read from a valid row instead and not added, so that nothing around
    // the loads branches
    for (int64_t r = r0 + wave; r < r1; r += 32) {
      float v[8][W];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int64_t rr = r + 4 * u < r1 ? r + 4 * u : r;
        ld_vec_c<W, XDT>(x, rr * ld + c, x_dt, v[u]);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const bool in = r + 4 * u < r1;
#pragma unroll
        for (int k = 0; k < W; ++k) s[k] += in ? v[u][k] : 0.f;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < W; ++k) red[wave][k * 64 + lane] = s[k];   // lane-contiguous: no bank conflicts
  __syncthreads();
  if (wave == 0 && c < cols) {
#pragma unroll
    for (int k = 0; k < W; ++k)
      ws[(int64_t)blockIdx.y * cols + c + k] =
          red[0][k * 64 + lane] + red[1][k * 64 + lane] + red[2][k * 64 + lane] + red[3][k * 64 + lane];
  }
}


// ---- GroupNorm on channels-last [B, HW, C] tensors ---------------------------------
// statistics: one workgroup per (batch, group); two passes over the group's HW x Cg
// elements (the second one hits L2)
__global__ __launch_bounds__(256) void groupnorm_stats_kernel(const void* x, int x_dt, float* mean, float* rstd,
                                                              int64_t HW, int64_t C, int G, float eps) {
  __shared__ float sm[4];
  const int64_t b = blockIdx.x / G, g = blockIdx.x % G;
  const int64_t Cg = C / G, n = HW * Cg;
  const int64_t base = b * HW * C + g * Cg;
  float s = 0.f;
  for (int64_t e = threadIdx.x; e < n; e += 256) s += pf_load_as_f32(x, base + (e / Cg) * C + e % Cg, x_dt);
  const float mu = pf_block_sum<4>(s, sm) / (float)n;
  float q = 0.f;
  for (int64_t e = threadIdx.x; e < n; e += 256) {
    const float t = pf_load_as_f32(x, base + (e / Cg) * C + e % Cg, x_dt) - mu;
    q += t * t;
  }
  const float var = pf_block_sum<4>(q, sm) / (float)n;
  if (threadIdx.x == 0) {
    mean[blockIdx.x] = mu;
    rstd[blockIdx.x] = 1.0f / sqrtf(var + eps);
  }
}

// Vectorised statistics (channels per group a multiple of 8, the usual case): a pixel's share of
// the group is Cg / 8 chunks of 8 consecutive channels; the workgroup's threads stride over the
// (pixel, chunk) pairs with 16- or 32-byte loads, several in flight per thread.
__global__ __launch_bounds__(256) void groupnorm_stats_vec_kernel(const void* x, int x_dt, float* mean, float* rstd,
                                                                  int HW, int64_t C, int G, float eps) {
  __shared__ float sm[4];
  const int64_t b = blockIdx.x / G, g = blockIdx.x % G;
  const int Cg = (int)(C / G), cpp = Cg / 8, nch = HW * cpp;
  const int64_t base = b * HW * C + g * Cg;
  float s = 0.f;
#pragma unroll 4
  for (int e = threadIdx.x; e < nch; e += 256) {
    float v[8];
    ld_vec<8>(x, base + (int64_t)(e / cpp) * C + (e % cpp) * 8, x_dt, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) s += v[k];
  }
  const float n = (float)HW * (float)Cg;
  const float mu = pf_block_sum<4>(s, sm) / n;
  float q = 0.f;
#pragma unroll 4
  for (int e = threadIdx.x; e < nch; e += 256) {
    float v[8];
    ld_vec<8>(x, base + (int64_t)(e / cpp) * C + (e % cpp) * 8, x_dt, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float t = v[k] - mu;
      q += t * t;
    }
  }
  const float var = pf_block_sum<4>(q, sm) / n;
  if (threadIdx.x == 0) {
    mean[blockIdx.x] = mu;
    rstd[blockIdx.x] = 1.0f / sqrtf(var + eps);
  }
}

// y = (x - mean[b,g]) * rstd[b,g] * gamma[c] + beta[c], 8 channels per thread (Cg % 8 == 0) or 1
template <int W>
__global__ __launch_bounds__(256) void groupnorm_apply_kernel(const void* x, int x_dt, const float* gamma,
                                                              const float* beta, const float* mean,
                                                              const float* rstd, void* y, int y_dt, int64_t total,
                                                              int64_t HW, int64_t C, int G) {
  const int64_t Cg = C / G;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * W; i < total; i += gsz * W) {
    const int64_t c = i % C, b = i / (HW * C);
    const int64_t sg = b * G + c / Cg;
    const float mu = mean[sg], rs = rstd[sg];
    float v[W], gm[W], bt[W];
    ld_vec<W>(x, i, x_dt, v);
    ld_vec<W>(gamma, c, PF_F32, gm);
    ld_vec<W>(beta, c, PF_F32, bt);
#pragma unroll
    for (int k = 0; k < W; ++k) v[k] = (v[k] - mu) * rs * gm[k] + bt[k];
    st_vec<W>(y, i, y_dt, v);
  }
}

// backward statistics: workgroup per (batch, group); lane = channel inside the group
// (Cg <= 64), the 4 wavefronts split the pixels.  Writes c1 = mean(dy*gamma),
// c2 = mean(dy*gamma*xhat) per (b, g) and the per-batch channel sums of dy*xhat and dy.
__global__ __launch_bounds__(256) void groupnorm_bwd_stats_kernel(const void* dy, int dy_dt, const void* x, int x_dt,
                                                                  const float* gamma, const float* mean,
                                                                  const float* rstd, float* c12, float* ws,
                                                                  int64_t HW, int64_t C, int G) {
  __shared__ float sm[4];
  __shared__ float red[2][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t b = blockIdx.x / G, g = blockIdx.x % G;
  const int64_t Cg = C / G;
  const float mu = mean[blockIdx.x], rs = rstd[blockIdx.x];
  float s1 = 0.f, s2 = 0.f, pg = 0.f, pb = 0.f;
  if (lane < Cg) {
    const int64_t c = g * Cg + lane;
    const float gm = gamma[c];
    for (int64_t p = wave; p < HW; p += 4) {
      const int64_t i = (b * HW + p) * C + c;
      const float d = pf_load_as_f32(dy, i, dy_dt);
      const float xh = (pf_load_as_f32(x, i, x_dt) - mu) * rs;
      s1 += d * gm;
      s2 += d * gm * xh;
      pg += d * xh;
      pb += d;
    }
  }
  red[0][wave][lane] = pg;
  red[1][wave][lane] = pb;
  const float n = (float)(HW * Cg);
  s1 = pf_block_sum<4>(s1, sm);
  s2 = pf_block_sum<4>(s2, sm);   // (the block sums synchronise, so `red` is complete below)
  if (threadIdx.x == 0) {
    c12[2 * blockIdx.x] = s1 / n;
    c12[2 * blockIdx.x + 1] = s2 / n;
  }
  if (wave == 0 && lane < Cg) {
    const int64_t c = g * Cg + lane;
    ws[(b * 2) * C + c] = red[0][0][lane] + red[0][1][lane] + red[0][2][lane] + red[0][3][lane];
    ws[(b * 2 + 1) * C + c] = red[1][0][lane] + red[1][1][lane] + red[1][2][lane] + red[1][3][lane];
  }
}

// Vectorised backward statistics (Cg % 8 == 0, Cg <= 64): thread t owns chunk t % cpp of the
// pixels t / cpp, t / cpp + 256 / cpp, ... (the threads past cpp * (256 / cpp) idle), so its eight
// channels are fixed and their partial sums stay in registers; the threads that share a chunk are
// combined through LDS in a fixed order.
__global__ __launch_bounds__(256) void groupnorm_bwd_stats_vec_kernel(const void* dy, int dy_dt, const void* x,
                                                                      int x_dt, const float* gamma, const float* mean,
                                                                      const float* rstd, float* c12, float* ws, int HW,
                                                                      int64_t C, int G) {
  __shared__ float sm[4];
  __shared__ float red[256][17];
  const int64_t b = blockIdx.x / G, g = blockIdx.x % G;
  const int Cg = (int)(C / G), cpp = Cg / 8, ppt = 256 / cpp;   // pixels handled per sweep
  const int t = threadIdx.x, j = t % cpp, p0 = t / cpp;
  const float mu = mean[blockIdx.x], rs = rstd[blockIdx.x];
  float s1 = 0.f, s2 = 0.f, pg[8], pb[8], gm[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) pg[k] = pb[k] = 0.f;
  const int64_t c0 = g * Cg + j * 8;
  ld_vec<8>(gamma, c0, PF_F32, gm);
  if (p0 < ppt) {
#pragma unroll 2
    for (int p = p0; p < HW; p += ppt) {
      const int64_t i = (b * HW + p) * C + c0;
      float d[8], v[8];
      ld_vec<8>(dy, i, dy_dt, d);
      ld_vec<8>(x, i, x_dt, v);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float xh = (v[k] - mu) * rs;
        const float dg = d[k] * gm[k];
        s1 += dg;
        s2 += dg * xh;
        pg[k] += d[k] * xh;
        pb[k] += d[k];
      }
    }
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    red[t][k] = pg[k];
    red[t][8 + k] = pb[k];
  }
  const float n = (float)HW * (float)Cg;
  s1 = pf_block_sum<4>(s1, sm);
  s2 = pf_block_sum<4>(s2, sm);   // (the block sums synchronise, so `red` is complete below)
  if (t == 0) {
    c12[2 * blockIdx.x] = s1 / n;
    c12[2 * blockIdx.x + 1] = s2 / n;
  }
  if (t < Cg) {   // thread t finishes channel t of the group: chunk t / 8, element t % 8
    const int jj = t / 8, k = t % 8;
    float a = 0.f, bsum = 0.f;
    for (int q = 0; q < ppt; ++q) {
      a += red[q * cpp + jj][k];
      bsum += red[q * cpp + jj][8 + k];
    }
    const int64_t c = g * Cg + t;
    ws[(b * 2) * C + c] = a;
    ws[(b * 2 + 1) * C + c] = bsum;
  }
}

template <int W>
__global__ __launch_bounds__(256) void groupnorm_bwd_apply_kernel(const void* dy, int dy_dt, const void* x, int x_dt,
                                                                  const float* gamma, const float* mean,
                                                                  const float* rstd, const float* c12, void* dx,
                                                                  int dx_dt, int64_t total, int64_t HW, int64_t C,
                                                                  int G) {
  const int64_t Cg = C / G;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * W; i < total; i += gsz * W) {
    const int64_t c = i % C, b = i / (HW * C);
    const int64_t sg = b * G + c / Cg;
    const float mu = mean[sg], rs = rstd[sg], c1 = c12[2 * sg], c2 = c12[2 * sg + 1];
    float d[W], v[W], gm[W];
    ld_vec<W>(dy, i, dy_dt, d);
    ld_vec<W>(x, i, x_dt, v);
    ld_vec<W>(gamma, c, PF_F32, gm);
#pragma unroll
    for (int k = 0; k < W; ++k) d[k] = rs * (d[k] * gm[k] - c1 - (v[k] - mu) * rs * c2);
    st_vec<W>(dx, i, dx_dt, d);
  }
}

inline int64_t colsum_chunks(int64_t rows) {
  int64_t chunks = (rows + 31) / 32;
  if (chunks > 256) chunks = 256;
  if (chunks < 1) chunks = 1;
  return chunks;
}

inline int norm_bwd_blocks(int64_t rows) {
  // every workgroup leaves one partial row per parameter gradient (written, then read again by
  // the finishing launch), so their number is kept near two per CU, with the same number of
  // rows for every wavefront.  Measured on 3152 x 1024: 394 workgroups of 2 rows per wavefront
  // take 17.9 us, 788 of one row 20.3 us, 197 of four rows 24.5 us.
  constexpr int64_t target = 512;
  const int64_t per_wave = (rows + 4 * target - 1) / (4 * target);
  int64_t b = (rows + 4 * per_wave - 1) / (4 * per_wave);
  if (b < 1) b = 1;
  if (b > COLRED_MAX_BLOCKS) b = COLRED_MAX_BLOCKS;
  return (int)b;
}

bool vec_ok(const void* p, int dt, int64_t ld) {
  if (!p) return true;
  return pf_aligned(p, 16) && (ld % 8 == 0) && pf_is_float_dtype(dt);
}

int norm_fwd(const void* x, int x_dt, const float* gamma, const float* beta, void* y, int y_dt, float* mean,
             float* rstd, int64_t rows, int64_t d, float eps, int rms, hipStream_t st, const char* name) {
  PF_REQUIRE(rows >= 0 && d > 0, "%s: bad shape rows=%lld d=%lld", name, (long long)rows, (long long)d);
  if (rows == 0) return PF_OK;
  PF_REQUIRE(x && gamma && y && rstd, "%s: null pointer", name);
  PF_REQUIRE(pf_is_float_dtype(x_dt) && pf_is_float_dtype(y_dt), "%s: bad dtype", name);
  PF_REQUIRE((rows + 3) / 4 < (1ll << 31), "%s: too many rows", name);
  const dim3 grid((unsigned)((rows + 3) / 4));
  const bool v = vec_ok(x, x_dt, d) && vec_ok(y, y_dt, d) && vec_ok(gamma, PF_F32, d) && vec_ok(beta, PF_F32, d);
#define PF_NF(W, NV) \
  hipLaunchKernelGGL((norm_fwd_kernel<W, NV>), grid, dim3(256), 0, st, x, x_dt, gamma, beta, y, y_dt, mean, rstd, rows, d, eps, rms)
#define PF_NFC(NV, XD, YD) \
  hipLaunchKernelGGL((norm_fwd_kernel<8, NV, XD, YD>), grid, dim3(256), 0, st, x, x_dt, gamma, beta, y, y_dt, mean, rstd, rows, d, eps, rms)
  // the residual stream is fp32 and the consumers are matrix products (16-bit) or fp32, or the
  // whole stream is 16-bit (a UNet's transformer blocks under autocast): those pairs get
  // straight-line code
#define PF_NFD(NV)                                                     \
  if (x_dt == PF_F32 && y_dt == PF_F16) PF_NFC(NV, PF_F32, PF_F16);     \
  else if (x_dt == PF_F32 && y_dt == PF_BF16) PF_NFC(NV, PF_F32, PF_BF16); \
  else if (x_dt == PF_F32 && y_dt == PF_F32) PF_NFC(NV, PF_F32, PF_F32); \
  else if (x_dt == PF_F16 && y_dt == PF_F16) PF_NFC(NV, PF_F16, PF_F16); \
  else if (x_dt == PF_BF16 && y_dt == PF_BF16) PF_NFC(NV, PF_BF16, PF_BF16); \
  else PF_NF(8, NV)
  if (v && d <= 64 * 8 * 1) { PF_NFD(1); }
  else if (v && d <= 64 * 8 * 2) { PF_NFD(2); }
  else if (v && d <= 64 * 8 * 3) { PF_NFD(3); }
  else if (v && d <= 64 * 8 * 4) { PF_NFD(4); }
  else if (v) PF_NF(8, 0);
  else PF_NF(1, 0);
#undef PF_NFD
#undef PF_NFC
#undef PF_NF
  PF_CHECK_LAUNCH(name);
  return PF_OK;
}

int norm_bwd(const void* dy, int dy_dt, const void* x, int x_dt, const float* gamma, const float* mean,
             const float* rstd, const void* dx_add, int add_dt, void* dx, int dx_dt, float* dgamma, float* dbeta,
             float* ws, int64_t rows, int64_t d, int rms, int defer, hipStream_t st, const char* name,
             void* dx_lp = nullptr, int lp_dt = PF_F16, int want_colsum = 0) {
  PF_REQUIRE(rows >= 0 && d > 0, "%s: bad shape", name);
  if (rows == 0) return PF_OK;
  PF_REQUIRE(dy && x && gamma && rstd && dx, "%s: null pointer", name);
  PF_REQUIRE(rms || mean, "%s: mean required", name);
  PF_REQUIRE(pf_is_float_dtype(dy_dt) && pf_is_float_dtype(x_dt) && pf_is_float_dtype(dx_dt), "%s: bad dtype", name);
  const int want = (dgamma || dbeta || defer) ? 1 : 0;
  if (want || want_colsum) PF_REQUIRE(ws, "%s: workspace required for parameter gradients", name);
  const int blocks = norm_bwd_blocks(rows);
  const bool v = vec_ok(dy, dy_dt, d) && vec_ok(x, x_dt, d) && vec_ok(dx, dx_dt, d) && vec_ok(gamma, PF_F32, d) &&
                 vec_ok(dx_add, dx_add ? add_dt : PF_F32, d) && vec_ok(dx_lp, lp_dt, d);
  if (want_colsum && !(v && d <= 64 * 8 * 4)) {
    pf_set_error("%s: the fused column sum needs 16-byte aligned operands and d <= 2048", name);
    return PF_ERR_UNSUPPORTED;
  }
#define PF_NB(W, NV)                                                                                          \
  hipLaunchKernelGGL((norm_bwd_kernel<W, NV>), dim3(blocks), dim3(256), 0, st, dy, dy_dt, x, x_dt, gamma, mean, \
                     rstd, dx_add, add_dt, dx, dx_dt, ws, rows, d, rms, want, dx_lp, lp_dt, want_colsum)
  // the residual stream and its gradient are fp32, the side copy 16-bit: straight-line variants
  // (the incoming gradient is the 16-bit result of a matrix product, or fp32)
  const bool io32 = x_dt == PF_F32 && dx_dt == PF_F32 && (!dx_add || add_dt == PF_F32);
  // ... or everything is one 16-bit dtype and there is no side copy
  const bool io16 = (x_dt == PF_F16 || x_dt == PF_BF16) && dx_dt == x_dt && dy_dt == x_dt && (!dx_add || add_dt == x_dt) &&
                    !dx_lp;
#define PF_NBC(NV, LP, DY) PF_NBI(NV, PF_F32, LP, DY)
#define PF_NBI(NV, IO, LP, DY)                                                                                       \
  hipLaunchKernelGGL((norm_bwd_kernel<8, NV, IO, LP, DY>), dim3(blocks), dim3(256), 0, st, dy, dy_dt, x, x_dt, gamma, \
                     mean, rstd, dx_add, add_dt, dx, dx_dt, ws, rows, d, rms, want, dx_lp, lp_dt, want_colsum)
#define PF_NBD(NV)                                                                          \
  if (io32 && dy_dt == PF_F16 && (!dx_lp || lp_dt == PF_F16)) PF_NBC(NV, PF_F16, PF_F16);    \
  else if (io32 && dy_dt == PF_BF16 && (!dx_lp || lp_dt == PF_BF16)) PF_NBC(NV, PF_BF16, PF_BF16); \
  else if (io32 && dy_dt == PF_F32 && (!dx_lp || lp_dt == PF_F16)) PF_NBC(NV, PF_F16, PF_F32);    \
  else if (io32 && dy_dt == PF_F32 && lp_dt == PF_BF16) PF_NBC(NV, PF_BF16, PF_F32);         \
  else if (io16 && x_dt == PF_F16) PF_NBI(NV, PF_F16, PF_F16, PF_F16);                       \
  else if (io16 && x_dt == PF_BF16) PF_NBI(NV, PF_BF16, PF_BF16, PF_BF16);                   \
  else PF_NB(8, NV)
  if (v) {
    if (d <= 64 * 8 * 2) { PF_NBD(2); }
    else if (d <= 64 * 8 * 3) { PF_NBD(3); }
    else if (d <= 64 * 8 * 4) { PF_NBD(4); }
    else if (d <= 64 * 8 * 8) PF_NB(8, 8);
    else if (d <= 64 * 8 * 16) PF_NB(8, 16);
    else { pf_set_error("%s: d=%lld exceeds 8192", name, (long long)d); return PF_ERR_UNSUPPORTED; }
  } else {
    if (d <= 64 * 16) PF_NB(1, 16);
    else if (d <= 64 * 64) PF_NB(1, 64);
    else { pf_set_error("%s: unaligned d=%lld exceeds 4096", name, (long long)d); return PF_ERR_UNSUPPORTED; }
  }
#undef PF_NBD
#undef PF_NBC
#undef PF_NBI
#undef PF_NB
  PF_CHECK_LAUNCH(name);
  if (want && !defer) {
    const dim3 fg((unsigned)((d + 31) / 32));
    if (dgamma) hipLaunchKernelGGL(colreduce_finalize_kernel, fg, dim3(256), 0, st, ws, blocks, 2 * d, d, dgamma);
    if (dbeta) hipLaunchKernelGGL(colreduce_finalize_kernel, fg, dim3(256), 0, st, ws + d, blocks, 2 * d, d, dbeta);
    PF_CHECK_LAUNCH(name);
  }
  return PF_OK;
}

}  // namespace

// fp32 elements needed by the two-stage column reductions over a [rows, cols]
// matrix: the norm backward writes 2 partial rows per workgroup, the column sum
// one partial row per row chunk.
// One launch finishing many deferred column reductions: block (x, y) handles 128 columns of
// item y (four per lane, 16-byte loads, up to eight partial rows in flight per lane) when the item's
// rows are 16-byte aligned, else 32 columns.  Items live in device memory.  Per column the partial
// rows are summed in a fixed order: rows part, part + 8, ... by group `part`, then the eight groups.
__global__ __launch_bounds__(256) void colreduce_finalize_batch_kernel(const pf_reduce_item* items) {
  __shared__ float red[8][128];
  const pf_reduce_item it = items[blockIdx.y];
  const int cl = threadIdx.x & 31, part = threadIdx.x >> 5;
  const bool vec = ((((uintptr_t)it.ws) | ((uintptr_t)it.acc)) & 15) == 0 && it.stride % 4 == 0 && it.cols % 4 == 0;
  if (vec) {
    if ((int64_t)blockIdx.x * 128 >= it.cols) return;  // uniform over the block
    const int64_t c = (int64_t)blockIdx.x * 128 + cl * 4;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c < it.cols) {
      int p = part;
      for (; p + 56 < it.n_partials; p += 64) {   // eight partial rows in flight, added in row order
        float4 a[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) a[u] = *(const float4*)(it.ws + (int64_t)(p + 8 * u) * it.stride + c);
#pragma unroll
        for (int u = 0; u < 8; ++u) { s.x += a[u].x; s.y += a[u].y; s.z += a[u].z; s.w += a[u].w; }
      }
      for (; p + 24 < it.n_partials; p += 32) {
        const float4 a0 = *(const float4*)(it.ws + (int64_t)p * it.stride + c);
        const float4 a1 = *(const float4*)(it.ws + (int64_t)(p + 8) * it.stride + c);
        const float4 a2 = *(const float4*)(it.ws + (int64_t)(p + 16) * it.stride + c);
        const float4 a3 = *(const float4*)(it.ws + (int64_t)(p + 24) * it.stride + c);
        s.x += a0.x; s.y += a0.y; s.z += a0.z; s.w += a0.w;
        s.x += a1.x; s.y += a1.y; s.z += a1.z; s.w += a1.w;
        s.x += a2.x; s.y += a2.y; s.z += a2.z; s.w += a2.w;
        s.x += a3.x; s.y += a3.y; s.z += a3.z; s.w += a3.w;
      }
      for (; p < it.n_partials; p += 8) {
        const float4 a = *(const float4*)(it.ws + (int64_t)p * it.stride + c);
        s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
      }
    }
    *(float4*)&red[part][cl * 4] = s;
    __syncthreads();
    if (part == 0 && c < it.cols) {
      float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float4 r = *(const float4*)&red[q][cl * 4];
        t.x += r.x; t.y += r.y; t.z += r.z; t.w += r.w;
      }
      float4 a = *(float4*)(it.acc + c);
      a.x += t.x; a.y += t.y; a.z += t.z; a.w += t.w;
      *(float4*)(it.acc + c) = a;
    }
    return;
  }
  // four 32-column strips per block, one after the other (same grid as the vector path)
  for (int strip = 0; strip < 4; ++strip) {
    const int64_t c0 = ((int64_t)blockIdx.x * 4 + strip) * 32;
    if (c0 >= it.cols) return;  // uniform over the block
    const int64_t c = c0 + cl;
    float s = 0.f;
    if (c < it.cols)
      for (int p = part; p < it.n_partials; p += 8) s += it.ws[(int64_t)p * it.stride + c];
    __syncthreads();
    red[part][cl] = s;
    __syncthreads();
    if (part == 0 && c < it.cols) {
      float t = 0.f;
#pragma unroll
      for (int q = 0; q < 8; ++q) t += red[q][cl];
      it.acc[c] += t;
    }
  }
}

extern "C" int pf_norm_bwd_fused(const pf_norm_bwd_desc* n, void* stream) {
  PF_REQUIRE(n != nullptr, "pf_norm_bwd_fused: null descriptor");
  PF_REQUIRE(!n->dx_lp || n->dx_lp_dtype == PF_F16 || n->dx_lp_dtype == PF_BF16,
             "pf_norm_bwd_fused: the second copy of dx is fp16 or bf16");
  PF_REQUIRE(!n->want_colsum || n->dx_lp, "pf_norm_bwd_fused: column sums are taken over the 16-bit copy");
  return norm_bwd(n->dy, n->dy_dtype, n->x, n->x_dtype, n->gamma, n->mean, n->rstd, n->dx_add, n->add_dtype, n->dx,
                  n->dx_dtype, nullptr, nullptr, n->workspace, n->rows, n->d, n->mean == nullptr ? 1 : 0,
                  n->want_wgrad ? 1 : 0, (hipStream_t)stream, "pf_norm_bwd_fused", n->dx_lp, n->dx_lp_dtype,
                  n->want_colsum ? 1 : 0);
}

extern "C" int pf_norm_bwd_partials(int64_t rows) { return norm_bwd_blocks(rows < 1 ? 1 : rows); }

extern "C" int pf_colsum_partials(int64_t rows) {
  if (rows < 1) rows = 1;
  int64_t chunks = colsum_chunks(rows);
  const int64_t rpc = (rows + chunks - 1) / chunks;
  return (int)((rows + rpc - 1) / rpc);
}

extern "C" int pf_colreduce_finalize_batch(const pf_reduce_item* items_dev, int n_items, int64_t max_cols,
                                           void* stream) {
  PF_REQUIRE(n_items >= 0 && max_cols >= 0, "pf_colreduce_finalize_batch: bad arguments");
  if (n_items == 0 || max_cols == 0) return PF_OK;
  PF_REQUIRE(items_dev != nullptr && n_items <= 65535, "pf_colreduce_finalize_batch: bad item list");
  hipLaunchKernelGGL(colreduce_finalize_batch_kernel, dim3((unsigned)((max_cols + 127) / 128), (unsigned)n_items),
                     dim3(256), 0, (hipStream_t)stream, items_dev);
  PF_CHECK_LAUNCH("pf_colreduce_finalize_batch");
  return PF_OK;
}

extern "C" int64_t pf_colreduce_workspace(int64_t rows, int64_t cols) {
  if (cols < 1) cols = 1;
  if (rows < 1) rows = 1;
  const int64_t norm = 2 * (int64_t)norm_bwd_blocks(rows) * cols;
  const int64_t colsum = colsum_chunks(rows) * cols;
  return norm > colsum ? norm : colsum;
}

extern "C" int pf_layernorm_fwd(const void* x, int x_dtype, const float* gamma, const float* beta, void* y,
                                int y_dtype, float* mean, float* rstd, int64_t rows, int64_t d, float eps,
                                void* stream) {
  PF_REQUIRE(mean != nullptr || rows == 0, "pf_layernorm_fwd: mean required");
  return norm_fwd(x, x_dtype, gamma, beta, y, y_dtype, mean, rstd, rows, d, eps, 0, (hipStream_t)stream,
                  "pf_layernorm_fwd");
}

extern "C" int pf_layernorm_bwd(const void* dy, int dy_dtype, const void* x, int x_dtype, const float* gamma,
                                const float* mean, const float* rstd, const void* dx_add, int add_dtype, void* dx,
                                int dx_dtype, float* dgamma_acc, float* dbeta_acc, float* workspace, int64_t rows,
                                int64_t d, int defer_reduce, void* stream) {
  return norm_bwd(dy, dy_dtype, x, x_dtype, gamma, mean, rstd, dx_add, add_dtype, dx, dx_dtype, dgamma_acc,
                  dbeta_acc, workspace, rows, d, 0, defer_reduce, (hipStream_t)stream, "pf_layernorm_bwd");
}

extern "C" int pf_rmsnorm_fwd(const void* x, int x_dtype, const float* gamma, void* y, int y_dtype, float* rstd,
                              int64_t rows, int64_t d, float eps, void* stream) {
  return norm_fwd(x, x_dtype, gamma, nullptr, y, y_dtype, nullptr, rstd, rows, d, eps, 1, (hipStream_t)stream,
                  "pf_rmsnorm_fwd");
}

extern "C" int pf_rmsnorm_bwd(const void* dy, int dy_dtype, const void* x, int x_dtype, const float* gamma,
                              const float* rstd, const void* dx_add, int add_dtype, void* dx, int dx_dtype,
                              float* dgamma_acc, float* workspace, int64_t rows, int64_t d, int defer_reduce,
                              void* stream) {
  return norm_bwd(dy, dy_dtype, x, x_dtype, gamma, nullptr, rstd, dx_add, add_dtype, dx, dx_dtype, dgamma_acc,
                  nullptr, workspace, rows, d, 1, defer_reduce, (hipStream_t)stream, "pf_rmsnorm_bwd");
}


extern "C" int pf_groupnorm_fwd(const void* x, int x_dtype, const float* gamma, const float* beta, void* y,
                                int y_dtype, float* mean, float* rstd, int64_t B, int64_t HW, int64_t C, int groups,
                                float eps, void* stream) {
  PF_REQUIRE(B >= 0 && HW > 0 && C > 0 && groups > 0 && C % groups == 0, "pf_groupnorm_fwd: bad shape");
  if (B == 0) return PF_OK;
  PF_REQUIRE(x && gamma && beta && y && mean && rstd, "pf_groupnorm_fwd: null pointer");
  PF_REQUIRE(pf_is_float_dtype(x_dtype) && pf_is_float_dtype(y_dtype), "pf_groupnorm_fwd: bad dtype");
  PF_REQUIRE(B * groups < (1ll << 31), "pf_groupnorm_fwd: too many groups");
  hipStream_t st = (hipStream_t)stream;
  const int64_t total = B * HW * C;
  const bool v = (C / groups) % 8 == 0 && vec_ok(x, x_dtype, C) && vec_ok(y, y_dtype, C) && vec_ok(gamma, PF_F32, C) &&
                 vec_ok(beta, PF_F32, C);
  if ((C / groups) % 8 == 0 && vec_ok(x, x_dtype, C) && HW * (C / groups) < (1ll << 31))
    hipLaunchKernelGGL(groupnorm_stats_vec_kernel, dim3((unsigned)(B * groups)), dim3(256), 0, st, x, x_dtype, mean, rstd,
                       (int)HW, C, groups, eps);
  else
    hipLaunchKernelGGL(groupnorm_stats_kernel, dim3((unsigned)(B * groups)), dim3(256), 0, st, x, x_dtype, mean, rstd, HW,
                       C, groups, eps);
  int64_t blocks = (total / (v ? 8 : 1) + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (blocks < 1) blocks = 1;
  if (v) hipLaunchKernelGGL(groupnorm_apply_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, st, x, x_dtype, gamma, beta, mean, rstd, y, y_dtype, total, HW, C, groups);
  else hipLaunchKernelGGL(groupnorm_apply_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, st, x, x_dtype, gamma, beta, mean, rstd, y, y_dtype, total, HW, C, groups);
  PF_CHECK_LAUNCH("pf_groupnorm_fwd");
  return PF_OK;
}

extern "C" int pf_groupnorm_bwd(const void* dy, int dy_dtype, const void* x, int x_dtype, const float* gamma,
                                const float* mean, const float* rstd, void* dx, int dx_dtype, float* dgamma_acc,
                                float* dbeta_acc, float* workspace, int64_t B, int64_t HW, int64_t C, int groups,
                                int defer_reduce, void* stream) {
  PF_REQUIRE(B >= 0 && HW > 0 && C > 0 && groups > 0 && C % groups == 0, "pf_groupnorm_bwd: bad shape");
  if (B == 0) return PF_OK;
  PF_REQUIRE(C / groups <= 64, "pf_groupnorm_bwd: more than 64 channels per group");
  PF_REQUIRE(dy && x && gamma && mean && rstd && dx && workspace, "pf_groupnorm_bwd: null pointer");
  PF_REQUIRE(pf_is_float_dtype(dy_dtype) && pf_is_float_dtype(x_dtype) && pf_is_float_dtype(dx_dtype),
             "pf_groupnorm_bwd: bad dtype");
  hipStream_t st = (hipStream_t)stream;
  float* ws = workspace;                 // [B][2][C] channel partials
  float* c12 = workspace + B * 2 * C;    // [B*G][2]
  const int64_t total = B * HW * C;
  const bool v = (C / groups) % 8 == 0 && vec_ok(dy, dy_dtype, C) && vec_ok(x, x_dtype, C) && vec_ok(dx, dx_dtype, C) &&
                 vec_ok(gamma, PF_F32, C);
  if ((C / groups) % 8 == 0 && vec_ok(dy, dy_dtype, C) && vec_ok(x, x_dtype, C) && vec_ok(gamma, PF_F32, C) &&
      HW < (1ll << 31))
    hipLaunchKernelGGL(groupnorm_bwd_stats_vec_kernel, dim3((unsigned)(B * groups)), dim3(256), 0, st, dy, dy_dtype, x,
                       x_dtype, gamma, mean, rstd, c12, ws, (int)HW, C, groups);
  else
    hipLaunchKernelGGL(groupnorm_bwd_stats_kernel, dim3((unsigned)(B * groups)), dim3(256), 0, st, dy, dy_dtype, x,
                       x_dtype, gamma, mean, rstd, c12, ws, HW, C, groups);
  int64_t blocks = (total / (v ? 8 : 1) + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (blocks < 1) blocks = 1;
  if (v) hipLaunchKernelGGL(groupnorm_bwd_apply_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, st, dy, dy_dtype, x, x_dtype, gamma, mean, rstd, c12, dx, dx_dtype, total, HW, C, groups);
  else hipLaunchKernelGGL(groupnorm_bwd_apply_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, st, dy, dy_dtype, x, x_dtype, gamma, mean, rstd, c12, dx, dx_dtype, total, HW, C, groups);
  PF_CHECK_LAUNCH("pf_groupnorm_bwd");
  if (!defer_reduce) {
    const dim3 fg((unsigned)((C + 31) / 32));
    if (dgamma_acc) hipLaunchKernelGGL(colreduce_finalize_kernel, fg, dim3(256), 0, st, ws, (int)B, 2 * C, C, dgamma_acc);
    if (dbeta_acc) hipLaunchKernelGGL(colreduce_finalize_kernel, fg, dim3(256), 0, st, ws + C, (int)B, 2 * C, C, dbeta_acc);
    PF_CHECK_LAUNCH("pf_groupnorm_bwd(finalize)");
  }
  return PF_OK;
}

extern "C" int64_t pf_groupnorm_workspace(int64_t B, int64_t C, int groups) { return B * 2 * C + B * groups * 2; }

extern "C" int pf_colsum_accumulate(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld, float* acc,
                                    float* workspace, int defer_reduce, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  PF_REQUIRE(rows >= 0 && cols >= 0 && ld >= cols, "pf_colsum_accumulate: bad shape");
  if (rows == 0 || cols == 0) return PF_OK;
  PF_REQUIRE(x && (acc || defer_reduce) && workspace, "pf_colsum_accumulate: null pointer");
  PF_REQUIRE(pf_is_float_dtype(x_dtype), "pf_colsum_accumulate: bad dtype");
  int64_t chunks = colsum_chunks(rows);
  const int64_t rpc = (rows + chunks - 1) / chunks;
  chunks = (rows + rpc - 1) / rpc;
  const bool v = vec_ok(x, x_dtype, ld) && cols % 8 == 0;
  if (v) {
    const dim3 grid((unsigned)((cols + 511) / 512), (unsigned)chunks);
#define PF_CS(DT) hipLaunchKernelGGL((colsum_kernel<8, DT>), grid, dim3(256), 0, st, x, x_dtype, rows, cols, ld, workspace, rpc)
    if (x_dtype == PF_F16) PF_CS(PF_F16);
    else if (x_dtype == PF_BF16) PF_CS(PF_BF16);
    else PF_CS(PF_F32);
#undef PF_CS
  } else {
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)chunks);
    hipLaunchKernelGGL(colsum_kernel<1>, grid, dim3(256), 0, st, x, x_dtype, rows, cols, ld, workspace, rpc);
  }
  PF_CHECK_LAUNCH("pf_colsum_accumulate");
  if (defer_reduce) return PF_OK;
  hipLaunchKernelGGL(colreduce_finalize_kernel, dim3((unsigned)((cols + 31) / 32)), dim3(256), 0, st, workspace,
                     (int)chunks, cols, cols, acc);
  PF_CHECK_LAUNCH("pf_colsum_accumulate(finalize)");
  return PF_OK;
}


// ---- column sum without any allocation ---------------------------------------------------
// The partial rows of the two-stage column reduction live in a device array that is part of
// the library image (each GPU the library runs on holds its own copy until the process ends)
// instead of a caller-supplied workspace.  Host code may only use the array's device address,
// fetched once per device with that device current; the array's name is a host-side stand-in.
constexpr int64_t STATIC_SCRATCH_FLOATS = 256 * 8192;   // 256 partial rows x 8192 columns = 8 MiB
static __device__ __align__(256) float pf_colsum_scratch[STATIC_SCRATCH_FLOATS];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[MAX_DEVICES] = {};

// address of the current device's copy of the scratch array (looked up once per device)
int scratch_for_current_device(float** out, const char* who) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    pf_set_error("%s: cannot identify the current device (%s)", who, e == hipSuccess ? "index out of range" : hipGetErrorString(e));
    return PF_ERR_HIP;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(pf_colsum_scratch));
    if (e != hipSuccess || p == nullptr) {
      pf_set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev, hipGetErrorString(e));
      return PF_ERR_HIP;
    }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return PF_OK;
}
}  // namespace

// called by pf_init with the device current
int pf_norm_init_device() {
  float* p = nullptr;
  return scratch_for_current_device(&p, "pf_init");
}

extern "C" int64_t pf_colsum_static_capacity(void) { return STATIC_SCRATCH_FLOATS; }

extern "C" int pf_colsum_accumulate_static(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld,
                                           float* acc, void* stream) {
  PF_REQUIRE(rows >= 0 && cols >= 0 && ld >= cols, "pf_colsum_accumulate_static: bad shape");
  if (rows == 0 || cols == 0) return PF_OK;
  PF_REQUIRE(x && acc, "pf_colsum_accumulate_static: null pointer");
  const int64_t need = (int64_t)pf_colsum_partials(rows) * cols;
  PF_REQUIRE(need <= STATIC_SCRATCH_FLOATS,
             "pf_colsum_accumulate_static: %lld partial rows x %lld columns = %lld floats exceed the built-in scratch "
             "of %lld floats; use pf_colsum_accumulate with a workspace",
             (long long)pf_colsum_partials(rows), (long long)cols, (long long)need, (long long)STATIC_SCRATCH_FLOATS);
  float* scratch = nullptr;
  const int rc = scratch_for_current_device(&scratch, "pf_colsum_accumulate_static");
  if (rc != PF_OK) return rc;
  // every partial the finalize pass reads is written by this call's first pass: nothing to clear
  return pf_colsum_accumulate(x, x_dtype, rows, cols, ld, acc, scratch, 0, stream);
}
