// Micro-batch split / merge (row gather / scatter of raw bytes) and the
// embedding lookup with its gradient.
//
// The split of pfeife/batch.py:45 is torch.tensor_split along dim 0; a chunk of
// a contiguous tensor is a contiguous run of rows, so the gather moves whole
// rows in the widest unit (16, 4 or 1 byte) that the alignment of source,
// destination and row size allows.  An optional int64 row index turns the same
// kernel into a general gather (and the scatter into a general row scatter).
#include "pf_common.h"

namespace {

template <typename U>
__global__ __launch_bounds__(256) void row_move_kernel(const char* src, char* dst, int64_t units_per_row,
                                                       int64_t row_start, int64_t n_rows, const int64_t* index,
                                                       int scatter) {
  const int64_t total = units_per_row * n_rows;
  const int64_t gsz = (int64_t)gridDim.x * blockDim.x;
  for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < total; u += gsz) {
    const int64_t r = u / units_per_row, o = u % units_per_row;
    const int64_t far = index ? index[r] : row_start + r;  // row in the un-split tensor
    const int64_t s = scatter ? r : far, d = scatter ? far : r;
    ((U*)dst)[d * units_per_row + o] = ((const U*)src)[s * units_per_row + o];
  }
}

int row_move(const void* src, void* dst, int64_t row_bytes, int64_t row_start, int64_t n_rows, const int64_t* index,
             int scatter, hipStream_t st, const char* name) {
  PF_REQUIRE(row_bytes >= 0 && n_rows >= 0 && row_start >= 0, "%s: bad arguments", name);
  if (row_bytes == 0 || n_rows == 0) return PF_OK;
  PF_REQUIRE(src && dst, "%s: null pointer", name);
  int unit = 1;
  if (row_bytes % 16 == 0 && pf_aligned(src, 16) && pf_aligned(dst, 16)) unit = 16;
  else if (row_bytes % 4 == 0 && pf_aligned(src, 4) && pf_aligned(dst, 4)) unit = 4;
  const int64_t upr = row_bytes / unit;
  int64_t blocks = (upr * n_rows + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  const dim3 grid((unsigned)blocks);
  if (unit == 16)
    hipLaunchKernelGGL(row_move_kernel<uint4>, grid, dim3(256), 0, st, (const char*)src, (char*)dst, upr, row_start,
                       n_rows, index, scatter);
  else if (unit == 4)
    hipLaunchKernelGGL(row_move_kernel<uint32_t>, grid, dim3(256), 0, st, (const char*)src, (char*)dst, upr, row_start,
                       n_rows, index, scatter);
  else
    hipLaunchKernelGGL(row_move_kernel<uint8_t>, grid, dim3(256), 0, st, (const char*)src, (char*)dst, upr, row_start,
                       n_rows, index, scatter);
  PF_CHECK_LAUNCH(name);
  return PF_OK;
}

template <int W>
__global__ __launch_bounds__(256) void embedding_fwd_kernel(const void* table, int t_dt, const int64_t* ids, void* out,
                                                            int o_dt, int64_t dim, int64_t vocab) {
  const int64_t i = blockIdx.x;
  int64_t id = ids[i];
  const bool ok = id >= 0 && id < vocab;
  for (int64_t c = (int64_t)threadIdx.x * W; c < dim; c += 256 * W) {
    float v[W];
    if (ok) ld_vec<W>(table, id * dim + c, t_dt, v);
    else {
#pragma unroll
      for (int k = 0; k < W; ++k) v[k] = NAN;  // an out-of-range id is visible, never a wild read
    }
    st_vec<W>(out, i * dim + c, o_dt, v);
  }
}

// One wavefront owns EMB_ROWS consecutive vocabulary rows: it scans the id list once, 64 entries
// at a time (the next 64 are already in flight), and adds the output-gradient rows whose id
// falls in its range, in id-list order.  No two wavefronts write the same row and the
// summation order within a row is the list order, so the result is deterministic; the id list
// is read vocab / EMB_ROWS times instead of once per row.  Ids outside [0, vocab) and the
// padding index (whose row keeps a zero gradient, as in aten::embedding_dense_backward) match
// no wavefront.
constexpr int EMB_ROWS = 16;

template <int W>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const void* dout, int d_dt, const int64_t* ids,
                                                            float* dtable, int64_t n_ids, int64_t dim, int64_t vocab,
                                                            int64_t padding_idx) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t v0 = ((int64_t)blockIdx.x * 4 + wave) * EMB_ROWS;
  if (v0 >= vocab) return;
  const int64_t v1 = v0 + EMB_ROWS < vocab ? v0 + EMB_ROWS : vocab;
  int64_t next = lane < n_ids ? ids[lane] : -1;
  for (int64_t base = 0; base < n_ids; base += 64) {
    const int64_t id = next;
    const int64_t jn = base + 64 + lane;
    next = jn < n_ids ? ids[jn] : -1;
    const bool hit = id >= v0 && id < v1 && id != padding_idx;
    unsigned long long mask = __ballot(hit);
    while (mask) {
      const int b = __ffsll((long long)mask) - 1;
      mask &= mask - 1;
      const int64_t r = base + b;
      const int64_t v = __shfl(id, b);
      for (int64_t c = (int64_t)lane * W; c < dim; c += 64 * W) {
        float g[W], a[W];
        ld_vec<W>(dout, r * dim + c, d_dt, g);
        ld_vec<W>(dtable, v * dim + c, PF_F32, a);
#pragma unroll
        for (int k = 0; k < W; ++k) a[k] += g[k];
        st_vec<W>(dtable, v * dim + c, PF_F32, a);
      }
    }
  }
}

}  // namespace

extern "C" int pf_split_gather(const void* src, void* dst, int64_t row_bytes, int64_t row_start, int64_t n_rows,
                               const int64_t* index, void* stream) {
  return row_move(src, dst, row_bytes, row_start, n_rows, index, 0, (hipStream_t)stream, "pf_split_gather");
}

extern "C" int pf_merge_scatter(const void* src, void* dst, int64_t row_bytes, int64_t row_start, int64_t n_rows,
                                const int64_t* index, void* stream) {
  return row_move(src, dst, row_bytes, row_start, n_rows, index, 1, (hipStream_t)stream, "pf_merge_scatter");
}

extern "C" int pf_embedding_fwd(const void* table, int t_dtype, const int64_t* ids, void* out, int o_dtype,
                                int64_t n_ids, int64_t dim, int64_t vocab, void* stream) {
  PF_REQUIRE(n_ids >= 0 && dim > 0 && vocab > 0 && pf_is_float_dtype(t_dtype) && pf_is_float_dtype(o_dtype),
             "pf_embedding_fwd: bad arguments");
  if (n_ids == 0) return PF_OK;
  PF_REQUIRE(table && ids && out, "pf_embedding_fwd: null pointer");
  PF_REQUIRE(n_ids < (1ll << 31), "pf_embedding_fwd: too many ids");
  const bool vec = dim % 8 == 0 && pf_aligned(table, 16) && pf_aligned(out, 16);
  if (vec)
    hipLaunchKernelGGL(embedding_fwd_kernel<8>, dim3((unsigned)n_ids), dim3(256), 0, (hipStream_t)stream, table,
                       t_dtype, ids, out, o_dtype, dim, vocab);
  else
    hipLaunchKernelGGL(embedding_fwd_kernel<1>, dim3((unsigned)n_ids), dim3(256), 0, (hipStream_t)stream, table,
                       t_dtype, ids, out, o_dtype, dim, vocab);
  PF_CHECK_LAUNCH("pf_embedding_fwd");
  return PF_OK;
}

extern "C" int pf_embedding_bwd(const void* dout, int d_dtype, const int64_t* ids, float* dtable_acc, int64_t n_ids,
                                int64_t dim, int64_t vocab, int64_t padding_idx, void* stream) {
  PF_REQUIRE(n_ids >= 0 && dim > 0 && vocab > 0 && pf_is_float_dtype(d_dtype), "pf_embedding_bwd: bad arguments");
  PF_REQUIRE(padding_idx >= -1 && padding_idx < vocab, "pf_embedding_bwd: padding_idx must be -1 (none) or a row");
  if (n_ids == 0) return PF_OK;
  PF_REQUIRE(dout && ids && dtable_acc, "pf_embedding_bwd: null pointer");
  const bool vec = dim % 8 == 0 && pf_aligned(dout, 16) && pf_aligned(dtable_acc, 16);
  const dim3 grid((unsigned)((vocab + 4 * EMB_ROWS - 1) / (4 * EMB_ROWS)));
  if (vec)
    hipLaunchKernelGGL(embedding_bwd_kernel<8>, grid, dim3(256), 0, (hipStream_t)stream, dout, d_dtype, ids,
                       dtable_acc, n_ids, dim, vocab, padding_idx);
  else
    hipLaunchKernelGGL(embedding_bwd_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, dout, d_dtype, ids,
                       dtable_acc, n_ids, dim, vocab, padding_idx);
  PF_CHECK_LAUNCH("pf_embedding_bwd");
  return PF_OK;
}
