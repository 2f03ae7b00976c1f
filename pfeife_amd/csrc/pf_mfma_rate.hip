// Measurement aid: the matrix-instruction stream of the 256x256 GEMM tile with nothing else around
// it.  Every wavefront keeps a 4 x 4 grid of 32x32 fp32 accumulator blocks (the register footprint
// of the direct-to-LDS kernel's 4-wavefront tiles) and issues v_mfma_f32_32x32x16 on fragments that
// stay in registers: no loads, no LDS, no barriers.  Timed on all CUs it gives the rate the MFMA
// pipes sustain under the board's power limit with this operand data, the ceiling any GEMM K loop
// on this device can approach (the published peak assumes the full boost clock).
#include "pf_gemm_common.h"

template <int DT>
__global__ __launch_bounds__(256, 1) void mfma_rate_kernel(const uint16_t* __restrict__ operands, int64_t iters,
                                                            float* __restrict__ sink) {
  typedef short short8_t __attribute__((ext_vector_type(8)));
  const int lane = threadIdx.x & 63;
  short8_t fa[4], fb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    fa[i] = *(const short8_t*)(operands + ((i * 64 + lane) * 8));
    fb[i] = *(const short8_t*)(operands + ((256 + i * 64 + lane) * 8));
  }
  float16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = Mfma<DT>::run8(fa[i], fb[j], acc[i][j]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  // every lane's share of the checksum keeps the loop alive; a wavefront's 64 values add up to
  // iters * sum_{i,j} sum(A_i . B_j)
  sink[(int64_t)blockIdx.x * 256 + threadIdx.x] = s;
}

extern "C" int pf_mfma_rate(int dtype, const void* operands, int64_t iters, int workgroups, float* sink, void* stream) {
  PF_REQUIRE(dtype == PF_F16 || dtype == PF_BF16, "pf_mfma_rate: dtype %d is not a 16-bit type", dtype);
  PF_REQUIRE(operands != nullptr && sink != nullptr && pf_aligned(operands, 16), "pf_mfma_rate: operands / sink missing or unaligned");
  PF_REQUIRE(iters > 0 && workgroups > 0 && workgroups <= 65536, "pf_mfma_rate: iters %lld, workgroups %d", (long long)iters, workgroups);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == PF_F16) mfma_rate_kernel<PF_F16><<<workgroups, 256, 0, st>>>((const uint16_t*)operands, iters, sink);
  else mfma_rate_kernel<PF_BF16><<<workgroups, 256, 0, st>>>((const uint16_t*)operands, iters, sink);
  PF_CHECK_LAUNCH("pf_mfma_rate");
  return PF_OK;
}
