// One (operand dtype, tile shape) pair of the direct-to-LDS MFMA kernel per object file: the
// build compiles this source once per pair with -DPF_X_DT=<PF_F16|PF_BF16 value> -DPF_X_TILE=<PF_XT_* value>
// (the instantiations of one pair take about half a minute to compile; the pairs build in parallel).
#include "pf_gemm_x.h"

#if !defined(PF_X_DT) || !defined(PF_X_TILE)
#error "compile with -DPF_X_DT=<dtype id> -DPF_X_TILE=<tile id>"
#endif

#define PF_X_CAT_(a, b, c, d) a##b##c##d
#define PF_X_CAT(a, b, c, d) PF_X_CAT_(a, b, c, d)

// pf_gemm_x_<dtype id>_<tile id>, pf_gemm_xgroup_<dtype id>_<tile id>: looked up through the table in pf_gemm.hip
int PF_X_CAT(pf_gemm_x_, PF_X_DT, _, PF_X_TILE)(const pf_gemm_desc& d, hipStream_t st) {
  return gemm_x_launch<PF_X_DT, PF_X_TILE>(d, st);
}
int PF_X_CAT(pf_gemm_xgroup_, PF_X_DT, _, PF_X_TILE)(const pf_gemm_desc* d, int n, hipStream_t st) {
  return gemm_x_group_launch<PF_X_DT, PF_X_TILE>(d, n, st);
}
