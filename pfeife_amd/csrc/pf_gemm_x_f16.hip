// f16 instantiations of the direct-to-LDS MFMA kernel.
#include "pf_gemm_x.h"

int pf_gemm_x_f16(const pf_gemm_desc& d, int tile, hipStream_t st) { return gemm_x_launch<PF_F16>(d, tile, st); }
int pf_gemm_xgroup_f16(const pf_gemm_desc* d, int n, int tile, hipStream_t st) { return gemm_x_group_launch<PF_F16>(d, n, tile, st); }
