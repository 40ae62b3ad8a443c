// GEMM kernel instantiations for operands stored as float and outputs stored as float.
#include "gemm_kernels.hpp"

template int dispatch_epi<float, float>(grl_ctx*, GemmArgs&, int);
template int dispatch_epi_ln<float, float>(grl_ctx*, GemmArgs&, int);
template int launch_gemm_resln<float, float>(grl_ctx*, GemmArgs&, int*);
