// GEMM kernel instantiations for operands stored as float and outputs stored as uint16_t.
#include "gemm_kernels.hpp"

template int dispatch_epi<float, uint16_t>(grl_ctx*, GemmArgs&, int);
template int dispatch_epi_ln<float, uint16_t>(grl_ctx*, GemmArgs&, int);
