// GEMM kernel instantiations for operands stored as uint16_t and outputs stored as uint16_t.
#include "gemm_kernels.hpp"

template int dispatch_epi<uint16_t, uint16_t>(grl_ctx*, GemmArgs&, int);
template int dispatch_epi_ln<uint16_t, uint16_t>(grl_ctx*, GemmArgs&, int);
template int launch_gemm_resln<uint16_t, uint16_t>(grl_ctx*, GemmArgs&, int*);
