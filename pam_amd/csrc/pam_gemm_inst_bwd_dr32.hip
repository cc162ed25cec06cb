// The matrix kernels with 32-deep k-tiles in mode MODE_BWD_DR (one file per pair: they compile side by side).
#include "pam_gemm_kernel.h"

template void pamgemm::launch_gemm<32, pamgemm::MODE_BWD_DR>(int, int, unsigned, hipStream_t, const pamgemm::GemmArgs&);
