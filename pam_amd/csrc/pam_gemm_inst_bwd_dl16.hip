// The matrix kernels with 16-deep k-tiles in mode MODE_BWD_DL (one file per pair: they compile side by side).
#include "pam_gemm_kernel.h"

template void pamgemm::launch_gemm<16, pamgemm::MODE_BWD_DL>(int, int, unsigned, hipStream_t, const pamgemm::GemmArgs&);
