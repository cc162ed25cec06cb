// The row-wise kernels for calls with an offset (see pam_rowops.h).
#define PAM_ROW_OFFSETS 1
#define PAM_ROW_FN(name) pam_row_offset_##name
#include "pam_rowops_kernels.h"
