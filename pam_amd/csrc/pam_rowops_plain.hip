// The row-wise kernels for calls without an offset (see pam_rowops.h).
#define PAM_ROW_OFFSETS 0
#define PAM_ROW_FN(name) pam_row_plain_##name
#include "pam_rowops_kernels.h"
