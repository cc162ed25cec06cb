// Entry points of the row-wise kernels: the variant without the offset's code in its fast path for an offset of 1.0,
// the other one otherwise (pam_rowops.h).
#include "../../include/pam_hip.h"
#include "pam_rowops.h"

extern "C" {

size_t pam_hip_rowop_workspace_bytes(void) { return (size_t)pamrows::kMaxPartials * sizeof(float); }

int pam_hip_softmax_fwd(const float* x, float* y, float* row_sum, float* shift, long rows, long n, float offset, void* workspace, size_t workspace_bytes, void* stream)
{
    return offset != 1.0f ? PAM_ROW_OFFSET(softmax_fwd)(x, y, row_sum, shift, rows, n, offset, workspace, workspace_bytes, stream)
                          : PAM_ROW_PLAIN(softmax_fwd)(x, y, row_sum, shift, rows, n, offset, workspace, workspace_bytes, stream);
}

int pam_hip_softmax_bwd(const float* x, const float* dy, const float* row_sum, const float* shift, float* dx, long rows, long n, float offset, int approx_a, int approx_b, int approx_exp, void* stream)
{
    return offset != 1.0f ? PAM_ROW_OFFSET(softmax_bwd)(x, dy, row_sum, shift, dx, rows, n, offset, approx_a, approx_b, approx_exp, stream)
                          : PAM_ROW_PLAIN(softmax_bwd)(x, dy, row_sum, shift, dx, rows, n, offset, approx_a, approx_b, approx_exp, stream);
}

int pam_hip_logsumexp_fwd(const float* x, float* lse, float* log_softmax, float* shift, long rows, long n, float offset, void* workspace, size_t workspace_bytes, void* stream)
{
    return offset != 1.0f ? PAM_ROW_OFFSET(logsumexp_fwd)(x, lse, log_softmax, shift, rows, n, offset, workspace, workspace_bytes, stream)
                          : PAM_ROW_PLAIN(logsumexp_fwd)(x, lse, log_softmax, shift, rows, n, offset, workspace, workspace_bytes, stream);
}

int pam_hip_row_mean_fwd(const float* x, float* y, long rows, long n, float offset, void* stream)
{
    return offset != 1.0f ? PAM_ROW_OFFSET(row_mean_fwd)(x, y, rows, n, offset, stream)
                          : PAM_ROW_PLAIN(row_mean_fwd)(x, y, rows, n, offset, stream);
}

int pam_hip_layer_norm_fwd(const float* x, const float* weight, const float* bias, float* y, long rows, long n, float eps, float offset, void* stream)
{
    return offset != 1.0f ? PAM_ROW_OFFSET(layer_norm_fwd)(x, weight, bias, y, rows, n, eps, offset, stream)
                          : PAM_ROW_PLAIN(layer_norm_fwd)(x, weight, bias, y, rows, n, eps, offset, stream);
}

int pam_hip_logsumexp_bwd(const float* x, const float* grad, const float* shift, float* dx, long rows, long n, int log_softmax, float offset, int approx_a, int approx_b, int approx_exp, void* stream)
{
    return offset != 1.0f ? PAM_ROW_OFFSET(logsumexp_bwd)(x, grad, shift, dx, rows, n, log_softmax, offset, approx_a, approx_b, approx_exp, stream)
                          : PAM_ROW_PLAIN(logsumexp_bwd)(x, grad, shift, dx, rows, n, log_softmax, offset, approx_a, approx_b, approx_exp, stream);
}

int pam_hip_layer_norm_bwd(const float* x, const float* weight, const float* dy, float* dx, float* dw_terms, long rows, long n, float eps, float offset, int approx_a, int approx_b, int approx_exp, void* stream)
{
    return offset != 1.0f ? PAM_ROW_OFFSET(layer_norm_bwd)(x, weight, dy, dx, dw_terms, rows, n, eps, offset, approx_a, approx_b, approx_exp, stream)
                          : PAM_ROW_PLAIN(layer_norm_bwd)(x, weight, dy, dx, dw_terms, rows, n, eps, offset, approx_a, approx_b, approx_exp, stream);
}

}  // extern "C"
