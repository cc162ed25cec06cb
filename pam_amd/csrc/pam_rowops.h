// The row-wise kernels exist in two variants, compiled from pam_rowops_kernels.h: `plain`, whose kernels' unchecked first
// attempt carries no code for an offset where that measured faster (a call with an offset would have every row redone by
// the checked functions), and `offset`, where it always does.  The entry points (pam_rowops.hip) call `plain` for an offset
// of 1.0 and `offset` otherwise; both give the same bits for any arguments.
#ifndef PAM_ROWOPS_H
#define PAM_ROWOPS_H
#include <stddef.h>

namespace pamrows {
constexpr int kMaxPartials = 1024;          // per-block maxima of the scaled input that a launch leaves in the workspace
}

#define PAM_ROW_DECLARE(FN) \
    int FN(softmax_fwd)(const float* x, float* y, float* row_sum, float* shift, long rows, long n, float offset, void* workspace, size_t workspace_bytes, void* stream); \
    int FN(softmax_bwd)(const float* x, const float* dy, const float* row_sum, const float* shift, float* dx, long rows, long n, float offset, int approx_a, int approx_b, int approx_exp, void* stream); \
    int FN(logsumexp_fwd)(const float* x, float* lse, float* log_softmax, float* shift, long rows, long n, float offset, void* workspace, size_t workspace_bytes, void* stream); \
    int FN(row_mean_fwd)(const float* x, float* y, long rows, long n, float offset, void* stream); \
    int FN(layer_norm_fwd)(const float* x, const float* weight, const float* bias, float* y, long rows, long n, float eps, float offset, void* stream); \
    int FN(logsumexp_bwd)(const float* x, const float* grad, const float* shift, float* dx, long rows, long n, int log_softmax, float offset, int approx_a, int approx_b, int approx_exp, void* stream); \
    int FN(layer_norm_bwd)(const float* x, const float* weight, const float* dy, float* dx, float* dw_terms, long rows, long n, float eps, float offset, int approx_a, int approx_b, int approx_exp, void* stream);

#define PAM_ROW_PLAIN(name) pam_row_plain_##name
#define PAM_ROW_OFFSET(name) pam_row_offset_##name
PAM_ROW_DECLARE(PAM_ROW_PLAIN)
PAM_ROW_DECLARE(PAM_ROW_OFFSET)
#endif  // PAM_ROWOPS_H
