/*
 * pam_hip_probe.h -- measurement aids of libpam_hip.so, kept apart from the drop-in interface of pam_hip.h.
 * None of them has a counterpart in the reference.  They are what bench.py uses to state the vector issue
 * rate that its roofline fractions are measured against, and to try other plans of the matrix kernel.
 */
#ifndef PAM_HIP_PROBE_H
#define PAM_HIP_PROBE_H

#ifdef __cplusplus
extern "C" {
#endif

/* Runs the matrix kernel's instruction mix (one v_add_u32
 * and one dependent v_add_f32 per product) on register operands only, blocks work-groups of 256 lanes, each lane
 * iters * 256 VALU lane-operations; timing it gives the vector issue rate the roofline figures are stated against.
 * seed: 1024 words, out: blocks * 256 floats. */
int pam_hip_issue_probe(const void *seed, float *out, int blocks, int iters, void *stream);
/* The same with every step's operands read from LDS as the matrix kernel's inner loop reads them, for a
 * tm x tn micro-tile (4x4, 8x4, 8x8); each lane iters * 32 * tm * tn pairs. */
int pam_hip_issue_probe_lds(const void *seed, float *out, int blocks, int iters, int tm, int tn, void *stream);

/* Tuning hook for experiments: forces the k-tile depth (16 or 32; 0 = automatic) and the number of pieces every
 * output tile's k range is cut into (0 = automatic; 1 = whole tiles) of the matrix products for the calling thread;
 * pam_hip_gemm_plan and pam_hip_gemm_workspace_bytes follow the forced values. */
void pam_hip_set_tuning(int k_tile, int pieces);

#ifdef __cplusplus
}
#endif
#endif /* PAM_HIP_PROBE_H */
