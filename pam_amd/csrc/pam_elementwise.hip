// Elementwise piecewise-affine kernels for gfx950: HBM-bound streams.
//
// One kernel template serves every op: each lane moves 128-bit vectors, a work-group
// covers kUnroll * 256 consecutive vectors per step (so every wavefront touches whole
// 1 KiB runs) and strides over the array by the grid size.  All loads of a step are
// issued before the arithmetic so several are in flight per lane.
// Algorithmic traffic: 12 B/element for the two-input forwards, 16 B/element for their
// exact backwards, 8 B/element for pa_exp/pa_log and the scalar-operand forwards,
// 12 B/element for the pa_exp/pa_log backwards.
#include <math.h>

#include "pam_common.h"
#include "pam_device.h"

using namespace pamdev;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kUnroll = 4;

struct OpPam {      // C = A (*) B                      (pam/cuda_kernels.cu:151)
    float off; bool has_off;
    __device__ float operator()(float a, float b, float) const { return pam_mul_off(a, b, off, has_off); }
};
struct OpPad {      // C = A (/) B                      (pam/cuda_kernels.cu:247)
    float off; bool has_off;
    __device__ float operator()(float a, float b, float) const { return pad_div_off(a, b, off, has_off); }
};
struct OpPamBwd {   // dA                               (pam/cuda_kernels.cu:196)
    float off; bool has_off;
    __device__ float operator()(float a, float b, float d) const { return pam_mul_bwd(a, b, d, off, has_off); }
};
struct OpPadBwd {   // dB                               (pam/cuda_kernels.cu:292)
    float off; bool has_off;
    __device__ float operator()(float a, float b, float d) const { return pad_div_bwd(a, b, d, off, has_off); }
};
struct OpPamBcastA { const float* s; float off; bool has_off;
    __device__ float operator()(float x, float, float) const { return pam_mul_off(*s, x, off, has_off); } };
struct OpPamBcastB { const float* s; float off; bool has_off;
    __device__ float operator()(float x, float, float) const { return pam_mul_off(x, *s, off, has_off); } };
struct OpPadBcastA { const float* s; float off; bool has_off;
    __device__ float operator()(float x, float, float) const { return pad_div_off(*s, x, off, has_off); } };
struct OpPadBcastB { const float* s; float off; bool has_off;
    __device__ float operator()(float x, float, float) const { return pad_div_off(x, *s, off, has_off); } };
struct OpExp {      // Y = pa_exp2(X (*) log2 base)     (pam/cuda_kernels.cu:344)
    float l2b, off; bool has_off;
    __device__ float operator()(float x, float, float) const { return pa_exp2(pam_mul_off(x, l2b, off, has_off)); }
};
struct OpLog {      // Y = pa_log2(X) (/) log2 base     (pam/cuda_kernels.cu:439)
    float l2b, off; bool has_off;
    __device__ float operator()(float x, float, float) const { return pad_div_off(pa_log2(x), l2b, off, has_off); }
};
struct OpExpBwd {   // (pam/cuda_kernels.cu:386-391)
    float l2b, off; bool has_off;
    __device__ float operator()(float x, float dy, float) const {
        return pam_mul_bwd(x, l2b, pa_exp2_bwd(pam_mul_off(x, l2b, off, has_off), dy), off, has_off);
    }
};
struct OpLogBwd {   // (pam/cuda_kernels.cu:481-484); the inner pam_bwd runs without offset
    float l2b, off; bool has_off;
    __device__ float operator()(float x, float dy, float) const {
        float inv = pad_div_off(1.0f, l2b, off, has_off);
        return pa_log2_bwd(x, pam_mul_bwd(pa_log2_signed(x), inv, dy, 1.0f, false));
    }
};

// A ** p for a scalar exponent as the op library composes it: exp2(log2(A) (*) p), zero where A is
// zero (pam/pam_ops.py:70-79), and the gradient for A that autograd chains from the three ops'
// backward formulas (pam/cuda_bindings.py:43-57, 224-239, 262-276): through the select, exp2, the
// product's first operand, log2.  ln 2 is math.log(2.0) rounded to fp32, as torch.full_like stores it.
constexpr float kLn2 = (float)0.6931471805599453;
struct OpPow {
    float p, off; bool has_off;
    __device__ float operator()(float a, float, float) const
    {
        if (a == 0.0f) return 0.0f;
        return exp2_entry(pam_mul_off(log2_entry(a, off, has_off), p, off, has_off), off, has_off);
    }
    // branch-free form, exact whenever every value it touches is a normal number and a > 0 (else redone checked)
    __device__ bool has_fast() const { return true; }
    __device__ float fast(float a, float, float, Span& sp) const
    {
        sp.in_exp_range = sp.in_exp_range && a > 0.0f;
        return exp2_entry_unchecked(pam_unchecked_off(log2_entry_unchecked(a, off, has_off, sp), p, off, has_off, sp), off, has_off, sp);
    }
};
struct OpPowBwd {
    float p, off; bool has_off, approx_a, approx_e;
    __device__ float operator()(float a, float g, float) const
    {
        const float l = log2_entry(a, off, has_off);
        const float t = pam_mul_off(l, p, off, has_off);
        const float gy = a == 0.0f ? 0.0f : g;
        const float gt = approx_e ? pam_mul_off(pam_mul_off(exp2_entry(t, off, has_off), kLn2, off, has_off), gy, off, has_off)
                                  : exp2_entry_bwd(t, gy, off, has_off);
        const float gl = approx_a ? pam_mul_off(gt, p, off, has_off) : pam_mul_bwd(l, p, gt, off, has_off);
        return approx_e ? pad_div_off(pad_div_off(gl, a, off, has_off), kLn2, off, has_off) : log2_entry_bwd(a, gl, off, has_off);
    }
    __device__ bool has_fast() const { return approx_a && approx_e; }       // the all-approximate chain
    __device__ float fast(float a, float g, float, Span& sp) const
    {
        sp.in_exp_range = sp.in_exp_range && a > 0.0f;
        const float l = log2_entry_unchecked(a, off, has_off, sp);
        const float t = pam_unchecked_off(l, p, off, has_off, sp);
        const float y = exp2_entry_unchecked(t, off, has_off, sp);
        const float gt = pam_unchecked_off(pam_unchecked_off(y, kLn2, off, has_off, sp), g, off, has_off, sp);
        const float gl = pam_unchecked_off(gt, p, off, has_off, sp);
        return pad_unchecked_off(pad_unchecked_off(gl, a, off, has_off, sp), kLn2, off, has_off, sp);
    }
};

// ops that also have a branch-free form `fast(a, b, c, Span&)`
template <class Op, class = void> struct HasFast { static constexpr bool value = false; };
template <class Op> struct HasFast<Op, decltype((void)&Op::has_fast)> { static constexpr bool value = true; };

template <class Op, int NIN>
__global__ __launch_bounds__(kThreads) void ew_vec_kernel(const v4f* __restrict__ p0, const v4f* __restrict__ p1,
                                                         const v4f* __restrict__ p2, v4f* __restrict__ out,
                                                         size_t nvec, Op op)
{
    const size_t step = (size_t)gridDim.x * (kThreads * kUnroll);
    for (size_t base = (size_t)blockIdx.x * (kThreads * kUnroll) + threadIdx.x; base < nvec; base += step) {
        v4f a[kUnroll], b[kUnroll], c[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            size_t i = base + (size_t)u * kThreads;
            if (i < nvec) {
                a[u] = __builtin_nontemporal_load(p0 + i);
                if (NIN > 1) b[u] = __builtin_nontemporal_load(p1 + i);
                if (NIN > 2) c[u] = __builtin_nontemporal_load(p2 + i);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            size_t i = base + (size_t)u * kThreads;
            if (i < nvec) {
                v4f r = {};
                bool done = false;
                if constexpr (HasFast<Op>::value) {
                    if (op.has_fast()) {
                        Span sp;
                        r.x = op.fast(a[u].x, NIN > 1 ? b[u].x : 0.f, NIN > 2 ? c[u].x : 0.f, sp);
                        r.y = op.fast(a[u].y, NIN > 1 ? b[u].y : 0.f, NIN > 2 ? c[u].y : 0.f, sp);
                        r.z = op.fast(a[u].z, NIN > 1 ? b[u].z : 0.f, NIN > 2 ? c[u].z : 0.f, sp);
                        r.w = op.fast(a[u].w, NIN > 1 ? b[u].w : 0.f, NIN > 2 ? c[u].w : 0.f, sp);
                        done = sp.normal();
                    }
                }
                if (!done) {
                    r.x = op(a[u].x, NIN > 1 ? b[u].x : 0.f, NIN > 2 ? c[u].x : 0.f);
                    r.y = op(a[u].y, NIN > 1 ? b[u].y : 0.f, NIN > 2 ? c[u].y : 0.f);
                    r.z = op(a[u].z, NIN > 1 ? b[u].z : 0.f, NIN > 2 ? c[u].z : 0.f);
                    r.w = op(a[u].w, NIN > 1 ? b[u].w : 0.f, NIN > 2 ? c[u].w : 0.f);
                }
                __builtin_nontemporal_store(r, out + i);
            }
        }
    }
}

// Unaligned pointers and the last n % 4 elements.
template <class Op, int NIN>
__global__ __launch_bounds__(kThreads) void ew_scalar_kernel(const float* __restrict__ p0, const float* __restrict__ p1,
                                                            const float* __restrict__ p2, float* __restrict__ out,
                                                            size_t first, size_t n, Op op)
{
    const size_t step = (size_t)gridDim.x * kThreads;
    for (size_t i = first + (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += step)
        out[i] = op(p0[i], NIN > 1 ? p1[i] : 0.f, NIN > 2 ? p2[i] : 0.f);
}

template <class Op, int NIN>
int launch(const char* what, const float* p0, const float* p1, const float* p2, float* out, size_t n, Op op, void* stream)
{
    if (n == 0) return PAM_HIP_OK;
    if (!p0 || !out || (NIN > 1 && !p1) || (NIN > 2 && !p2)) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: null pointer", what);
    hipStream_t st = (hipStream_t)stream;
    uintptr_t align = (uintptr_t)p0 | (uintptr_t)out | (NIN > 1 ? (uintptr_t)p1 : 0) | (NIN > 2 ? (uintptr_t)p2 : 0);
    size_t nvec = (align & 15u) ? 0 : n / 4;
    const size_t cap = (size_t)1 << 30;      // one pass per lane for any realistic size; grid-stride beyond
    if (nvec) {
        size_t blocks = (nvec + kThreads * kUnroll - 1) / (kThreads * kUnroll);
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((ew_vec_kernel<Op, NIN>), dim3((unsigned)blocks), dim3(kThreads), 0, st,
                           (const v4f*)p0, (const v4f*)p1, (const v4f*)p2, (v4f*)out, nvec, op);
    }
    if (nvec * 4 < n) {
        size_t rest = n - nvec * 4;
        size_t blocks = (rest + kThreads - 1) / kThreads;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((ew_scalar_kernel<Op, NIN>), dim3((unsigned)blocks), dim3(kThreads), 0, st,
                           p0, p1, p2, out, nvec * 4, n, op);
    }
    return pamhost::check_launch(what);
}

// ---------------------------------------------------------------- both gradients of a product / quotient in one pass
// autograd asks for dA and dB of C = A (*) B or A (/) B together; the reference computes them with two
// to six launches (pam/cuda_bindings.py:43-57, 78-97).  Same formulas per element, one read of A, B, dC.
struct PairPam {
    float off; bool has_off, approx_a, approx_b;
    __device__ void operator()(float a, float b, float d, float& da, float& db) const
    {
        da = approx_a ? pam_mul_off(d, b, off, has_off) : pam_mul_bwd(a, b, d, off, has_off);
        db = approx_b ? pam_mul_off(d, a, off, has_off) : pam_mul_bwd(b, a, d, off, has_off);
    }
};
struct PairPad {
    float off; bool has_off, approx_a, approx_b;
    __device__ void operator()(float a, float b, float d, float& da, float& db) const
    {
        const float inv = pad_div_off(1.0f, b, off, has_off);
        da = approx_a ? pam_mul_off(inv, d, off, has_off) : pam_mul_bwd(a, inv, d, 1.0f, false);
        db = approx_b ? -pam_mul_off(pad_div_off(pad_div_off(a, b, off, has_off), b, off, has_off), d, off, has_off)
                      : pad_div_bwd(a, b, d, off, has_off);
    }
};

template <class Op>
__global__ __launch_bounds__(kThreads) void pair_vec_kernel(const v4f* __restrict__ pa, const v4f* __restrict__ pb, const v4f* __restrict__ pd,
                                                           v4f* __restrict__ oa, v4f* __restrict__ ob, size_t nvec, Op op)
{
    constexpr int U = 2;
    const size_t step = (size_t)gridDim.x * (kThreads * U);
    for (size_t base = (size_t)blockIdx.x * (kThreads * U) + threadIdx.x; base < nvec; base += step) {
        v4f a[U], b[U], d[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            size_t i = base + (size_t)u * kThreads;
            if (i < nvec) { a[u] = __builtin_nontemporal_load(pa + i); b[u] = __builtin_nontemporal_load(pb + i); d[u] = __builtin_nontemporal_load(pd + i); }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            size_t i = base + (size_t)u * kThreads;
            if (i < nvec) {
                v4f ra, rb; float x, y;
                op(a[u].x, b[u].x, d[u].x, x, y); ra.x = x; rb.x = y;
                op(a[u].y, b[u].y, d[u].y, x, y); ra.y = x; rb.y = y;
                op(a[u].z, b[u].z, d[u].z, x, y); ra.z = x; rb.z = y;
                op(a[u].w, b[u].w, d[u].w, x, y); ra.w = x; rb.w = y;
                __builtin_nontemporal_store(ra, oa + i); __builtin_nontemporal_store(rb, ob + i);
            }
        }
    }
}

template <class Op>
__global__ __launch_bounds__(kThreads) void pair_scalar_kernel(const float* __restrict__ pa, const float* __restrict__ pb, const float* __restrict__ pd,
                                                              float* __restrict__ oa, float* __restrict__ ob, size_t first, size_t n, Op op)
{
    const size_t step = (size_t)gridDim.x * kThreads;
    for (size_t i = first + (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += step) {
        float x, y;
        op(pa[i], pb[i], pd[i], x, y);
        oa[i] = x; ob[i] = y;
    }
}

template <class Op>
int launch_pair(const char* what, const float* a, const float* b, const float* d, float* da, float* db, size_t n, Op op, void* stream)
{
    if (n == 0) return PAM_HIP_OK;
    if (!a || !b || !d || !da || !db) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: null pointer", what);
    hipStream_t st = (hipStream_t)stream;
    uintptr_t align = (uintptr_t)a | (uintptr_t)b | (uintptr_t)d | (uintptr_t)da | (uintptr_t)db;
    size_t nvec = (align & 15u) ? 0 : n / 4;
    const size_t cap = (size_t)1 << 30;
    if (nvec) {
        size_t blocks = (nvec + kThreads * 2 - 1) / (kThreads * 2);
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(pair_vec_kernel<Op>, dim3((unsigned)blocks), dim3(kThreads), 0, st,
                           (const v4f*)a, (const v4f*)b, (const v4f*)d, (v4f*)da, (v4f*)db, nvec, op);
    }
    if (nvec * 4 < n) {
        size_t blocks = (n - nvec * 4 + kThreads - 1) / kThreads;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(pair_scalar_kernel<Op>, dim3((unsigned)blocks), dim3(kThreads), 0, st, a, b, d, da, db, nvec * 4, n, op);
    }
    return pamhost::check_launch(what);
}

// ---------------------------------------------------------------- Adam step
// One update of a parameter tensor by the Adam variant whose products, quotient and square
// root are PAM ops (the training recipe's optimizer, fairseq/optim/adam.py:226-252 in the
// reference tree): eleven elementwise launches there, one here.  Reads p, g, m, v and
// writes p, m, v: 28 B/element.
struct AdamArgs {
    float beta1, one_minus_beta1, beta2, one_minus_beta2, eps, decay, step_size, off;
    bool has_decay, has_off;
};

// the update with every operand and result in the normal range: no branches; `sp` records whether that held
__device__ __forceinline__ void adam_one_unchecked(float& p, float g, float& m, float& v, const AdamArgs& a, Span& sp)
{
    const float off = a.off; const bool ho = a.has_off;
    m = pam_unchecked_off(m, a.beta1, off, ho, sp) + pam_unchecked_off(g, a.one_minus_beta1, off, ho, sp);
    v = pam_unchecked_off(v, a.beta2, off, ho, sp);
    v = v + pam_unchecked_off(pam_unchecked_off(g, g, off, ho, sp), a.one_minus_beta2, off, ho, sp);
    const float denom = pow_half_unchecked(v, off, ho, sp) + a.eps;
    if (a.has_decay) p = p - pam_unchecked_off(p, a.decay, off, ho, sp);
    p = p - pam_unchecked_off(pad_unchecked_off(m, denom, off, ho, sp), a.step_size, off, ho, sp);
}

__device__ __forceinline__ void adam_one(float& p, float g, float& m, float& v, const AdamArgs& a)
{
    const float off = a.off; const bool ho = a.has_off;
    m = pam_mul_off(m, a.beta1, off, ho) + pam_mul_off(g, a.one_minus_beta1, off, ho);
    v = pam_mul_off(v, a.beta2, off, ho);
    v = v + pam_mul_off(pam_mul_off(g, g, off, ho), a.one_minus_beta2, off, ho);
    const float denom = pow_half(v, off, ho) + a.eps;
    if (a.has_decay) p = p - pam_mul_off(p, a.decay, off, ho);
    p = p - pam_mul_off(pad_div_off(m, denom, off, ho), a.step_size, off, ho);
}

// kAdamVectors 128-bit vectors per lane and stream, all loads issued before the arithmetic, everything read and
// written past the caches (each value is touched once per step): 345 -> 315 us for 2^26 parameters against one vector
// per lane with cached loads.
__device__ __forceinline__ void adam_vector(v4f& pp, const v4f& gg, v4f& mm, v4f& vv, const AdamArgs& a)
{
    v4f p1 = pp, m1 = mm, v1 = vv;
    Span sp;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float pc = pp[c], mc = mm[c], vc = vv[c];
        adam_one_unchecked(pc, gg[c], mc, vc, a, sp);
        p1[c] = pc; m1[c] = mc; v1[c] = vc;
    }
    if (!sp.normal()) {                     // a zero, subnormal, inf, NaN or out-of-range value somewhere: redo checked
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float pc = pp[c], mc = mm[c], vc = vv[c];
            adam_one(pc, gg[c], mc, vc, a);
            p1[c] = pc; m1[c] = mc; v1[c] = vc;
        }
    }
    pp = p1; mm = m1; vv = v1;
}

constexpr int kAdamVectors = 2;               // 128-bit vectors per lane and stream (four measured the same)
__global__ __launch_bounds__(kThreads) void adam_vec_kernel(v4f* __restrict__ p, const v4f* __restrict__ g,
                                                           v4f* __restrict__ m, v4f* __restrict__ v, size_t nvec, AdamArgs a)
{
    // work-group b takes kAdamVectors x kThreads consecutive vectors: lane t the vectors t, t + kThreads, ... of them
    const size_t first = (size_t)blockIdx.x * (kAdamVectors * kThreads) + threadIdx.x;
    if (first + (kAdamVectors - 1) * kThreads < nvec) {
        v4f pp[kAdamVectors], gg[kAdamVectors], mm[kAdamVectors], vv[kAdamVectors];
#pragma unroll
        for (int u = 0; u < kAdamVectors; ++u) {
            const size_t i = first + (size_t)u * kThreads;
            pp[u] = __builtin_nontemporal_load(p + i); gg[u] = __builtin_nontemporal_load(g + i);
            mm[u] = __builtin_nontemporal_load(m + i); vv[u] = __builtin_nontemporal_load(v + i);
        }
#pragma unroll
        for (int u = 0; u < kAdamVectors; ++u) {
            const size_t i = first + (size_t)u * kThreads;
            adam_vector(pp[u], gg[u], mm[u], vv[u], a);
            __builtin_nontemporal_store(pp[u], p + i); __builtin_nontemporal_store(mm[u], m + i); __builtin_nontemporal_store(vv[u], v + i);
        }
    } else {
        for (size_t i = first; i < nvec; i += kThreads) {
            v4f p0 = p[i], g0 = g[i], m0 = m[i], v0 = v[i];
            adam_vector(p0, g0, m0, v0, a);
            p[i] = p0; m[i] = m0; v[i] = v0;
        }
    }
}

__global__ __launch_bounds__(kThreads) void adam_scalar_kernel(float* __restrict__ p, const float* __restrict__ g,
                                                              float* __restrict__ m, float* __restrict__ v,
                                                              size_t first, size_t n, AdamArgs a)
{
    const size_t step = (size_t)gridDim.x * kThreads;
    for (size_t i = first + (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += step) {
        float pp = p[i], mm = m[i], vv = v[i];
        adam_one(pp, g[i], mm, vv, a);
        p[i] = pp; m[i] = mm; v[i] = vv;
    }
}

}  // namespace

extern "C" {

int pam_hip_abi_version(void) { return PAM_HIP_ABI_VERSION; }
const char* pam_hip_last_error(void) { return pamhost::error_buffer(); }

int pam_hip_device_info(int* compute_units, int* clock_khz)
{
    int dev = 0; hipDeviceProp_t prop;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return pamhost::fail(PAM_HIP_ERR_LAUNCH, "device query: %s", hipGetErrorString(e));
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    return PAM_HIP_OK;
}

int pam_hip_pam_fwd(const float* a, const float* b, float* c, size_t n, float offset, void* stream)
{ return launch<OpPam, 2>("pam_fwd", a, b, nullptr, c, n, OpPam{offset, offset != 1.0f}, stream); }

int pam_hip_pad_fwd(const float* a, const float* b, float* c, size_t n, float offset, void* stream)
{ return launch<OpPad, 2>("pad_fwd", a, b, nullptr, c, n, OpPad{offset, offset != 1.0f}, stream); }

int pam_hip_pam_bwd(const float* a, const float* b, const float* dc, float* da, size_t n, float offset, void* stream)
{ return launch<OpPamBwd, 3>("pam_bwd", a, b, dc, da, n, OpPamBwd{offset, offset != 1.0f}, stream); }

int pam_hip_pad_bwd(const float* a, const float* b, const float* dc, float* db, size_t n, float offset, void* stream)
{ return launch<OpPadBwd, 3>("pad_bwd", a, b, dc, db, n, OpPadBwd{offset, offset != 1.0f}, stream); }

int pam_hip_pam_bwd_pair(const float* a, const float* b, const float* dc, float* da, float* db, size_t n, float offset,
                         int approx_a, int approx_b, void* stream)
{ return launch_pair("pam_bwd_pair", a, b, dc, da, db, n, PairPam{offset, offset != 1.0f, approx_a != 0, approx_b != 0}, stream); }

int pam_hip_pad_bwd_pair(const float* a, const float* b, const float* dc, float* da, float* db, size_t n, float offset,
                         int approx_a, int approx_b, void* stream)
{ return launch_pair("pad_bwd_pair", a, b, dc, da, db, n, PairPad{offset, offset != 1.0f, approx_a != 0, approx_b != 0}, stream); }

int pam_hip_pam_fwd_bcast(const float* x, const float* s, int scalar_is_a, float* c, size_t n, float offset, void* stream)
{
    if (!s) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "pam_fwd_bcast: null pointer");
    bool ho = offset != 1.0f;
    return scalar_is_a ? launch<OpPamBcastA, 1>("pam_fwd_bcast", x, nullptr, nullptr, c, n, OpPamBcastA{s, offset, ho}, stream)
                       : launch<OpPamBcastB, 1>("pam_fwd_bcast", x, nullptr, nullptr, c, n, OpPamBcastB{s, offset, ho}, stream);
}

int pam_hip_pad_fwd_bcast(const float* x, const float* s, int scalar_is_a, float* c, size_t n, float offset, void* stream)
{
    if (!s) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "pad_fwd_bcast: null pointer");
    bool ho = offset != 1.0f;
    return scalar_is_a ? launch<OpPadBcastA, 1>("pad_fwd_bcast", x, nullptr, nullptr, c, n, OpPadBcastA{s, offset, ho}, stream)
                       : launch<OpPadBcastB, 1>("pad_fwd_bcast", x, nullptr, nullptr, c, n, OpPadBcastB{s, offset, ho}, stream);
}

// log2 of the base is taken once on the host, as the reference's CPU path does with
// torch.log2(torch.tensor(base)) (pam/native.py:203, 211-212); the reference's GPU kernel evaluates log2(base) on
// the device per element (pam/cuda_kernels.cu:343, 385, 438, 481), and no fixture of the reference pins that
// value.  Here it is the double-precision logarithm rounded once to fp32, so that the constant does not depend on
// the accuracy of a libm's single-precision routine: 0x3fb8aa3b for e, 0x40549a78 for 10, exactly -1 for 0.5.
float pam_hip_log2_base(float base) { return (float)log2((double)base); }

int pam_hip_pa_exp_fwd(const float* x, float* y, size_t n, float base, float offset, void* stream)
{ return launch<OpExp, 1>("pa_exp_fwd", x, nullptr, nullptr, y, n, OpExp{pam_hip_log2_base(base), offset, offset != 1.0f}, stream); }

int pam_hip_pa_log_fwd(const float* x, float* y, size_t n, float base, float offset, void* stream)
{ return launch<OpLog, 1>("pa_log_fwd", x, nullptr, nullptr, y, n, OpLog{pam_hip_log2_base(base), offset, offset != 1.0f}, stream); }

int pam_hip_pa_exp_bwd(const float* x, const float* dy, float* dx, size_t n, float base, float offset, void* stream)
{ return launch<OpExpBwd, 2>("pa_exp_bwd", x, dy, nullptr, dx, n, OpExpBwd{pam_hip_log2_base(base), offset, offset != 1.0f}, stream); }

int pam_hip_pa_log_bwd(const float* x, const float* dy, float* dx, size_t n, float base, float offset, void* stream)
{ return launch<OpLogBwd, 2>("pa_log_bwd", x, dy, nullptr, dx, n, OpLogBwd{pam_hip_log2_base(base), offset, offset != 1.0f}, stream); }

int pam_hip_pow_fwd(const float* x, float* y, size_t n, float exponent, float offset, void* stream)
{ return launch<OpPow, 1>("pow_fwd", x, nullptr, nullptr, y, n, OpPow{exponent, offset, offset != 1.0f}, stream); }

int pam_hip_pow_bwd(const float* x, const float* dy, float* dx, size_t n, float exponent, float offset,
                    int approx_a, int approx_exp, void* stream)
{
    return launch<OpPowBwd, 2>("pow_bwd", x, dy, nullptr, dx, n,
                               OpPowBwd{exponent, offset, offset != 1.0f, approx_a != 0, approx_exp != 0}, stream);
}

int pam_hip_adam_step(float* p, const float* g, float* m, float* v, size_t n, float beta1, float one_minus_beta1,
                      float beta2, float one_minus_beta2, float eps, float decay, int has_decay, float step_size,
                      float offset, void* stream)
{
    if (n == 0) return PAM_HIP_OK;
    if (!p || !g || !m || !v) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "adam_step: null pointer");
    AdamArgs a{beta1, one_minus_beta1, beta2, one_minus_beta2, eps, decay, step_size, offset, has_decay != 0, offset != 1.0f};
    hipStream_t st = (hipStream_t)stream;
    uintptr_t align = (uintptr_t)p | (uintptr_t)g | (uintptr_t)m | (uintptr_t)v;
    size_t nvec = (align & 15u) ? 0 : n / 4;
    const size_t cap = (size_t)1 << 30;
    if (nvec) {
        const size_t blocks = (nvec + kAdamVectors * kThreads - 1) / (kAdamVectors * kThreads);
        if (blocks > cap) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "adam_step: more than 2^41 parameters");
        hipLaunchKernelGGL(adam_vec_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, st, (v4f*)p, (const v4f*)g, (v4f*)m,
                           (v4f*)v, nvec, a);
    }
    if (nvec * 4 < n) {
        size_t blocks = (n - nvec * 4 + kThreads - 1) / kThreads;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(adam_scalar_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, st, p, g, m, v, nvec * 4, n, a);
    }
    return pamhost::check_launch("adam_step");
}

}  // extern "C"
