/*
 * pam_oracle.c -- CPU restatement of the piecewise-affine arithmetic of epfml/pam.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls
 * this file; it exists so that the HIP kernels can be checked against an
 * independently written implementation of the same arithmetic, and so that the
 * benchmark can time a CPU baseline next to the GPU figure.
 *
 * Two flavours of every product/quotient are provided:
 *
 *   exact   the integer definition  bits(a) + bits(b) - BIAS   (reference
 *           pam/cuda_kernels.cu:17-19, 62-64) extended to every fp32 input with
 *           the edge classes of the reference's float emulation pam/native.py
 *           (zero, subnormal, inf, NaN, overflow, gradual underflow; read off
 *           pam/native.py:16-20, 38-39, 54-55, 163-164).  This is what the GPU
 *           kernels compute.
 *
 *   chain   a model of pam/native.py's float chain itself
 *           (log = fl(e + m), s = fl(la + lb), u = fl(fl(1 + s) - floor s),
 *            out = fl(2^floor(s) * u); pam/native.py:29-30, 38-39, 54-55)
 *           with the exponent e taken exactly.  It differs from native.py only
 *           where torch's floor(log2(x)) misreports e (just below powers of two).
 *           It is used to explain, element by element, where the float emulation
 *           departs from the integer definition.
 *
 * Parity pinning (see tests/test_oracle_*.py):
 *   pam/pad exact, normal range ...... closed form, reference vectors
 *                                      pam/test_pam.py:13-29, invariants, brute force
 *   edge classes ..................... golden vectors written from pam/native.py
 *   pam_bwd .......................... closed form pam/cuda_kernels.cu:48-57 and
 *                                      native goldens (pam/native.py:65-77)
 *   pa_log2 / pa_exp2 / pa_exp / pa_log  native goldens
 *   chain flavour .................... native goldens (bit-for-bit outside the
 *                                      log2f glitch band)
 *   pad_bwd, pa_exp_bwd, pa_log_bwd .. closed forms of pam/cuda_kernels.cu:85-136,
 *                                      375-393,470-486 (the reference has no CPU
 *                                      implementation, test or vector of them), pinned
 *                                      as the slope of the pinned forward functions by
 *                                      finite differences inside one affine piece
 *                                      (pad_bwd up to the reference's sign convention
 *                                      for negative divisors, which the test states).
 *   row-wise compositions ............ equal, bit for bit, to the same chain built from
 *                                      the pinned primitives above whenever the row sums
 *                                      are exact (short-mantissa rows), and to it within
 *                                      summation-order noise otherwise; the softmax
 *                                      gradient likewise against the primitives' backward
 *                                      formulas chained by hand (tests/test_rowops.py)
 *   GEMM ............................. power-of-two operands == fp32 matmul
 *                                      (pam/test_pam.py:151-216 construction), the
 *                                      reference's deterministic 5x4 / 4x3 operands
 *                                      (pam/test_pam.py:96-97,129-130), brute force.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define BIAS_BITS 0x3f800000u
#define MANT_MASK 0x007fffffu
#define EXPO_MASK 0x7f800000u
#define ONE_M (1u << 23)

static inline uint32_t f2u(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float u2f(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

enum { CLS_ZERO = 0, CLS_FIN = 1, CLS_INF = 2, CLS_NAN = 3 };

/* |x| = 2^e * (1 + m / 2^23) for finite non-zero x, subnormals normalised.
 * Mirrors get_exp_mantissa (pam/native.py:12-20) with an exact exponent. */
typedef struct { int cls; int neg; int e; uint32_t m; } dec_t;

static dec_t decomp(float x)
{
    dec_t d; uint32_t u = f2u(x), mag = u & 0x7fffffffu;
    d.neg = (int)(u >> 31); d.e = 0; d.m = 0;
    if (mag > EXPO_MASK) { d.cls = CLS_NAN; return d; }
    if (mag == EXPO_MASK) { d.cls = CLS_INF; return d; }
    if (mag == 0) { d.cls = CLS_ZERO; return d; }
    d.cls = CLS_FIN;
    uint32_t ef = mag >> 23, mf = mag & MANT_MASK;
    if (ef) { d.e = (int)ef - 127; d.m = mf; }
    else {
        int p = 31 - __builtin_clz(mf);          /* leading one at bit p, value mf * 2^-149 */
        d.e = p - 149; d.m = (mf << (23 - p)) & MANT_MASK;
    }
    return d;
}

/* 2**k as torch evaluates it in fp32 for integer-valued k (probed: exact for
 * -149..127, 0 at and below -150, inf at and above 128). */
static float pow2i(int k)
{
    if (k >= 128) return INFINITY;
    if (k <= -150) return 0.0f;
    return ldexpf(1.0f, k);
}

/* sign * 2^E * (1 + M/2^23), rounded once to nearest-even into fp32, with the
 * range classes of pa_exp2_fwd (pam/native.py:38-39): E >= 128 -> inf,
 * E <= -150 -> 0 (2**E is already 0 before the multiply). */
static float compose(int neg, int E, uint32_t M)
{
    uint32_t s = neg ? 0x80000000u : 0u;
    if (E >= 128) return u2f(s | EXPO_MASK);
    if (E <= -150) return u2f(s);
    if (E >= -126) return u2f(s | ((uint32_t)(E + 127) << 23) | M);
    {
        uint32_t full = ONE_M | M;               /* 24 significant bits */
        int sh = -126 - E;                       /* 1..23 */
        uint32_t q = full >> sh, rem = full & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return u2f(s | q);                       /* q == 2^23 is the smallest normal */
    }
}

/* ------------------------------------------------------------------ exact */

/* pam_fwd without offset (pam/native.py:54-55; integer form pam/cuda_kernels.cu:17-19) */
static float pam1(float a, float b)
{
    dec_t A = decomp(a), B = decomp(b);
    if (A.cls >= CLS_INF || B.cls >= CLS_INF) return NAN;   /* x_m = (inf-inf)/inf */
    if (A.cls == CLS_ZERO || B.cls == CLS_ZERO) {
        /* torch.sign(+-0) = +0: the zero takes the sign of the non-zero operand only */
        int neg = (A.cls == CLS_ZERO ? 0 : A.neg) ^ (B.cls == CLS_ZERO ? 0 : B.neg);
        return u2f(neg ? 0x80000000u : 0u);
    }
    int E = A.e + B.e; uint32_t M = A.m + B.m;
    if (M >= ONE_M) { E++; M -= ONE_M; }
    return compose(A.neg ^ B.neg, E, M);
}

/* pad_fwd without offset (pam/native.py:163-164; integer form pam/cuda_kernels.cu:62-64) */
static float pad1(float a, float b)
{
    dec_t A = decomp(a), B = decomp(b);
    if (A.cls >= CLS_INF || B.cls >= CLS_INF) return NAN;
    if (B.cls == CLS_ZERO) {
        if (A.cls == CLS_ZERO) return NAN;                  /* 0/0 in the sign */
        return A.neg ? -INFINITY : INFINITY;                /* sign(a)/(+0) */
    }
    if (A.cls == CLS_ZERO) return u2f(B.neg ? 0x80000000u : 0u);
    int E = A.e - B.e; int32_t M = (int32_t)A.m - (int32_t)B.m;
    if (M < 0) { E--; M += (int32_t)ONE_M; }
    return compose(A.neg ^ B.neg, E, (uint32_t)M);
}

/* offset: the result is PAM-multiplied (PAD: divided) once more by the offset
 * (pam/native.py:59-60, 168-169).  1.0 means "off" as on the reference's GPU
 * path (pam/cuda_bindings.py:31-32). */
static float pam_off(float a, float b, float off)
{ float c = pam1(a, b); return off == 1.0f ? c : pam1(c, off); }
static float pad_off(float a, float b, float off)
{ float c = pad1(a, b); return off == 1.0f ? c : pad1(c, off); }

/* pa_log2_fwd (pam/native.py:24-30): fl(e + m), sign ignored */
static float palog2(float x)
{
    dec_t X = decomp(x);
    if (X.cls >= CLS_INF) return NAN;
    if (X.cls == CLS_ZERO) return -INFINITY;
    return (float)((double)X.e + (double)X.m / 8388608.0);
}

/* pa_exp2_fwd (pam/native.py:34-39): (2**floor x) * where(isfinite(floor x), (1 + x) - floor x, 1),
 * every operation rounded to fp32 in that order. */
static float paexp2(float x)
{
    float f = floorf(x), t, p;
    if (isnan(f)) return NAN;
    if (isinf(f)) { t = 1.0f; p = f > 0 ? INFINITY : 0.0f; }
    else {
        volatile float t1 = 1.0f + x;
        volatile float t2 = t1 - f;
        t = t2;
        p = (f >= 128.0f) ? INFINITY : (f <= -150.0f) ? 0.0f : ldexpf(1.0f, (int)f);
    }
    return (float)((double)p * (double)t);
}

/* pa_exp_fwd / pa_log_fwd (pam/native.py:199-212) */
static float paexp(float x, float l2b, float off) { return paexp2(pam_off(x, l2b, off)); }
static float palog(float x, float l2b, float off) { return pad_off(palog2(x), l2b, off); }

/* pam_bwd, exact derivative w.r.t. a (pam/native.py:65-77; integer form
 * pam/cuda_kernels.cu:48-57): delta * sign(b) * 2**(b_e + [a_m + b_m >= 1]). */
static float pam_bwd1(float a, float b, float delta, float off)
{
    if (off != 1.0f) b = pam1(b, off);
    dec_t A = decomp(a), B = decomp(b);
    float sgn, p;
    if (B.cls == CLS_NAN) return NAN;
    if (B.cls == CLS_ZERO) { sgn = 0.0f; p = 0.0f; }
    else if (B.cls == CLS_INF) { sgn = B.neg ? -1.0f : 1.0f; p = INFINITY; }
    else {
        int carry = (A.cls <= CLS_FIN) && (A.m + B.m >= ONE_M);   /* NaN mantissa compares false */
        sgn = B.neg ? -1.0f : 1.0f; p = pow2i(B.e + carry);
    }
    volatile float t = delta * sgn;
    return (float)((double)t * (double)p);
}

/* pad_bwd, derivative w.r.t. b (pam/cuda_kernels.cu:85-108), literal */
static float pad_bwd1(float a, float b, float delta, float off)
{
    float out = pad_off(a, b, off);
    float om = u2f(f2u(out) & ~MANT_MASK);
    float bm = u2f(f2u(b) & EXPO_MASK);
    volatile float q = om / bm;
    volatile float r = -q;
    return r * delta;
}

/* pa_exp2_bwd (pam/cuda_kernels.cu:115-123) */
static float paexp2_bwd(float x, float dy)
{ return u2f(f2u(paexp2(x)) & ~MANT_MASK) * dy; }

/* pa_log2_bwd (pam/cuda_kernels.cu:132-136): pow(2, -floor(log2 x)) * dy, no abs */
static float palog2_bwd(float x, float dy)
{
    dec_t X = decomp(x); float p;
    if (X.cls == CLS_NAN) return NAN;
    if (X.cls == CLS_ZERO) p = INFINITY;            /* log2(+-0) = -inf */
    else if (X.neg) return NAN;                     /* log2 of a negative number */
    else if (X.cls == CLS_INF) p = 0.0f;
    else p = pow2i(-X.e);
    return p * dy;
}

/* the unsigned-abs-free pa_log2 of the GPU reference (pam/cuda_kernels.cu:125-130) */
static float palog2_signed(float x)
{ return (f2u(x) >> 31) && !isnan(x) && x != 0.0f ? NAN : palog2(x); }

/* pa_exp_bwd / pa_log_bwd kernels (pam/cuda_kernels.cu:386-391, 481-484) */
static float paexp_bwd(float x, float dy, float l2b, float off)
{ return pam_bwd1(x, l2b, paexp2_bwd(pam_off(x, l2b, off), dy), off); }
static float palog_bwd(float x, float dy, float l2b, float off)
{ return palog2_bwd(x, pam_bwd1(palog2_signed(x), pad_off(1.0f, l2b, off), dy, 1.0f)); }

/* ------------------------------------------------------------------ chain */

/* fl(e + m) with exact e: equals palog2; -inf for 0, NaN for inf/NaN */
static float chain_exp2(float s)
{
    /* pa_exp2_fwd on an already-rounded fp32 argument */
    return paexp2(s);
}

static float pam_chain1(float a, float b)
{
    dec_t A = decomp(a), B = decomp(b);
    float sa = A.cls == CLS_ZERO ? 0.0f : A.cls == CLS_NAN ? 0.0f : (A.neg ? -1.0f : 1.0f);
    float sb = B.cls == CLS_ZERO ? 0.0f : B.cls == CLS_NAN ? 0.0f : (B.neg ? -1.0f : 1.0f);
    volatile float sign = sa * sb;
    volatile float s = palog2(a) + palog2(b);
    volatile float r = sign * chain_exp2(s);
    return r;
}

static float pad_chain1(float a, float b)
{
    dec_t A = decomp(a), B = decomp(b);
    float sa = A.cls == CLS_ZERO ? 0.0f : A.cls == CLS_NAN ? 0.0f : (A.neg ? -1.0f : 1.0f);
    float sb = B.cls == CLS_ZERO ? 0.0f : B.cls == CLS_NAN ? 0.0f : (B.neg ? -1.0f : 1.0f);
    volatile float sign = sa / sb;
    volatile float s = palog2(a) - palog2(b);
    volatile float r = sign * chain_exp2(s);
    return r;
}

static float pam_chain(float a, float b, float off, int has_off)
{ float c = pam_chain1(a, b); return has_off ? pam_chain1(c, off) : c; }
static float pad_chain(float a, float b, float off, int has_off)
{ float c = pad_chain1(a, b); return has_off ? pad_chain1(c, off) : c; }

/* pa_exp_fwd / pa_log_fwd as native.py composes them from its float-chain pam/pad */
static float paexp_chain(float x, float l2b, float off, int has_off)
{ return paexp2(pam_chain(x, l2b, off, has_off)); }
static float palog_chain(float x, float l2b, float off, int has_off)
{ return pad_chain(palog2(x), l2b, off, has_off); }

/* ------------------------------------------------------------------ arrays */

#define EW2(NAME, EXPR) \
    void NAME(const float *a, const float *b, float *c, size_t n, float off) { \
        _Pragma("omp parallel for schedule(static)") \
        for (size_t i = 0; i < n; i++) c[i] = EXPR; }

EW2(pamo_pam,       pam_off(a[i], b[i], off))
EW2(pamo_pad,       pad_off(a[i], b[i], off))
/* chain flavour: off == 1.0 is still applied when has_off is requested through the
 * *_chain_off entry points (native.py applies an explicit offset of 1.0). */
EW2(pamo_pam_chain, pam_chain(a[i], b[i], off, 0))
EW2(pamo_pad_chain, pad_chain(a[i], b[i], off, 0))
EW2(pamo_pam_chain_off, pam_chain(a[i], b[i], off, 1))
EW2(pamo_pad_chain_off, pad_chain(a[i], b[i], off, 1))

#define EW3(NAME, EXPR) \
    void NAME(const float *a, const float *b, const float *d, float *c, size_t n, float off) { \
        _Pragma("omp parallel for schedule(static)") \
        for (size_t i = 0; i < n; i++) c[i] = EXPR; }

EW3(pamo_pam_bwd, pam_bwd1(a[i], b[i], d[i], off))
EW3(pamo_pad_bwd, pad_bwd1(a[i], b[i], d[i], off))

void pamo_pa_log2(const float *x, float *y, size_t n)
{ for (size_t i = 0; i < n; i++) y[i] = palog2(x[i]); }
void pamo_pa_exp2(const float *x, float *y, size_t n)
{ for (size_t i = 0; i < n; i++) y[i] = paexp2(x[i]); }

void pamo_pa_exp(const float *x, float *y, size_t n, float log2_base, float off)
{
    _Pragma("omp parallel for schedule(static)")
    for (size_t i = 0; i < n; i++) y[i] = paexp(x[i], log2_base, off);
}
void pamo_pa_log(const float *x, float *y, size_t n, float log2_base, float off)
{
    _Pragma("omp parallel for schedule(static)")
    for (size_t i = 0; i < n; i++) y[i] = palog(x[i], log2_base, off);
}
void pamo_pa_exp_chain(const float *x, float *y, size_t n, float log2_base, float off, int has_off)
{ for (size_t i = 0; i < n; i++) y[i] = paexp_chain(x[i], log2_base, off, has_off); }
void pamo_pa_log_chain(const float *x, float *y, size_t n, float log2_base, float off, int has_off)
{ for (size_t i = 0; i < n; i++) y[i] = palog_chain(x[i], log2_base, off, has_off); }
void pamo_pa_exp_bwd(const float *x, const float *dy, float *dx, size_t n, float log2_base, float off)
{
    _Pragma("omp parallel for schedule(static)")
    for (size_t i = 0; i < n; i++) dx[i] = paexp_bwd(x[i], dy[i], log2_base, off);
}
void pamo_pa_log_bwd(const float *x, const float *dy, float *dx, size_t n, float log2_base, float off)
{
    _Pragma("omp parallel for schedule(static)")
    for (size_t i = 0; i < n; i++) dx[i] = palog_bwd(x[i], dy[i], log2_base, off);
}

/* ------------------------------------------------------------------ GEMM
 *
 * Y[b][i][j] = sum_k  mul(L[b][i][k], R[b][k][j])            (pam/cuda_kernels.cu:608-627)
 *
 * mode 0  PAM forward; the offset is folded into the right operand first,
 *         R' = pam(R, offset), so each product is pam(L, R')
 * mode 1  ordinary fp32 multiply (standard_mul, pam/cuda_kernels.cu:522-524), fused into the
 *         accumulate as one fma, which is what the reference's compiler does with a*b + c
 * mode 2  exact backward, delta on the left:  pam_bwd(D[i][j], R[k][j], L[i][k])
 * mode 3  exact backward, delta on the right: pam_bwd(D[i][j], L[i][k], R[k][j])
 *         (operand roles pam/cuda_kernels.cu:795-809)
 *
 * Accumulation: fp32, k ascending into one accumulator that starts at +0
 * (pam/cuda_kernels.cu:601).  kchunk > 0 selects a split order: every chunk of kchunk
 * consecutive k is summed that way from +0; every kgroup consecutive chunk sums are added in
 * ascending order (the first one is the starting value); the group sums are then added in
 * ascending order from +0.
 * Strides are in elements: (batch, row, col) per operand.
 */
void pamo_gemm(int mode, long batch, long M, long N, long K,
               const float *L, long lb, long lr, long lc,
               const float *R, long rb, long rr, long rc,
               const float *D, long db, long dr, long dc,
               float *Y, long yb, long yr, long yc,
               float off, long kchunk, long kgroup)
{
    if (kchunk <= 0 || kchunk > K) kchunk = K > 0 ? K : 1;
    if (kgroup <= 0) kgroup = 1;
    _Pragma("omp parallel for collapse(2) schedule(static)")
    for (long b = 0; b < batch; b++)
        for (long i = 0; i < M; i++) {
            const float *Lp = L + b * lb + i * lr;
            for (long j = 0; j < N; j++) {
                const float *Rp = R + b * rb + j * rc;
                float d = (mode >= 2) ? D[b * db + i * dr + j * dc] : 0.0f;
                volatile float total = 0.0f, group = 0.0f;
                long nchunk = 0;
                for (long k0 = 0; k0 < K || k0 == 0; k0 += kchunk) {
                    long k1 = k0 + kchunk < K ? k0 + kchunk : K;
                    volatile float acc = 0.0f;
                    for (long k = k0; k < k1; k++) {
                        float l = Lp[k * lc], r = Rp[k * rr], p;
                        switch (mode) {
                        case 0: p = pam1(l, off == 1.0f ? r : pam1(r, off)); break;
                        case 1: acc = fmaf(l, r, acc); continue;   /* nvcc contracts a*b + c into one fma */
                        case 2: p = pam_bwd1(d, r, l, off); break;
                        default: p = pam_bwd1(d, l, r, off); break;
                        }
                        acc = acc + p;
                    }
                    group = (nchunk % kgroup == 0) ? acc : group + acc;
                    nchunk++;
                    if (nchunk % kgroup == 0 || k1 >= K) total = total + group;
                    if (K == 0) break;
                }
                Y[b * yb + i * yr + j * yc] = total;
            }
        }
}

/* Fast forward GEMM for timing the CPU baseline: same arithmetic as mode 0 in the
 * normal range only (integer add, no edge classes), contiguous row-major L[M,K],
 * R[K,N].  Used by the benchmark, never by parity tests. */
void pamo_gemm_fast(long M, long N, long K, const float *L, const float *R, float *Y)
{
    _Pragma("omp parallel for schedule(static)")
    for (long i = 0; i < M; i++) {
        float *y = Y + i * N;
        for (long j = 0; j < N; j++) y[j] = 0.0f;
        for (long k = 0; k < K; k++) {
            uint32_t li = f2u(L[i * K + k]) - BIAS_BITS;
            const float *r = R + k * N;
            for (long j = 0; j < N; j++) y[j] += u2f(li + f2u(r[j]));
        }
    }
}

/* ------------------------------------------------------------------ row-wise compositions
 * softmax, logsumexp / log_softmax, mean and layer_norm of the reference's op library
 * (pam/pam_ops.py:288-378) written out as the chain of primitive calls they make, and the
 * softmax gradient as autograd chains the primitives' backward formulas
 * (pam/cuda_bindings.py:43-57, 78-97, 224-239).  The one thing the reference leaves open,
 * the order of torch.sum along a row, is fixed to the order of the GPU kernels:
 * 64 strided partial sums from +0, then a butterfly p[l] = p[l] + p[l ^ s], s = 32 .. 1.
 * Rows of 4097 ... 16384 values are summed by 1024 threads instead: 1024 strided partial sums
 * from +0, the butterfly within each group of 64 consecutive partial sums, then the 16 group
 * sums added in ascending order. */
static float butterfly64(const float *in)
{
    float p[64], q[64];
    memcpy(p, in, sizeof p);
    for (int s = 32; s >= 1; s >>= 1) {
        for (int l = 0; l < 64; ++l) { volatile float t = p[l] + p[l ^ s]; q[l] = t; }
        memcpy(p, q, sizeof p);
    }
    return p[0];
}

static float row_sum_fixed(const float *v, long n)
{
    if (n > 4096 && n <= 16384) {
        float part[1024];
        for (int t = 0; t < 1024; ++t) {
            volatile float s = 0.0f;
            for (long i = t; i < n; i += 1024) s = s + v[i];
            part[t] = s;
        }
        volatile float total = butterfly64(part);
        for (int w = 1; w < 16; ++w) total = total + butterfly64(part + 64 * w);
        return total;
    }
    float p[64], q[64];
    for (int l = 0; l < 64; ++l) {
        volatile float s = 0.0f;
        for (long i = l; i < n; i += 64) s = s + v[i];
        p[l] = s;
    }
    for (int s = 32; s >= 1; s >>= 1) {
        for (int l = 0; l < 64; ++l) { volatile float t = p[l] + p[l ^ s]; q[l] = t; }
        memcpy(p, q, sizeof p);
    }
    return p[0];
}

static float *row_buffer(long n) { return (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1)); }

static const float LOG2_E = (float)1.4426950408889634;   /* math.log2(math.e) as an fp32 tensor */
static const float LN_2 = (float)0.6931471805599453;     /* math.log(2.0) as an fp32 tensor */

static int is_neg_inf(float x) { return f2u(x) == 0xff800000u; }
static float scaled_x(float x, float off, int mask_inf)
{ return (mask_inf && is_neg_inf(x)) ? x : pam_off(x, LOG2_E, off); }
static float exp2_op(float t, float off) { return paexp(t, 1.0f, off); }     /* pa_exp_fwd(base 2) */
static float log2_op(float v, float off) { return palog(v, 1.0f, off); }     /* pa_log_fwd(base 2) */

/* floor(max) over the whole tensor, NaN propagating like torch.max (pam/pam_ops.py:318-319) */
static float global_shift(const float *x, size_t count, float off, int mask_inf)
{
    float mx = -INFINITY; int nan = 0;
    for (size_t i = 0; i < count; ++i) {
        float v = scaled_x(x[i], off, mask_inf);
        if (isnan(v)) nan = 1; else if (v > mx) mx = v;
    }
    return nan ? NAN : floorf(mx);
}

static float softmax_weight(float x, float shift, float off)
{
    if (is_neg_inf(x)) return 0.0f;
    volatile float t = scaled_x(x, off, 0) - shift;
    return exp2_op(t, off);
}

void pamo_softmax_fwd(const float *x, float *y, float *row_sum, float *shift_out, long rows, long n, float off)
{
    float shift = global_shift(x, (size_t)rows * (size_t)n, off, 1);
    *shift_out = shift;
    #pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        float *e = row_buffer(n);
        for (long i = 0; i < n; ++i) e[i] = softmax_weight(x[r * n + i], shift, off);
        float total = row_sum_fixed(e, n);
        for (long i = 0; i < n; ++i) y[r * n + i] = pad_off(e[i], total, off);
        row_sum[r] = total;
        free(e);
    }
}

void pamo_softmax_bwd(const float *x, const float *dy, const float *row_sum, float shift, float *dx,
                      long rows, long n, float off, int approx_a, int approx_b, int approx_exp)
{
    #pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        const float *xr = x + r * n, *g = dy + r * n;
        float total = row_sum[r], inv = pad_off(1.0f, total, off);
        float *e = row_buffer(n), *term = row_buffer(n);
        for (long i = 0; i < n; ++i) {
            e[i] = softmax_weight(xr[i], shift, off);
            /* pad_autograd.backward, second operand (the broadcast row sum) */
            if (approx_b) { volatile float t = pam_off(pad_off(pad_off(e[i], total, off), total, off), g[i], off); term[i] = -t; }
            else term[i] = pad_bwd1(e[i], total, g[i], off);
        }
        float dtotal = row_sum_fixed(term, n);          /* gradient of the expanded row sum */
        for (long i = 0; i < n; ++i) {
            int masked = is_neg_inf(xr[i]);
            float de0 = approx_a ? pam_off(inv, g[i], off) : pam_bwd1(e[i], inv, g[i], 1.0f);
            volatile float de = de0 + dtotal;            /* pad's first operand + the sum's broadcast */
            if (masked) de = 0.0f;                       /* where(x == -inf, 0, exp2(..)) */
            volatile float t = scaled_x(xr[i], off, 1) - shift;
            float dt;
            if (approx_exp) dt = pam_off(pam_off(exp2_op(t, off), LN_2, off), de, off);
            else dt = paexp_bwd(t, de, 1.0f, off);
            if (masked) dt = 0.0f;                       /* where(x == -inf, -inf, mul(..)) */
            dx[r * n + i] = approx_a ? pam_off(dt, LOG2_E, off) : pam_bwd1(xr[i], LOG2_E, dt, off);
        }
        free(e); free(term);
    }
}

/* lse[r] and/or y[r][i] = x - lse (either may be NULL) */
void pamo_logsumexp_fwd(const float *x, float *lse, float *y, long rows, long n, float off)
{
    float shift = global_shift(x, (size_t)rows * (size_t)n, off, 0);
    #pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        float *e = row_buffer(n);
        for (long i = 0; i < n; ++i) { volatile float t = scaled_x(x[r * n + i], off, 0) - shift; e[i] = exp2_op(t, off); }
        float total = row_sum_fixed(e, n);
        free(e);
        /* log2 of the total is called without the keyword arguments (pam/pam_ops.py:341): no offset */
        volatile float s = shift + log2_op(total, 1.0f);
        float out = pad_off(s, LOG2_E, off);
        if (lse) lse[r] = out;
        if (y) for (long i = 0; i < n; ++i) { volatile float d = x[r * n + i] - out; y[r * n + i] = d; }
    }
}

void pamo_row_mean_fwd(const float *x, float *y, long rows, long n, float off)
{
    #pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) y[r] = pad_off(row_sum_fixed(x + r * n, n), (float)n, off);
}

void pamo_layer_norm_fwd(const float *x, const float *weight, const float *bias, float *y, long rows, long n,
                         float eps, float off)
{
    #pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        const float *xr = x + r * n;
        float *c = row_buffer(n), *q = row_buffer(n);
        float mu = pad_off(row_sum_fixed(xr, n), (float)n, off);
        for (long i = 0; i < n; ++i) { volatile float d = xr[i] - mu; c[i] = d; q[i] = pam_off(d, d, off); }
        float var = pad_off(row_sum_fixed(q, n), (float)n, off);
        volatile float v = var + eps;
        /* pow(v, 0.5) (pam/pam_ops.py:70-79) */
        float denom = v == 0.0f ? 0.0f : exp2_op(pam_off(log2_op(v, off), 0.5f, off), off);
        for (long i = 0; i < n; ++i) {
            float out = pad_off(c[i], denom, off);
            if (weight) out = pam_off(out, weight[i], off);
            if (bias) { volatile float b = out + bias[i]; out = b; }
            y[r * n + i] = out;
        }
        free(c); free(q);
    }
}

/* ---- gradients of logsumexp / log_softmax and layer_norm: autograd's chain over the unfused ops
 * (formulas pam/cuda_bindings.py:43-57, 78-97, 224-239, 262-276; ops pam/pam_ops.py:331-378) ---- */
typedef struct { float off; int a, b, e; } grad_cfg;
static float g_mul_da(grad_cfg k, float a, float b, float g) { return k.a ? pam_off(g, b, k.off) : pam_bwd1(a, b, g, k.off); }
static float g_mul_db(grad_cfg k, float a, float b, float g) { return k.b ? pam_off(g, a, k.off) : pam_bwd1(b, a, g, k.off); }
static float g_div_da(grad_cfg k, float a, float b, float g)
{ float inv = pad_off(1.0f, b, k.off); return k.a ? pam_off(inv, g, k.off) : pam_bwd1(a, inv, g, 1.0f); }
static float g_div_db(grad_cfg k, float a, float b, float g)
{
    if (!k.b) return pad_bwd1(a, b, g, k.off);
    volatile float t = pam_off(pad_off(pad_off(a, b, k.off), b, k.off), g, k.off);
    return -t;
}
static float g_exp2_dx(grad_cfg k, float x, float g)
{ return k.e ? pam_off(pam_off(exp2_op(x, k.off), LN_2, k.off), g, k.off) : paexp_bwd(x, g, 1.0f, k.off); }
static float g_log2_dx(grad_cfg k, float x, float g)
{ return k.e ? pad_off(pad_off(g, x, k.off), LN_2, k.off) : palog_bwd(x, g, 1.0f, k.off); }

/* grad: [rows] for logsumexp, [rows][n] for log_softmax (y = x - logsumexp(x)) */
void pamo_logsumexp_bwd(const float *x, const float *grad, float shift, float *dx, long rows, long n, int log_softmax,
                        float off, int approx_a, int approx_b, int approx_exp)
{
    grad_cfg k = {off, approx_a, approx_b, approx_exp};
    #pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        const float *xr = x + r * n;
        float *e = row_buffer(n);
        for (long i = 0; i < n; ++i) { volatile float t = scaled_x(xr[i], off, 0) - shift; e[i] = exp2_op(t, off); }
        float total = row_sum_fixed(e, n);
        float g_out;
        if (log_softmax) { volatile float s = row_sum_fixed(grad + r * n, n); g_out = -s; } else g_out = grad[r];
        /* log2(total) carries no keyword arguments in the reference (pam/pam_ops.py:341): no offset, and the exact
         * gradient (pa_log_bwd) whatever approx_bwd says */
        volatile float u = shift + log2_op(total, 1.0f);
        float du = g_div_da(k, u, LOG2_E, g_out);
        float dtotal = palog_bwd(total, du, 1.0f, 1.0f);
        for (long i = 0; i < n; ++i) {
            volatile float t = scaled_x(xr[i], off, 0) - shift;
            float d = g_mul_da(k, xr[i], LOG2_E, g_exp2_dx(k, t, dtotal));
            if (log_softmax) { volatile float s = grad[r * n + i] + d; d = s; }
            dx[r * n + i] = d;
        }
        free(e);
    }
}

/* dx and, if dw_terms is given, the per-element terms whose sum over rows is the weight gradient */
void pamo_layer_norm_bwd(const float *x, const float *weight, const float *gy, float *dx, float *dw_terms, long rows, long n,
                         float eps, float off, int approx_a, int approx_b, int approx_exp)
{
    grad_cfg k = {off, approx_a, approx_b, approx_exp};
    #pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        const float *xr = x + r * n, *gr = gy + r * n;
        float *c = row_buffer(n), *q = row_buffer(n), *g = row_buffer(n), *t = row_buffer(n);
        float count = (float)n;
        float s1 = row_sum_fixed(xr, n), mu = pad_off(s1, count, off);
        for (long i = 0; i < n; ++i) { volatile float d = xr[i] - mu; c[i] = d; q[i] = pam_off(d, d, off); }
        float s2 = row_sum_fixed(q, n);
        volatile float v = pad_off(s2, count, off) + eps;
        float lg = log2_op(v, off), half = pam_off(lg, 0.5f, off);
        float denom = v == 0.0f ? 0.0f : exp2_op(half, off);
        for (long i = 0; i < n; ++i) {
            g[i] = gr[i];
            if (weight) {
                float xn = pad_off(c[i], denom, off);
                if (dw_terms) dw_terms[r * n + i] = g_mul_db(k, xn, weight[i], gr[i]);
                g[i] = g_mul_da(k, xn, weight[i], gr[i]);
            }
            t[i] = g_div_db(k, c[i], denom, g[i]);
        }
        float d = row_sum_fixed(t, n);
        if (v == 0.0f) d = 0.0f;
        d = g_exp2_dx(k, half, d);
        d = g_mul_da(k, lg, 0.5f, d);
        d = g_log2_dx(k, v, d);
        float ds2 = g_div_da(k, s2, count, d);
        for (long i = 0; i < n; ++i) {
            volatile float dc = g_div_da(k, c[i], denom, g[i]);
            dc = dc + g_mul_da(k, c[i], c[i], ds2);
            dc = dc + g_mul_db(k, c[i], c[i], ds2);
            t[i] = dc;
        }
        volatile float sdc = row_sum_fixed(t, n);
        float ds1 = g_div_da(k, s1, count, -sdc);
        for (long i = 0; i < n; ++i) { volatile float o = t[i] + ds1; dx[r * n + i] = o; }
        free(c); free(q); free(g); free(t);
    }
}

/* One Adam update with PAM ops (submodules/fairseq/fairseq/optim/adam.py:226-252 of the
 * reference tree), the chain of primitive calls written out; in place. */
void pamo_adam_step(float *p, const float *g, float *m, float *v, size_t n, float beta1, float one_minus_beta1,
                    float beta2, float one_minus_beta2, float eps, float decay, int has_decay, float step_size, float off)
{
    #pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        volatile float m1 = pam_off(m[i], beta1, off) + pam_off(g[i], one_minus_beta1, off);
        volatile float v0 = pam_off(v[i], beta2, off);
        volatile float v1 = v0 + pam_off(pam_off(g[i], g[i], off), one_minus_beta2, off);
        float root = v1 == 0.0f ? 0.0f : exp2_op(pam_off(log2_op(v1, off), 0.5f, off), off);
        volatile float denom = root + eps;
        volatile float p1 = p[i];
        if (has_decay) p1 = p1 - pam_off(p1, decay, off);
        volatile float p2 = p1 - pam_off(pad_off(m1, denom, off), step_size, off);
        p[i] = p2; m[i] = m1; v[i] = v1;
    }
}

int pamo_version(void) { return 2; }
