// Scalar piecewise-affine arithmetic for gfx950 device code.
//
// Every function takes and returns fp32 values; "bits" are their IEEE-754 patterns.
// The common case (normal operands, normal result) is the integer add of the
// reference's GPU kernel (pam/cuda_kernels.cu:17-19, 62-64).  Everything that kernel
// delegates to a float-multiply guard is decided here on the bit patterns instead, and
// follows the classes of the reference's float emulation (pam/native.py:16-20, 38-39,
// 54-55, 163-164): inf/NaN operands give NaN, a zero operand gives a zero whose sign is
// that of the other operand, subnormal operands count as the real numbers they are,
// results underflow gradually (round to nearest even) and overflow to +-inf.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pamdev {

constexpr uint32_t kBias = 0x3f800000u;
constexpr uint32_t kMant = 0x007fffffu;
constexpr uint32_t kExpo = 0x7f800000u;
constexpr uint32_t kSign = 0x80000000u;
constexpr uint32_t kQNaN = 0x7fc00000u;

__device__ __forceinline__ uint32_t f2u(float x) { return __float_as_uint(x); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

// The matrix kernels' plain inner loop (integer add of the bit patterns) is exact when every value of a k-tile is a
// normal number with magnitude in [2^-63, 2^64) -- biased exponent 64 ... 190 -- or a zero, which has loops of its
// own.  Any other value (subnormal, inf, NaN, an extreme exponent) needs the full definition of the product.
// The staging classifier, the per-k-step record and the marked k-step of the mixed loop all decide by this.
constexpr uint32_t kPlainExpMin = 64u, kPlainExpMax = 190u;
__device__ __forceinline__ bool needs_full_definition(uint32_t bits)
{
    return (bits & ~kSign) != 0 && ((bits >> 23) & 0xffu) - kPlainExpMin > kPlainExpMax - kPlainExpMin;
}
// The same predicate over many values at two instructions each: the biased exponents of the values (a zero counts as
// 127) folded by min and max, compared once at the end.  The staging classifier sees sixteen values per lane and
// k-tile; the predicate per value cost the convolutions, whose padding sends nearly every k-tile through it, 8 %.
struct ExponentRange {
    uint32_t emin = 255u, emax = 0u;
    __device__ __forceinline__ void see(uint32_t bits, bool is_zero)
    {
        const uint32_t e = is_zero ? 127u : (bits >> 23) & 0xffu;
        emin = min(emin, e); emax = max(emax, e);
    }
    __device__ __forceinline__ bool needs_full_definition() const { return emin < kPlainExpMin || emax > kPlainExpMax; }
};

// Finite non-zero magnitude -> unbiased exponent and 23-bit fraction, subnormals normalised.
__device__ __forceinline__ void split_mag(uint32_t mag, int& e, uint32_t& m)
{
    if (mag >= 0x00800000u) { e = (int)(mag >> 23) - 127; m = mag & kMant; }
    else {
        int sh = __clz((int)mag) - 8;            // brings the leading one to bit 23
        e = -126 - sh; m = (mag << sh) & kMant;
    }
}

// sign | 2^E (1 + M / 2^23) rounded once (nearest even) into fp32; E >= 128 -> inf,
// E <= -150 -> 0 (the reference evaluates 2**E first, and 2**-150 is already 0).
__device__ __forceinline__ uint32_t join_mag(uint32_t sign, int E, uint32_t M)
{
    if (E >= 128) return sign | kExpo;
    if (E <= -150) return sign;
    if (E >= -126) return sign | ((uint32_t)(E + 127) << 23) | M;
    uint32_t sig = 0x00800000u | M;
    int sh = -126 - E;                           // 1 .. 23
    uint32_t q = sig >> sh;
    uint32_t rest = sig << (32 - sh);            // discarded bits, left aligned
    q += (rest > 0x80000000u) || (rest == 0x80000000u && (q & 1u));
    return sign | q;
}

// An operand decomposed for the general (any class) product and quotient:
//   ex = unbiased exponent plus `bias`, or a sentinel: -4096 for zero, +2^20 for inf/NaN;
//   fr = 23-bit fraction with subnormals normalised, the sign in bit 31 (cleared for zeros,
//        whose sign the reference's float emulation ignores, pam/native.py:54, 163).
struct Split { int ex; uint32_t fr; };

__device__ __forceinline__ Split split_operand(uint32_t u, int bias)
{
    uint32_t mag = u & ~kSign;
    Split s;
    if (__builtin_expect(mag - 0x00800000u < 0x7f000000u, 1)) {
        s.ex = (int)(mag >> 23) - 127 + bias; s.fr = u & (kSign | kMant);
    } else if (mag == 0) { s.ex = -4096; s.fr = 0; }
    else if (mag >= kExpo) { s.ex = 1 << 20; s.fr = 0; }
    else { int e; uint32_t m; split_mag(mag, e, m); s.ex = e + bias; s.fr = (u & kSign) | m; }
    return s;
}

// Product of decomposed operands whose biases add up to 127.  Zeros fall out of the
// underflow branch with the sign of the other operand, inf/NaN out of the overflow branch.
__device__ __forceinline__ float pam_from_split(const Split& a, const Split& b)
{
    uint32_t f = a.fr + b.fr;                        // bit 31: sign, bit 23: fraction carry
    int eb = a.ex + b.ex + (int)((f >> 23) & 1u);    // biased exponent of the product
    uint32_t sign = f & kSign, frac = f & kMant;
    if (__builtin_expect((uint32_t)(eb - 1) < 254u, 1)) return u2f(sign | ((uint32_t)eb << 23) | frac);
    if (eb > (1 << 19)) return u2f(kQNaN);           // an inf/NaN operand
    return u2f(join_mag(sign, eb - 127, frac));      // overflow, gradual underflow, zero
}

// Quotient of decomposed operands (a carries bias 127, b bias 0).
__device__ __forceinline__ float pad_from_split(const Split& a, const Split& b)
{
    uint32_t f = a.fr - b.fr;                        // bit 31: sign (xor), bit 23: fraction borrow
    int eb = a.ex - b.ex - (int)((f >> 23) & 1u);
    uint32_t sign = (a.fr ^ b.fr) & kSign, frac = f & kMant;
    if (__builtin_expect((uint32_t)(eb - 1) < 254u && (uint32_t)(b.ex + 2048) < 4096u, 1))
        return u2f(sign | ((uint32_t)eb << 23) | frac);
    if (a.ex > (1 << 19) || b.ex > (1 << 19)) return u2f(kQNaN);          // inf/NaN anywhere
    if (b.ex == -4096) return u2f(a.ex == -4096 ? kQNaN : (sign | kExpo));        // x / 0, 0 / 0
    return u2f(join_mag(sign, eb - 127, frac));
}

// Any class of operands, without a branch: the hardware's frexp takes subnormal operands apart, the two fractions are
// added exactly in fp32 (23-bit fractions, sums below 2), and ldexp puts the result together with the one rounding
// that gradual underflow needs (nearest even) and the overflow to inf.  What remains are selects: results at or below
// 2^-150 are zero (the reference evaluates 2**E first, pam/native.py:38-39), a zero operand gives a zero with the
// sign of the other operand only, an inf or NaN operand gives NaN.
//   |a| = ma 2^xa with ma in [0.5, 1): fraction fa = 2 ma - 1, exponent xa - 1; ga = ma - 0.5 = fa / 2.
constexpr unsigned kClassZero = 0x060u;     // v_cmp_class masks: 0x060 = +-0, 0x207 = signalling NaN, quiet NaN, -inf, +inf

__device__ __forceinline__ float pam_general(uint32_t ai, uint32_t bi)
{
    const float a = u2f(ai), b = u2f(bi);
    const float ga = __builtin_amdgcn_frexp_mantf(__builtin_fabsf(a)) - 0.5f, gb = __builtin_amdgcn_frexp_mantf(__builtin_fabsf(b)) - 0.5f;
    const int xa = __builtin_amdgcn_frexp_expf(a), xb = __builtin_amdgcn_frexp_expf(b);
    const float s = ga + gb;                                   // (fa + fb) / 2, exact
    const bool carry = s >= 0.5f;
    const float half_mant = carry ? s : s + 0.5f;               // (fa + fb) / 2 or (1 + fa + fb) / 2, in [0.5, 1), exact
    const int e2 = xa + xb + (carry ? 0 : -1);                  // result = half_mant 2^e2, its exponent E = e2 - 1
    float r = __builtin_amdgcn_ldexpf(half_mant, e2);
    r = e2 <= -149 ? 0.0f : r;
    const bool za = __builtin_amdgcn_classf(a, kClassZero), zb = __builtin_amdgcn_classf(b, kClassZero);
    const uint32_t sign = ((za ? 0u : ai) ^ (zb ? 0u : bi)) & kSign;
    uint32_t out = (za | zb) ? sign : (f2u(r) | sign);
    const bool bad = __builtin_amdgcn_classf(a, 0x207u) | __builtin_amdgcn_classf(b, 0x207u);    // NaN or inf
    return u2f(bad ? kQNaN : out);
}

// PAM product a (*) b.
__device__ __forceinline__ float pam_mul(float a, float b)
{
    uint32_t ai = f2u(a), bi = f2u(b);
    uint32_t ma = ai & ~kSign, mb = bi & ~kSign;
    uint32_t s = ma + mb - kBias;                // magnitude of the product when all is normal
    bool normal = (ma - 0x00800000u < 0x7f000000u) & (mb - 0x00800000u < 0x7f000000u) &
                  (s - 0x00800000u < 0x7f000000u);
    if (__builtin_expect(normal, 1)) return u2f(s | ((ai ^ bi) & kSign));
    return pam_general(ai, bi);
}

// The quotient the same way: the fractions are subtracted; a negative difference borrows from the exponent.
// x / +-0 is +-inf by the sign of x, 0 / 0 is NaN, 0 / y is a zero with the sign of y only, inf or NaN anywhere is NaN
// (pam/native.py:163-164).
__device__ __forceinline__ float pad_general(uint32_t ai, uint32_t bi)
{
    const float a = u2f(ai), b = u2f(bi);
    const float ga = __builtin_amdgcn_frexp_mantf(__builtin_fabsf(a)), gb = __builtin_amdgcn_frexp_mantf(__builtin_fabsf(b));
    const int xa = __builtin_amdgcn_frexp_expf(a), xb = __builtin_amdgcn_frexp_expf(b);
    const float d = ga - gb;                                    // (fa - fb) / 2, exact, in (-0.5, 0.5)
    const bool borrow = d < 0.0f;
    const float half_mant = borrow ? d + 1.0f : d + 0.5f;        // (2 + fa - fb) / 2 or (1 + fa - fb) / 2, in [0.5, 1), exact
    const int e2 = xa - xb + (borrow ? 0 : 1);                   // result = half_mant 2^e2
    float r = __builtin_amdgcn_ldexpf(half_mant, e2);
    r = e2 <= -149 ? 0.0f : r;
    const bool za = __builtin_amdgcn_classf(a, kClassZero), zb = __builtin_amdgcn_classf(b, kClassZero);
    const uint32_t sign = ((za ? 0u : ai) ^ (zb ? 0u : bi)) & kSign;
    uint32_t out = zb ? ((ai & kSign) | kExpo) : za ? sign : (f2u(r) | sign);
    const bool bad = __builtin_amdgcn_classf(a, 0x207u) | __builtin_amdgcn_classf(b, 0x207u) | (za & zb);
    return u2f(bad ? kQNaN : out);
}

// PAM quotient a (/) b.
__device__ __forceinline__ float pad_div(float a, float b)
{
    uint32_t ai = f2u(a), bi = f2u(b);
    uint32_t ma = ai & ~kSign, mb = bi & ~kSign;
    uint32_t s = ma - mb + kBias;
    bool normal = (ma - 0x00800000u < 0x7f000000u) & (mb - 0x00800000u < 0x7f000000u) &
                  (s - 0x00800000u < 0x7f000000u);
    if (__builtin_expect(normal, 1)) return u2f(s | ((ai ^ bi) & kSign));
    return pad_general(ai, bi);
}

// The offset is one more PAM product (quotient for pad) applied to the result
// (pam/native.py:59-60, 168-169); 1.0 switches it off (pam/cuda_bindings.py:31-32).
__device__ __forceinline__ float pam_mul_off(float a, float b, float off, bool has_off)
{ float c = pam_mul(a, b); return has_off ? pam_mul(c, off) : c; }
__device__ __forceinline__ float pad_div_off(float a, float b, float off, bool has_off)
{ float c = pad_div(a, b); return has_off ? pad_div(c, off) : c; }

// 2**k for an integer k the way fp32 pow gives it: exact down to 2^-149, 0 below, inf above 127.
__device__ __forceinline__ float pow2_int(int k)
{
    uint32_t u = k >= 128 ? kExpo : k >= -126 ? (uint32_t)(k + 127) << 23 : k >= -149 ? 1u << (k + 149) : 0u;
    return u2f(u);
}

// pa_log2 (pam/native.py:24-30): exponent plus mantissa fraction of |x|, one rounding.
__device__ __forceinline__ float pa_log2(float x)
{
    uint32_t mag = f2u(x) & ~kSign;
    if (mag >= kExpo) return u2f(kQNaN);
    if (mag == 0) return u2f(0xff800000u);
    int e; uint32_t m; split_mag(mag, e, m);
    return (float)(e * (1 << 23) + (int)m) * 0x1p-23f;
}

// pa_exp2 (pam/native.py:34-39): 2**floor(x) * ((1 + x) - floor(x)), fp32 operations in that order.
__device__ __forceinline__ float pa_exp2(float x)
{
    float f = floorf(x);
    if (f != f) return u2f(kQNaN);
    uint32_t fm = f2u(f) & ~kSign;
    if (fm == kExpo) return f > 0.0f ? f : 0.0f;
    float t = (1.0f + x) - f;
    float p = f >= 128.0f ? u2f(kExpo) : f <= -150.0f ? 0.0f : pow2_int((int)f);
    return p * t;
}

// Exact derivative of a (*) b w.r.t. a, times delta (pam/native.py:65-77,
// pam/cuda_kernels.cu:48-57): (delta * sign(b)) * 2**(e_b + [m_a + m_b >= 1]).
__device__ __forceinline__ float pam_mul_bwd(float a, float b, float delta, float off, bool has_off)
{
    if (has_off) b = pam_mul(b, off);
    uint32_t ai = f2u(a), bi = f2u(b);
    uint32_t ma = ai & ~kSign, mb = bi & ~kSign;
    bool fast = (mb - 0x00800000u < 0x7e800000u) & (ma - 0x00800000u < 0x7f000000u);
    if (__builtin_expect(fast, 1))
        return delta * u2f((bi + (ai & kMant)) & ~kMant);
    if (mb > kExpo) return u2f(kQNaN);
    float sgn, p;
    if (mb == 0) { sgn = 0.0f; p = 0.0f; }
    else if (mb == kExpo) { sgn = (bi & kSign) ? -1.0f : 1.0f; p = u2f(kExpo); }
    else {
        int eb; uint32_t fb; split_mag(mb, eb, fb);
        uint32_t fa = 0;
        if (ma != 0 && ma < kExpo) { int ea; split_mag(ma, ea, fa); }
        sgn = (bi & kSign) ? -1.0f : 1.0f;
        p = pow2_int(eb + (int)((fa + fb) >> 23));
    }
    float t = delta * sgn;
    return t * p;
}

// Derivative of a (/) b w.r.t. b, times delta, as the reference writes it
// (pam/cuda_kernels.cu:85-108): -(pow2 part of a (/) b) / 2^e_b * delta.
__device__ __forceinline__ float pad_div_bwd(float a, float b, float delta, float off, bool has_off)
{
    float out = pad_div_off(a, b, off, has_off);
    float om = u2f(f2u(out) & ~kMant);
    float bm = u2f(f2u(b) & kExpo);
    float q = om / bm;
    return (-q) * delta;
}

// pa_exp2_bwd (pam/cuda_kernels.cu:115-123)
__device__ __forceinline__ float pa_exp2_bwd(float x, float dy)
{ return u2f(f2u(pa_exp2(x)) & ~kMant) * dy; }

// pa_log2_bwd (pam/cuda_kernels.cu:132-136): 2**(-floor(log2 x)) * dy, x is not made positive
__device__ __forceinline__ float pa_log2_bwd(float x, float dy)
{
    uint32_t xi = f2u(x), mag = xi & ~kSign;
    if (mag > kExpo) return u2f(kQNaN);
    float p;
    if (mag == 0) p = u2f(kExpo);
    else if (xi & kSign) return u2f(kQNaN);
    else if (mag == kExpo) p = 0.0f;
    else { int e; uint32_t m; split_mag(mag, e, m); p = pow2_int(-e); }
    return p * dy;
}

// pa_log2 without the abs, as the reference GPU kernel has it (pam/cuda_kernels.cu:125-130)
__device__ __forceinline__ float pa_log2_signed(float x)
{
    uint32_t xi = f2u(x);
    if ((xi & kSign) && (xi & ~kSign) != 0 && (xi & ~kSign) <= kExpo) return u2f(kQNaN);
    return pa_log2(x);
}

// exp2, log2 and the square root as the op library reaches them: through the base-2 forms of
// the exp / log entry points, pa_exp2(t (*) log2 2) and pa_log2(v) (/) log2 2
// (pam/cuda_bindings.py:246, 283), and pow(v, 0.5) = exp2(log2(v) (*) 0.5) with zero kept at
// zero (pam/pam_ops.py:70-79).
__device__ __forceinline__ float exp2_entry(float t, float off, bool has_off)
{ return pa_exp2(pam_mul_off(t, 1.0f, off, has_off)); }
__device__ __forceinline__ float log2_entry(float v, float off, bool has_off)
{ return pad_div_off(pa_log2(v), 1.0f, off, has_off); }
__device__ __forceinline__ float pow_half(float v, float off, bool has_off)
{ return v == 0.0f ? 0.0f : exp2_entry(pam_mul_off(log2_entry(v, off, has_off), 0.5f, off, has_off), off, has_off); }

// Exact gradients of the base-2 exp / log entry points as the reference's kernels compute them
// (pam/cuda_kernels.cu:386-391, 481-484 with log2 2 = 1).
__device__ __forceinline__ float exp2_entry_bwd(float x, float dy, float off, bool has_off)
{ return pam_mul_bwd(x, 1.0f, pa_exp2_bwd(pam_mul_off(x, 1.0f, off, has_off), dy), off, has_off); }
__device__ __forceinline__ float log2_entry_bwd(float x, float dy, float off, bool has_off)
{ return pa_log2_bwd(x, pam_mul_bwd(pa_log2_signed(x), pad_div_off(1.0f, 1.0f, off, has_off), dy, 1.0f, false)); }

// ---------------------------------------------------------------- unchecked forms
// Chains of many primitive calls per element (row kernels, optimizer step) pay a range check
// and a branch per call when built from the functions above.  The forms below compute the
// normal-range result without branching and fold every magnitude they touch into a running
// min / max; `Span::normal()` then tells, once per chain, whether each operand and each
// result was a normal number -- in which case every value equals what the checked function
// returns -- or the chain has to be redone with the checked functions.
struct Span {
    uint32_t lo = 0x7f7fffffu, hi = 0x00800000u;
    uint32_t exp_arg = 0u;                        // largest magnitude given to pa_exp2_unchecked
    bool in_exp_range = true;
    __device__ __forceinline__ void see(uint32_t mag) { lo = min(lo, mag); hi = max(hi, mag); }
    __device__ __forceinline__ bool normal() const
    { return in_exp_range && lo >= 0x00800000u && hi < kExpo && exp_arg <= 0x42fc0000u; }     // |exp2 argument| <= 126
};

__device__ __forceinline__ float pam_unchecked(float a, float b, Span& sp)
{
    uint32_t ai = f2u(a), bi = f2u(b), ma = ai & ~kSign, mb = bi & ~kSign;
    uint32_t s = ma + mb - kBias;
    sp.see(ma); sp.see(mb); sp.see(s);
    return u2f(s | ((ai ^ bi) & kSign));
}
__device__ __forceinline__ float pad_unchecked(float a, float b, Span& sp)
{
    uint32_t ai = f2u(a), bi = f2u(b), ma = ai & ~kSign, mb = bi & ~kSign;
    uint32_t s = ma - mb + kBias;                 // a wrap lands above the exponent mask and is caught
    sp.see(ma); sp.see(mb); sp.see(s);
    return u2f(s | ((ai ^ bi) & kSign));
}
__device__ __forceinline__ float pam_unchecked_off(float a, float b, float off, bool has_off, Span& sp)
{ float c = pam_unchecked(a, b, sp); return has_off ? pam_unchecked(c, off, sp) : c; }
__device__ __forceinline__ float pad_unchecked_off(float a, float b, float off, bool has_off, Span& sp)
{ float c = pad_unchecked(a, b, sp); return has_off ? pad_unchecked(c, off, sp) : c; }

// pa_log2 of a normal number: (bits(|x|) - bias) / 2^23, one rounding in the conversion
__device__ __forceinline__ float pa_log2_unchecked(float x, Span& sp)
{
    uint32_t mag = f2u(x) & ~kSign;
    sp.see(mag);
    return (float)((int)mag - (int)kBias) * 0x1p-23f;
}
// pa_exp2 for |x| <= 126, where 2**floor(x) is a normal number and so is the result (the arguments in
// (126, 128), which would also do, are left to the checked function: one max per call instead of two compares)
__device__ __forceinline__ float pa_exp2_unchecked(float x, Span& sp)
{
    sp.exp_arg = max(sp.exp_arg, f2u(x) & ~kSign);                             // NaN is larger than any bound
    float f = floorf(x);
    float t = (1.0f + x) - f;
    return u2f((uint32_t)((int)f + 127) << 23) * t;
}
// Without an offset t (*) 1 is t itself when t is a normal number: only that is recorded.
__device__ __forceinline__ float exp2_entry_unchecked(float t, float off, bool has_off, Span& sp)
{
    if (!has_off) { sp.see(f2u(t) & ~kSign); return pa_exp2_unchecked(t, sp); }
    return pa_exp2_unchecked(pam_unchecked_off(t, 1.0f, off, has_off, sp), sp);
}

// Cheaper forms for the usual places in a chain.  Each records its result and those operands that its name does not
// excuse; for the excused ones the caller vouches: a constant, a value recorded earlier in the chain, a value that
// is a normal number by construction (a result of pa_exp2_unchecked).
// a (*) k, k a positive normal constant: records a and the result
__device__ __forceinline__ float pam_unchecked_const(float a, float k, Span& sp)
{
    const uint32_t ai = f2u(a), ma = ai & ~kSign, s = ma + (f2u(k) - kBias);
    sp.see(ma); sp.see(s);
    return u2f(s | (ai & kSign));
}
// a (*) b, a recorded earlier: records b and the result
__device__ __forceinline__ float pam_unchecked_seen(float a, float b, Span& sp)
{
    const uint32_t ai = f2u(a), bi = f2u(b), mb = bi & ~kSign, s = (ai & ~kSign) + mb - kBias;
    sp.see(mb); sp.see(s);
    return u2f(s | ((ai ^ bi) & kSign));
}
// a (*) a: records a and the result (which is positive)
__device__ __forceinline__ float pam_unchecked_square(float a, Span& sp)
{
    const uint32_t ma = f2u(a) & ~kSign, s = ma + ma - kBias;
    sp.see(ma); sp.see(s);
    return u2f(s);
}
// a (/) b, b a positive normal number recorded by the caller, a recorded earlier (or normal by construction):
// records the result
__device__ __forceinline__ float pad_unchecked_by_positive(float a, float b, Span& sp)
{
    const uint32_t ai = f2u(a), s = (ai & ~kSign) - f2u(b) + kBias;            // a wrap lands above the exponent mask and is caught
    sp.see(s);
    return u2f(s | (ai & kSign));
}
__device__ __forceinline__ float log2_entry_unchecked(float v, float off, bool has_off, Span& sp)
{ return pad_unchecked_off(pa_log2_unchecked(v, sp), 1.0f, off, has_off, sp); }
__device__ __forceinline__ float pow_half_unchecked(float v, float off, bool has_off, Span& sp)
{ return exp2_entry_unchecked(pam_unchecked_off(log2_entry_unchecked(v, off, has_off, sp), 0.5f, off, has_off, sp), off, has_off, sp); }

}  // namespace pamdev
