"""PAM products as a chain of float tensor operations on the CPU -- test infrastructure and a benchmark baseline only.

The same class of algorithm as the reference's CPU path (pam/native.py:11-61, 117-131: piecewise-affine log2 of both
operands, a float add, piecewise-affine exp2, the products of a matrix product as one broadcast n x k x m tensor that
is then summed over k), written here on torch.frexp / torch.ldexp.  The log2 sum is rounded to fp32, so results agree
with the exact integer definition to about 1e-6 relative, not bit for bit; tests/test_oracle_kat.py holds that bound.
Zeros give zero; other special values are not handled (the benchmark feeds normal numbers).
"""
import torch


def pa_log2(mag):
    """e + (m - 1) for mag = m 2^e, 1 <= m < 2."""
    half, exp = torch.frexp(mag)                      # mag = half 2^exp, 0.5 <= half < 1
    return (exp - 1).to(mag.dtype) + (2.0 * half - 1.0)


def pa_exp2(t):
    """(1 + frac(t)) 2^floor(t)."""
    whole = torch.floor(t)
    return torch.ldexp(1.0 + (t - whole), whole.to(torch.int32))


def pam(a, b):
    """a (*) b elementwise, broadcasting."""
    sign = torch.sign(a) * torch.sign(b)              # zero for a zero operand
    tiny = torch.finfo(a.dtype).tiny
    return sign * pa_exp2(pa_log2(a.abs().clamp_min(tiny)) + pa_log2(b.abs().clamp_min(tiny)))


def pam_matmul(a, b):
    """sum over k of a[n, k] (*) b[k, m]: every product materialised, as the reference's CPU path does."""
    return pam(a[:, :, None], b[None, :, :]).sum(dim=1)
