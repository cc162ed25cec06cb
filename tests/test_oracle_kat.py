"""Pins the CPU oracle without running the reference: its own known-answer vectors,
closed forms, invariants and brute force against the real-number definition."""
import itertools
import math

import numpy as np
import pytest

from _util import assert_same_bits, bits, f32, same_bits

BIAS = 0x3F800000


def test_reference_vectors(oracle):
    # the 15 triples of pam/test_pam.py:13-29, compared as the reference does (allclose)
    abc = np.array([
        [1.0, 1.0, 1.0], [1.2345, 1.0, 1.2345], [1.2345, 32.0, 32.0 * 1.2345], [-1.2345, 32.0, -32.0 * 1.2345],
        [1.2345, -32.0, -32.0 * 1.2345], [-1.2345, -32.0, 32.0 * 1.2345], [1.0, 0.0, 0.0], [0.0, -1.0, -0.0],
        [1.5, 1.5, 2.0], [1.3, -1.3, -1.6], [4.5, 3.0, 8 * (1 + (4.5 - 4) / 4 + (3.0 - 2) / 2)], [-6.0, 3.0, -16.0],
        [-3.5, -3.5, 8 * (1 + (3.5 - 2) / 2 + (3.5 - 2) / 2 - 1)], [1e-30, 1e-30, 0.0], [1e-30, -1e-30, -0.0],
    ], dtype=np.float32)
    for fn in (oracle.pam, oracle.pam_chain):
        c = fn(abc[:, 0], abc[:, 1])
        assert np.allclose(c, abc[:, 2], rtol=1e-5, atol=1e-8)
    # what the integer definition gives exactly: x32 is exact, 1.5*1.5 = 2, PAM(1.3,-1.3) is 1 ulp from -1.6
    c = oracle.pam(abc[:, 0], abc[:, 1])
    assert_same_bits(c[[0, 1, 2, 8, 11]], np.array([1.0, 1.2345, np.float32(32) * np.float32(1.2345), 2.0, -16.0], np.float32))
    assert bits(c[9:10])[0] == 0xBFCCCCCC
    # sign of an underflowed product and of a product with zero (pam/test_pam.py:20-21,27-28)
    assert_same_bits(c[[6, 7, 13, 14]], np.array([0.0, -0.0, 0.0, -0.0], np.float32))


def test_reference_nonfinite_vectors(oracle):
    # pam/test_pam.py:36-43: all six must be non-finite
    ab = np.array([[1e30, 1e30], [1e30, -1e30], [-np.inf, 1e-20], [np.nan, -1e-20], [np.inf, 0.0], [np.nan, 0.0]], np.float32)
    c = oracle.pam(ab[:, 0], ab[:, 1])
    assert (~np.isfinite(c)).all()
    assert_same_bits(c[:2], np.array([np.inf, -np.inf], np.float32))   # overflow keeps the sign (native classes)
    assert np.isnan(c[2:]).all()


def test_closed_form_integer_add(oracle):
    rng = np.random.RandomState(0)
    a = (rng.standard_normal(20000) * 2.0 ** rng.randint(-30, 30, 20000)).astype(np.float32)
    b = (rng.standard_normal(20000) * 2.0 ** rng.randint(-30, 30, 20000)).astype(np.float32)
    want = f32((bits(a) + bits(b) - np.uint32(BIAS)).astype(np.uint32))          # pam/cuda_kernels.cu:17-19
    assert_same_bits(oracle.pam(a, b), want, "pam")
    want = f32((bits(a) - bits(b) + np.uint32(BIAS)).astype(np.uint32))          # pam/cuda_kernels.cu:62-64
    assert_same_bits(oracle.pad(a, b), want, "pad")
    off = np.float32(1.0552)
    off_i = bits(np.array([off]))[0] - np.uint32(BIAS)                            # pam/cuda_kernels.cu:168
    assert_same_bits(oracle.pam(a, b, off), f32((bits(a) + bits(b) - np.uint32(BIAS) + off_i).astype(np.uint32)), "pam off")
    assert_same_bits(oracle.pad(a, b, off), f32((bits(a) - bits(b) + np.uint32(BIAS) - off_i).astype(np.uint32)), "pad off")
    d = rng.standard_normal(20000).astype(np.float32)
    s = f32(((bits(b) + (bits(a) & np.uint32(0x7FFFFF)) + off_i) & np.uint32(0xFF800000)).astype(np.uint32))
    assert_same_bits(oracle.pam_bwd(a, b, d, off), d * s, "pam_bwd")               # pam/cuda_kernels.cu:52-57


def test_invariants(oracle):
    rng = np.random.RandomState(1)
    a = (rng.standard_normal(5000) * 2.0 ** rng.randint(-20, 20, 5000)).astype(np.float32)
    b = (rng.standard_normal(5000) * 2.0 ** rng.randint(-20, 20, 5000)).astype(np.float32)
    assert_same_bits(oracle.pam(a, b), oracle.pam(b, a), "commutative")
    assert_same_bits(oracle.pam(a, 1.0), a, "x*1")
    p2 = (2.0 ** rng.randint(-20, 20, 5000)).astype(np.float32)
    assert_same_bits(oracle.pam(a, p2), a * p2, "x*2^k exact")            # relied on by pam/test_pam.py:151-216
    assert_same_bits(oracle.pad(a, p2), a / p2, "x/2^k exact")
    assert_same_bits(oracle.pad(a, a), np.ones_like(a), "x/x")
    assert_same_bits(oracle.pad(oracle.pam(a, b), b), a, "pad inverts pam")
    assert_same_bits(oracle.pam(-a, b), -oracle.pam(a, b), "sign symmetry")
    r = oracle.pam(a, b).astype(np.float64) / (a.astype(np.float64) * b.astype(np.float64))
    assert (r <= 1.0 + 1e-12).all() and (r >= 8.0 / 9.0 - 1e-12).all()


def _real_pam(x, y):
    """PAM on real numbers: 2^(ex+ey) (1 + mx + my), or 2^(ex+ey+1) (mx + my) when mx + my >= 1."""
    sx, sy = math.copysign(1, x), math.copysign(1, y)
    mx, ex = math.frexp(abs(x)); my, ey = math.frexp(abs(y))
    mx, ex, my, ey = 2 * mx - 1, ex - 1, 2 * my - 1, ey - 1
    m = mx + my
    v = 2.0 ** (ex + ey) * (1 + m) if m < 1 else 2.0 ** (ex + ey + 1) * m
    return sx * sy * v


def test_bruteforce_small_grid(oracle):
    # every pair of a 5-bit-mantissa grid over 9 exponents and both signs, against exact rationals
    vals = [s * 2.0 ** e * (1 + m / 32) for s in (1, -1) for e in range(-4, 5) for m in range(32)]
    a, b = map(np.array, zip(*itertools.product(vals, vals)))
    want = np.array([_real_pam(x, y) for x, y in zip(a, b)], dtype=np.float64)
    got = oracle.pam(a.astype(np.float32), b.astype(np.float32)).astype(np.float64)
    assert (got == want).all()
    # pad against its definition as the inverse of pam on this grid
    q = oracle.pad(a.astype(np.float32), b.astype(np.float32))
    assert_same_bits(oracle.pam(q, b.astype(np.float32)), a.astype(np.float32), "pam(pad(a,b),b)")


def test_subnormal_and_range_classes(oracle):
    tiny = f32(np.array([1], np.uint32))[0]                  # 2^-149
    # subnormal operands count as the real numbers they are
    assert_same_bits(oracle.pam([tiny], [2.0 ** 100]), np.array([2.0 ** -49], np.float32))
    assert_same_bits(oracle.pam([tiny * 3], [2.0 ** 100]), np.array([3 * 2.0 ** -49], np.float32))
    # gradual underflow rounds to nearest even on the subnormal grid
    assert_same_bits(oracle.pam([2.0 ** -100], [1.5 * 2.0 ** -49]), f32(np.array([2], np.uint32)))   # 1.5*2^-149 -> tie -> even
    assert_same_bits(oracle.pam([2.0 ** -100], [1.75 * 2.0 ** -49]), f32(np.array([2], np.uint32)))
    assert_same_bits(oracle.pam([2.0 ** -100], [1.25 * 2.0 ** -49]), f32(np.array([1], np.uint32)))
    assert_same_bits(oracle.pam([2.0 ** -100], [1.99 * 2.0 ** -50]), np.zeros(1, np.float32))        # 2**-150 is already 0
    assert_same_bits(oracle.pam([-(2.0 ** 100)], [2.0 ** 28]), np.array([-np.inf], np.float32))
    assert_same_bits(oracle.pam([2.0 ** 100], [1.5 * 2.0 ** 27]), np.array([1.5 * 2.0 ** 127], np.float32))
    # zero takes the sign of the other operand only (torch.sign(-0.) is +0)
    z = oracle.pam(np.array([0.0, -0.0, 0.0, -0.0, -0.0], np.float32), np.array([3.0, 3.0, -3.0, -3.0, -0.0], np.float32))
    assert_same_bits(z, np.array([0.0, 0.0, -0.0, -0.0, 0.0], np.float32))
    # division classes (pam/native.py:163-164)
    q = oracle.pad(np.array([1.0, -1.0, 0.0, 0.0, -0.0, np.inf, 1.0], np.float32),
                   np.array([0.0, -0.0, 0.0, -2.0, 2.0, 2.0, np.inf], np.float32))
    assert_same_bits(q, np.array([np.inf, -np.inf, np.nan, -0.0, 0.0, np.nan, np.nan], np.float32))


def test_exp_log_closed_forms(oracle):
    k = np.arange(-149, 128).astype(np.float32)
    assert_same_bits(oracle.pa_exp2_raw(k), np.ldexp(np.float32(1), k.astype(np.int32)).astype(np.float32), "exp2(k)")
    assert_same_bits(oracle.pa_exp2_raw(k[1:] + 0.5), (1.5 * np.ldexp(np.float64(1), k[1:].astype(np.int32))).astype(np.float32), "exp2(k+.5)")
    assert_same_bits(oracle.pa_exp2_raw([128.0, -150.0, -np.inf, np.inf, np.nan, 2.0 ** 26]),
                     np.array([np.inf, 0.0, 0.0, np.inf, np.nan, np.nan], np.float32))
    x = np.ldexp(np.float32(1.25), np.arange(-126, 128)).astype(np.float32)
    assert_same_bits(oracle.pa_log2_raw(x), (np.arange(-126, 128) + 0.25).astype(np.float32), "log2(1.25*2^k)")
    # pa_log2 of a normal number is an int -> float conversion of the re-biased bit pattern
    rng = np.random.RandomState(2)
    y = np.abs(rng.standard_normal(10000) * 2.0 ** rng.randint(-60, 60, 10000)).astype(np.float32)
    want = ((bits(y).astype(np.int64) - BIAS).astype(np.float32) * np.float32(2.0 ** -23)).astype(np.float32)
    assert_same_bits(oracle.pa_log2_raw(y), want, "log2 int form")
    assert_same_bits(oracle.pa_log2_raw(-y), want, "log2 ignores the sign")
    assert_same_bits(oracle.pa_log2_raw([0.0, np.inf, np.nan]), np.array([-np.inf, np.nan, np.nan], np.float32))
    # base 2 leaves exp2 / log2 untouched
    xs = (rng.standard_normal(2000) * 5).astype(np.float32)
    assert_same_bits(oracle.pa_exp(xs, 2.0), oracle.pa_exp2_raw(xs), "pa_exp base 2")
    assert_same_bits(oracle.pa_log(y, 2.0), oracle.pa_log2_raw(y), "pa_log base 2")


def test_pam_bwd_is_slope_of_forward(oracle):
    # derivative of the piecewise-affine forward by finite difference inside a segment
    rng = np.random.RandomState(3)
    a = ((1 + rng.randint(1, 2 ** 10 - 1, 3000) / 2.0 ** 10) * 2.0 ** rng.randint(-8, 8, 3000)).astype(np.float32)
    b = ((1 + rng.randint(1, 2 ** 10 - 1, 3000) / 2.0 ** 10) * 2.0 ** rng.randint(-8, 8, 3000) * rng.choice([-1, 1], 3000)).astype(np.float32)
    h = (a * 2.0 ** -12).astype(np.float32)
    slope = (oracle.pam(a + h, b).astype(np.float64) - oracle.pam(a, b)) / h
    got = oracle.pam_bwd(a, b, np.ones_like(a)).astype(np.float64)
    ma = np.frexp(a)[0] * 2 - 1; mb = np.frexp(np.abs(b))[0] * 2 - 1
    inside = np.abs(ma + mb - 1) > 2.0 ** -10          # away from the kink where the slope doubles
    assert inside.sum() > 2000 and (slope[inside] == got[inside]).all()
    # pad_bwd: d/db pad(a,b) by the same construction, away from kinks.  The reference formula
    # (pam/cuda_kernels.cu:97-107) divides by 2^e_b without b's sign, so it is the derivative for
    # b > 0 and its negative for b < 0; the oracle keeps the formula as written.
    hb = (np.abs(b) * 2.0 ** -12).astype(np.float32)
    slope = (oracle.pad(a, b + hb).astype(np.float64) - oracle.pad(a, b)) / hb
    got = oracle.pad_bwd(a, b, np.ones_like(a)).astype(np.float64)
    inside = (np.abs(ma - mb) > 2.0 ** -9) & (mb < 1 - 2.0 ** -9)
    assert inside.sum() > 2000 and (slope[inside] == (np.sign(b) * got)[inside]).all()


def test_exp_log_bwd_are_slopes_of_forward(oracle):
    """pa_exp_bwd / pa_log_bwd (closed forms of pam/cuda_kernels.cu:375-393, 470-486, for which the
    reference holds no CPU implementation and no test) against the derivative of the pinned forward
    functions: both are piecewise affine with power-of-two slopes, so a finite difference inside one
    affine piece gives the slope up to the rounding of the forward values."""
    rng = np.random.RandomState(6)
    n = 6000
    for base in (math.e, 2.0, 10.0):
        for off in (None, 1.0552):
            # exp: x with short mantissas; keep the points whose neighbours share the affine piece
            x = ((1 + rng.randint(1, 2 ** 10 - 1, n) / 2.0 ** 10) * 2.0 ** rng.randint(-3, 3, n) * rng.choice([-1, 1], n)).astype(np.float32)
            h = (np.abs(x) * 2.0 ** -10).astype(np.float32)
            f0, f1, f2 = (oracle.pa_exp(v, base, off).astype(np.float64) for v in (x - h, x, x + h))
            got = oracle.pa_exp_bwd(x, np.ones_like(x), base, off).astype(np.float64)
            left, right = (f1 - f0) / h, (f2 - f1) / h
            same_piece = np.abs(left / right - 1) < 2.0 ** -9               # no kink between x - h and x + h
            assert same_piece.sum() > n // 2
            assert (np.abs(right[same_piece] / got[same_piece] - 1) < 2.0 ** -7).all(), (base, off)
            # log: positive x
            y = np.abs(x)
            hy = (y * 2.0 ** -10).astype(np.float32)
            g0, g1, g2 = (oracle.pa_log(v, base, off).astype(np.float64) for v in (y - hy, y, y + hy))
            got = oracle.pa_log_bwd(y, np.ones_like(y), base, off).astype(np.float64)
            left, right = (g1 - g0) / hy, (g2 - g1) / hy
            same_piece = (np.abs(left / right - 1) < 2.0 ** -9) & (g1 != g0) & (np.abs(y - 1) > 2.0 ** -6)   # log2 near 0 runs through many pieces
            assert same_piece.sum() > n // 2
            assert (np.abs(right[same_piece] / got[same_piece] - 1) < 2.0 ** -6).all(), (base, off)
    # upstream gradient scales linearly
    x = np.array([0.7, -1.3, 2.5], np.float32); d = np.array([2.0, -4.0, 0.5], np.float32)
    assert_same_bits(oracle.pa_exp_bwd(x, d), (oracle.pa_exp_bwd(x, np.ones(3, np.float32)) * d).astype(np.float32), "linear in dy")


def test_gemm_power_of_two_equals_matmul(oracle):
    # construction of pam/test_pam.py:198-216: right operand all powers of two => PAM bmm == bmm
    rng = np.random.RandomState(4)
    X = (rng.randint(-128, 128, (11, 13, 15)) / 64.0).astype(np.float32)
    W = (2.0 ** rng.randint(-8, 8, (11, 15, 19))).astype(np.float32)
    assert_same_bits(oracle.gemm(X, W), np.matmul(X.astype(np.float64), W.astype(np.float64)).astype(np.float32), "bmm")
    assert_same_bits(oracle.gemm(X, W, mode=oracle.MODE_STD), oracle.gemm(X, W), "std == pam here")
    # transposed (column-major) operands through strides
    Xt = np.ascontiguousarray(X.transpose(0, 2, 1)).transpose(0, 2, 1)
    Wt = np.ascontiguousarray(W.transpose(0, 2, 1)).transpose(0, 2, 1)
    assert_same_bits(oracle.gemm(Xt, Wt), oracle.gemm(X, W), "strided")


def test_gemm_bruteforce_and_orders(oracle):
    rng = np.random.RandomState(5)
    A = rng.standard_normal((7, 37)).astype(np.float32); B = rng.standard_normal((37, 5)).astype(np.float32)
    A[2, 3] = 0.0; B[4, 1] = -0.0; A[5, 5] = 1e-39
    want = np.zeros((7, 5), np.float32)
    for i in range(7):
        for j in range(5):
            acc = np.float32(0)
            for k in range(37):
                acc = np.float32(acc + oracle.pam(A[i, k:k + 1], B[k:k + 1, j])[0])
            want[i, j] = acc
    assert_same_bits(oracle.gemm(A, B), want, "sequential-k")
    # chunked order: chunk sums added in ascending order
    want = np.zeros((7, 5), np.float32)
    for i in range(7):
        for j in range(5):
            tot = np.float32(0)
            for k0 in range(0, 37, 8):
                acc = np.float32(0)
                for k in range(k0, min(k0 + 8, 37)):
                    acc = np.float32(acc + oracle.pam(A[i, k:k + 1], B[k:k + 1, j])[0])
                tot = np.float32(tot + acc)
            want[i, j] = tot
    assert_same_bits(oracle.gemm(A, B, kchunk=8), want, "chunked-k")
    # offset folds into the right operand
    assert_same_bits(oracle.gemm(A, B, offset=1.0552), oracle.gemm(A, oracle.pam(B, 1.0552)), "offset")
    # exact backward modes against the elementwise definition (pam/cuda_kernels.cu:795-809)
    D = rng.standard_normal((7, 5)).astype(np.float32)
    got = oracle.gemm(A, B, mode=oracle.MODE_BWD_DELTA_L, D=D)
    want = np.zeros((7, 5), np.float32)
    for i in range(7):
        for j in range(5):
            acc = np.float32(0)
            for k in range(37):
                acc = np.float32(acc + oracle.pam_bwd(D[i, j:j + 1], B[k:k + 1, j], A[i, k:k + 1])[0])
            want[i, j] = acc
    assert_same_bits(got, want, "exact bwd delta_L")
    got = oracle.gemm(A, B, mode=oracle.MODE_BWD_DELTA_R, D=D)
    for i in range(7):
        for j in range(5):
            acc = np.float32(0)
            for k in range(37):
                acc = np.float32(acc + oracle.pam_bwd(D[i, j:j + 1], A[i, k:k + 1], B[k:k + 1, j])[0])
            want[i, j] = acc
    assert_same_bits(got, want, "exact bwd delta_R")


def test_float_chain_baseline_agrees_with_the_integer_definition(oracle):
    """The torch float-chain restatement that bench.py times as its second CPU baseline (the reference's class of CPU
    algorithm: float log2 / add / exp2, all products materialised) against the exact oracle: powers of two exactly,
    full mantissas to the rounding of the fp32 log2 sum (a few 1e-7 of the largest sum)."""
    import torch
    from oracle import float_chain
    rng = np.random.RandomState(5)
    a = rng.standard_normal((24, 40)).astype(np.float32); b = rng.standard_normal((40, 28)).astype(np.float32)
    a[3, 5] = 0.0; b[7, 2] = -0.0
    got = float_chain.pam_matmul(torch.from_numpy(a), torch.from_numpy(b)).numpy()
    want = oracle.gemm(a, b)
    assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max()
    p2a = np.ldexp(1.0, rng.randint(-8, 8, (6, 9))).astype(np.float32) * rng.choice([-1.0, 1.0], (6, 9)).astype(np.float32)
    p2b = np.ldexp(1.0, rng.randint(-8, 8, (9, 5))).astype(np.float32)
    assert_same_bits(float_chain.pam_matmul(torch.from_numpy(p2a), torch.from_numpy(p2b)).numpy(), p2a @ p2b, "powers of two")
    x = rng.standard_normal(4096).astype(np.float32); y = rng.standard_normal(4096).astype(np.float32)
    e = float_chain.pam(torch.from_numpy(x), torch.from_numpy(y)).numpy()
    assert np.abs(e - oracle.pam(x, y)).max() <= 2e-6 * np.abs(e).max()
