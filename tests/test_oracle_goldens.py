"""Pins the CPU oracle against golden vectors written from the reference's pam/native.py
(tests/golden/make_goldens.py).  Two facts are established:

  * the oracle's `chain` flavour reproduces native.py bit for bit (outside the band just
    below powers of two, where torch's floor(log2 x) is off by one), so it is a faithful
    model of the reference's float emulation;
  * the oracle's `exact` flavour (the integer definition the GPU kernels implement) equals
    native.py bit for bit wherever the float emulation is itself exact, has the same edge
    class everywhere, and otherwise stays within the float emulation's own rounding noise.
"""
import math

import numpy as np
import pytest

from _util import GOLDEN, assert_same_bits, below_pow2, f32, fclass, same_bits


def _grid():
    g = np.load(GOLDEN / "edge_grid.npz")
    ev = f32(g["values"])
    A = np.repeat(ev, len(ev)); B = np.tile(ev, len(ev))
    keep = ~(below_pow2(A) | below_pow2(B))
    return g, A, B, keep, float(g["offset"])


def test_edge_grid_chain_is_native(oracle):
    g, A, B, keep, off = _grid()
    assert keep.sum() > 3500
    assert_same_bits(oracle.pam_chain(A, B)[keep], f32(g["pam"])[keep], "pam")
    assert_same_bits(oracle.pad_chain(A, B)[keep], f32(g["pad"])[keep], "pad")
    assert_same_bits(oracle.pam_chain(A, B, off)[keep], f32(g["pam_off"])[keep], "pam offset")
    assert_same_bits(oracle.pad_chain(A, B, off)[keep], f32(g["pad_off"])[keep], "pad offset")


@pytest.mark.parametrize("op", ["pam", "pad", "pam_off", "pad_off"])
def test_edge_grid_exact_classes(oracle, op):
    g, A, B, keep, off = _grid()
    fn = oracle.pam if op.startswith("pam") else oracle.pad
    got = fn(A, B, off if op.endswith("off") else None)[keep]
    want = f32(g[op])[keep]
    # same class (zero / finite / inf / NaN) and same sign, zeros included
    assert (fclass(got) == fclass(want)).all()
    nn = ~np.isnan(want)
    assert (np.signbit(got[nn]) == np.signbit(want[nn])).all()
    # values: within the float emulation's noise (it keeps ~16 fraction bits of the log near |e| = 127)
    fin = fclass(want) == 1
    rel = np.abs(got[fin].astype(np.float64) - want[fin]) / np.abs(want[fin].astype(np.float64))
    assert rel.max() <= 2.0 ** -16
    # operands with |exponent| <= 100 and short mantissas: bit for bit
    ea = np.abs(np.frexp(A[keep])[1]); eb = np.abs(np.frexp(B[keep])[1])
    short = ((A[keep].view(np.uint32) | B[keep].view(np.uint32)) & 0xFF) == 0
    sel = short & (ea <= 100) & (eb <= 100) & (fclass(A[keep]) == 1) & (fclass(B[keep]) == 1) if not op.endswith("off") else np.zeros_like(short)
    assert_same_bits(got[sel], want[sel], op)


def test_short_mantissa_exact_is_native(oracle):
    g = np.load(GOLDEN / "short_mantissa.npz")
    a, b, d = f32(g["a"]), f32(g["b"]), f32(g["d"])
    assert_same_bits(oracle.pam(a, b), f32(g["pam"]), "pam")
    assert_same_bits(oracle.pad(a, b), f32(g["pad"]), "pad")
    assert_same_bits(oracle.pam_bwd(a, b, d), f32(g["pam_bwd"]), "pam_bwd")
    off = float(g["offset"])
    assert_same_bits(oracle.pam_chain(a, b, off), f32(g["pam_off"]), "pam offset (chain)")
    assert_same_bits(oracle.pad_chain(a, b, off), f32(g["pad_off"]), "pad offset (chain)")
    assert np.allclose(oracle.pam(a, b, off), f32(g["pam_off"]), rtol=1e-5, atol=1e-8)
    assert np.allclose(oracle.pad(a, b, off), f32(g["pad_off"]), rtol=1e-5, atol=1e-8)


def test_full_mantissa(oracle):
    g = np.load(GOLDEN / "normal_fullmant.npz")
    a, b, d = f32(g["a"]), f32(g["b"]), f32(g["d"]); off = float(g["offset"])
    assert not (below_pow2(a) | below_pow2(b)).any()
    # the chain model explains every bit of native.py here
    assert_same_bits(oracle.pam_chain(a, b), f32(g["pam"]), "pam chain")
    assert_same_bits(oracle.pad_chain(a, b), f32(g["pad"]), "pad chain")
    assert_same_bits(oracle.pam_chain(a, b, off), f32(g["pam_off"]), "pam offset chain")
    assert_same_bits(oracle.pad_chain(a, b, off), f32(g["pad_off"]), "pad offset chain")
    # the exact backward has no float chain in it: bit for bit
    assert_same_bits(oracle.pam_bwd(a, b, d), f32(g["pam_bwd"]), "pam_bwd")
    assert_same_bits(oracle.pam_bwd(a, b, d, off), f32(g["pam_bwd_off"]), "pam_bwd offset")
    # the integer definition against native.py: the reference's own bar, and how far apart they are
    for name, got in (("pam", oracle.pam(a, b)), ("pad", oracle.pad(a, b)),
                      ("pam_off", oracle.pam(a, b, off)), ("pad_off", oracle.pad(a, b, off))):
        want = f32(g[name])
        assert np.allclose(got, want, rtol=1e-5, atol=1e-8), name
        ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
        assert ulp.max() <= 96, (name, ulp.max())      # wide-exponent half: |e| up to 40 costs ~6 bits
        assert 0.1 < (ulp == 0).mean() < 0.6       # native.py is NOT the integer add on general inputs


def test_ulp_histogram_is_the_recorded_one(oracle):
    """Distance between the integer definition and pam/native.py per ulp, the kept artifact
    tests/golden/ulp_histogram.json (tests/golden/make_ulp_histogram.py writes it)."""
    import json
    from _util import full_mantissa_histograms
    kept = json.loads((GOLDEN / "ulp_histogram.json").read_text())
    assert full_mantissa_histograms({"pam": oracle.pam, "pad": oracle.pad}) == kept
    for name, halves in kept.items():
        unit = halves["unit_normal"]; total = sum(unit.values())
        assert unit["0"] / total > 0.6 and max(map(int, unit)) <= 16, name            # N(0,1): two thirds identical, the rest a few ulp
        assert max(map(int, halves["wide_exponent"])) <= 96, name                     # |e| up to 40 costs native.py ~6 bits


def test_quotient_gradients_of_the_cpu_flavour(oracle):
    """pam/native.py:173-188 (pad_autograd, approx_bwd=True) computes the quotient's gradients by other formulas
    than pam/cuda_bindings.py:78-97, which the kernels follow.  The oracle keeps native's as an alternate:
    its chain flavour equals what torch autograd gave through native.pad bit for bit, its exact flavour to the
    reference's tolerance, and the two flavours of gradient agree to PAM's own accuracy."""
    g = np.load(GOLDEN / "pad_native_bwd.npz")
    a, b, d = f32(g["a"]), f32(g["b"]), f32(g["d"]); off = float(g["offset"])
    assert not (below_pow2(a) | below_pow2(b) | below_pow2(d)).any()
    for tag, o in (("", None), ("_off", off)):
        assert_same_bits(oracle.pad_chain(a, b, o), f32(g["c" + tag]), "forward" + tag)
        da, db = oracle.pad_grads_native(a, b, d, o, flavour="chain")
        keep = ~(below_pow2(oracle.pam_chain(a, d, o)) | below_pow2(oracle.pam_chain(b, b, o)))    # intermediate values in the log2 band
        assert_same_bits(da, f32(g["da" + tag]), "dA" + tag)
        assert_same_bits(db[keep], f32(g["db" + tag])[keep], "dB" + tag)
        assert keep.mean() > 0.999
        ea, eb = oracle.pad_grads_native(a, b, d, o, flavour="exact")
        assert np.allclose(ea, f32(g["da" + tag]), rtol=1e-5, atol=1e-12) and np.allclose(eb[keep], f32(g["db" + tag])[keep], rtol=1e-5, atol=1e-12)
        # the GPU flavour (pam/cuda_bindings.py:78-97): dA = pam(pad(1, B), delta), dB = -pam(pad(pad(A, B), B), delta)
        one = np.ones_like(a)
        ga = oracle.pam(oracle.pad(one, b, o), d, o)
        gb = -oracle.pam(oracle.pad(oracle.pad(a, b, o), b, o), d, o)
        assert np.allclose(ga, ea, rtol=0.15) and np.allclose(gb, eb, rtol=0.25)      # each PAM op is within 1/9 of the true one


def test_pow2_band(oracle):
    g = np.load(GOLDEN / "pow2_band.npz")
    x = f32(g["x"]); glitch = below_pow2(x)
    e_native = f32(g["exp"]); e_true = np.floor(np.log2(x.astype(np.float64))).astype(np.float32)
    # the reference reads the exponent one too high just below most powers of two, nowhere else
    assert (e_native[~glitch] == e_true[~glitch]).all()
    assert ((e_native[glitch] - e_true[glitch]) == 1).sum() >= 240
    assert_same_bits(oracle.pa_log2_raw(x)[~glitch], f32(g["pa_log2"])[~glitch], "pa_log2")
    b = np.full_like(x, 1.75); d = np.full_like(x, 3.0)
    assert_same_bits(oracle.pam_bwd(x, b, d)[~glitch], f32(g["pam_bwd_a"])[~glitch], "pam_bwd wrt band operand")
    assert_same_bits(oracle.pam_bwd(b, x, d)[~glitch], f32(g["pam_bwd_b"])[~glitch], "pam_bwd other operand")
    assert_same_bits(oracle.pam_chain(x, b), f32(g["pam"]), "pam chain on the band")
    # inside the band the exact slope is the true one: carry happens, native's misses it
    got = oracle.pam_bwd(x, b, d)[glitch]; nat = f32(g["pam_bwd_a"])[glitch]
    assert ((got == 6.0) & ((nat == 3.0) | (nat == 6.0))).all()


def test_exp_log(oracle):
    g = np.load(GOLDEN / "exp_log.npz")
    xs, xl = f32(g["x_exp"]), f32(g["x_log"]); off = float(g["offset"])
    ok_l = ~below_pow2(xl); ok_s = ~below_pow2(xs)
    assert_same_bits(oracle.pa_exp2_raw(xs), f32(g["pa_exp2_fwd"]), "pa_exp2_fwd")
    assert_same_bits(oracle.pa_log2_raw(xl)[ok_l], f32(g["pa_log2_fwd"])[ok_l], "pa_log2_fwd")
    for name, base in (("e", math.e), ("2", 2.0), ("10", 10.0)):
        assert_same_bits(oracle.pa_exp_chain(xs, base)[ok_s], f32(g[f"exp_{name}"])[ok_s], f"exp {name} chain")
        assert_same_bits(oracle.pa_log_chain(xl, base)[ok_l], f32(g[f"log_{name}"])[ok_l], f"log {name} chain")
        assert_same_bits(oracle.pa_exp_chain(xs, base, off)[ok_s], f32(g[f"exp_{name}_off"])[ok_s], f"exp {name} off chain")
        assert_same_bits(oracle.pa_log_chain(xl, base, off)[ok_l], f32(g[f"log_{name}_off"])[ok_l], f"log {name} off chain")
        # integer-definition flavour: same class, close in value where the result is normal
        for got, want in ((oracle.pa_exp(xs, base)[ok_s], f32(g[f"exp_{name}"])[ok_s]),
                          (oracle.pa_log(xl, base)[ok_l], f32(g[f"log_{name}"])[ok_l])):
            assert (fclass(got) == fclass(want)).mean() > 0.999
            sel = (fclass(want) == 1) & (np.abs(want) > 1e-30)
            assert np.allclose(got[sel], want[sel], rtol=3e-4, atol=1e-6)


def test_matmul_small_reference_operands(oracle):
    g = np.load(GOLDEN / "matmul_small.npz")
    for tag in ("p21", "p20"):
        A = f32(g[f"{tag}_a"]).reshape(5, 4); B = f32(g[f"{tag}_b"]).reshape(4, 3)
        C = oracle.gemm(A, B)
        assert np.allclose(C, f32(g[f"{tag}_c"]).reshape(5, 3), rtol=1e-5, atol=1e-8)
        ones = np.ones((5, 3), np.float32)
        dA = oracle.gemm(ones, np.ascontiguousarray(B.T), mode=oracle.MODE_BWD_DELTA_L, D=A)
        dB = oracle.gemm(np.ascontiguousarray(A.T), ones, mode=oracle.MODE_BWD_DELTA_R, D=B)
        assert np.allclose(dA, f32(g[f"{tag}_da_exact_sum"]).reshape(5, 4), rtol=1e-5, atol=1e-8)
        assert np.allclose(dB, f32(g[f"{tag}_db_exact_sum"]).reshape(4, 3), rtol=1e-5, atol=1e-8)
        delta = f32(g[f"{tag}_delta"]).reshape(5, 3)
        dA = oracle.gemm(delta, np.ascontiguousarray(B.T))
        dB = oracle.gemm(np.ascontiguousarray(A.T), delta)
        assert np.allclose(dA, f32(g[f"{tag}_da_approx"]).reshape(5, 4), rtol=1e-5, atol=1e-8)
        assert np.allclose(dB, f32(g[f"{tag}_db_approx"]).reshape(4, 3), rtol=1e-5, atol=1e-8)
    # with the -2.0 shift every entry is a signed power of two: products are exact, so bit for bit
    A = f32(g["p20_a"]).reshape(5, 4); B = f32(g["p20_b"]).reshape(4, 3)
    assert_same_bits(oracle.gemm(A, B), f32(g["p20_c"]).reshape(5, 3), "p20 forward")


def c0_operands():
    import torch
    A = torch.randn(256, 512, generator=torch.Generator().manual_seed(0)).numpy()
    B = torch.randn(512, 256, generator=torch.Generator().manual_seed(1)).numpy()
    dY = torch.randn(256, 256, generator=torch.Generator().manual_seed(2)).numpy()
    return A, B, dY


def test_matmul_config0(oracle):
    g = np.load(GOLDEN / "matmul_c0.npz")
    A, B, dY = c0_operands()
    assert_same_bits(A[0, :8], f32(g["a_head"]), "seeded A changed"); assert_same_bits(B[0, :8], f32(g["b_head"]), "seeded B changed")
    Y = oracle.gemm(A, B); want = f32(g["y"]).reshape(256, 256)
    assert np.abs(Y - want).max() / np.abs(want).max() <= 1e-5
    dA = oracle.gemm(dY, np.ascontiguousarray(B.T))[::8]; want = f32(g["da_rows"]).reshape(32, 512)
    assert np.abs(dA - want).max() / np.abs(want).max() <= 1e-5
    dB = oracle.gemm(np.ascontiguousarray(A.T), dY)[::8]; want = f32(g["db_rows"]).reshape(64, 256)
    assert np.abs(dB - want).max() / np.abs(want).max() <= 1e-5
