"""Parity of the HIP kernels with the CPU oracle, through the C ABI, on a real MI355X.

Bars: bit-exact (NaN compared as a class) against the oracle's exact flavour for every
elementwise op and for matrix products in the fixed accumulation order; against the
golden vectors written from the reference's pam/native.py: bit-exact where its float
emulation is exact, and its own allclose(rtol=1e-5, atol=1e-8) elsewhere, with every
differing element required to be one the oracle's model of that emulation reproduces.
"""
import math

import numpy as np
import pytest
import torch

from _util import GOLDEN, assert_same_bits, below_pow2, edge_values, f32, fclass, mixed_operands, same_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from pam_amd._abi import HipKernels, load_library
    load_library()
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return HipKernels()


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


OFFS = [None, 1.0552]


def ogemm(oracle, L, R, plan_shape=None, **kw):
    """The oracle's product in the fixed accumulation order the library uses for this shape
    (plan_shape = (batch, m, n, k) of the full product when L, R are a sample of it)."""
    from pam_amd import _abi
    L = np.asarray(L); R = np.asarray(R)
    batch = L.shape[0] if L.ndim == 3 else 1
    chunk = _abi.gemm_plan(*(plan_shape or (batch, L.shape[-2], R.shape[-1], L.shape[-1])))
    return oracle.gemm(L, R, kchunk=chunk, **kw)


def _o(off):
    return 1.0 if off is None else off


# ------------------------------------------------------------------ elementwise vs oracle

@pytest.mark.parametrize("off", OFFS)
def test_pam_pad_mixed(K, oracle, off):
    n = (1 << 20) + 3
    a, b = mixed_operands(n, 10), mixed_operands(n, 11)
    assert_same_bits(host(K.pam_fwd(dev(a), dev(b), _o(off))), oracle.pam(a, b, off), "pam_fwd")
    assert_same_bits(host(K.pad_fwd(dev(a), dev(b), _o(off))), oracle.pad(a, b, off), "pad_fwd")


@pytest.mark.parametrize("off", OFFS)
def test_edge_grid_all_pairs(K, oracle, off):
    ev = edge_values()
    a = np.repeat(ev, len(ev)); b = np.tile(ev, len(ev))
    assert_same_bits(host(K.pam_fwd(dev(a), dev(b), _o(off))), oracle.pam(a, b, off), "pam_fwd")
    assert_same_bits(host(K.pad_fwd(dev(a), dev(b), _o(off))), oracle.pad(a, b, off), "pad_fwd")
    d = np.resize(np.array([1.0, -3.0, 0.0, np.inf, 1e-40, np.nan, 2.5e38], np.float32), a.size)
    assert_same_bits(host(K.pam_bwd(dev(a), dev(b), dev(d), _o(off))), oracle.pam_bwd(a, b, d, off), "pam_bwd")
    assert_same_bits(host(K.pad_bwd(dev(a), dev(b), dev(d), _o(off))), oracle.pad_bwd(a, b, d, off), "pad_bwd")


@pytest.mark.parametrize("off", OFFS)
def test_exact_backward_mixed(K, oracle, off):
    n = (1 << 18) + 1
    a, b, d = mixed_operands(n, 20), mixed_operands(n, 21), mixed_operands(n, 22, edge_frac=0.005)
    assert_same_bits(host(K.pam_bwd(dev(a), dev(b), dev(d), _o(off))), oracle.pam_bwd(a, b, d, off), "pam_bwd")
    assert_same_bits(host(K.pad_bwd(dev(a), dev(b), dev(d), _o(off))), oracle.pad_bwd(a, b, d, off), "pad_bwd")


@pytest.mark.parametrize("off", OFFS)
@pytest.mark.parametrize("base", [math.e, 2.0, 10.0, 0.5])
def test_exp_log(K, oracle, base, off):
    rng = np.random.RandomState(30)
    xs = np.concatenate([np.linspace(-160, 160, 4097), rng.standard_normal(1 << 16) * 8, edge_values(),
                         [127.5, 128.0, -149.0, -149.5, -150.0, 2.0 ** 24, 2.0 ** 25, 1e30, -1e30]]).astype(np.float32)
    xl = np.concatenate([rng.rand(1 << 16) * 10, 2.0 ** (rng.rand(1 << 14) * 250 - 125), edge_values()]).astype(np.float32)
    dy = np.resize(mixed_operands(4099, 31, edge_frac=0.01), xs.size)
    assert_same_bits(host(K.pa_exp_fwd(dev(xs), base, _o(off))), oracle.pa_exp(xs, base, off), "pa_exp_fwd")
    assert_same_bits(host(K.pa_log_fwd(dev(xl), base, _o(off))), oracle.pa_log(xl, base, off), "pa_log_fwd")
    assert_same_bits(host(K.pa_exp_bwd(dev(xs), dev(dy), base, _o(off))), oracle.pa_exp_bwd(xs, dy, base, off), "pa_exp_bwd")
    dyl = np.resize(dy, xl.size)
    assert_same_bits(host(K.pa_log_bwd(dev(xl), dev(dyl), base, _o(off))), oracle.pa_log_bwd(xl, dyl, base, off), "pa_log_bwd")


def test_ragged_unaligned_and_broadcast(K, oracle):
    for n in (0, 1, 3, 5, 1023, 1025, 4099):
        a, b = mixed_operands(n + 1, 40 + n), mixed_operands(n + 1, 41 + n)
        # views that start 4 bytes into an allocation: the vector path must not be taken
        ta, tb = dev(a)[1:], dev(b)[1:]
        assert_same_bits(host(K.pam_fwd(ta, tb, 1.0)), oracle.pam(a[1:], b[1:]), f"pam n={n}")
        assert_same_bits(host(K.pad_fwd(ta, dev(b[1:]), 1.0)), oracle.pad(a[1:], b[1:]), f"pad n={n}")
    a = mixed_operands(70001, 50)
    for s in (1.5, 0.0, -0.0, float("inf"), 1e-41, -3.0e38):
        st = torch.tensor(s, device="cuda")
        A = dev(a[:70000]).reshape(7, 10000)
        assert_same_bits(host(K.pam_fwd(A, st.expand(A.shape), 1.0552)), oracle.pam(a[:70000].reshape(7, 10000), np.float32(s), 1.0552), "pam x*s")
        assert_same_bits(host(K.pam_fwd(st.expand(A.shape), A, 1.0)), oracle.pam(np.float32(s), a[:70000].reshape(7, 10000)), "pam s*x")
        assert_same_bits(host(K.pad_fwd(A, st.expand(A.shape), 1.0)), oracle.pad(a[:70000].reshape(7, 10000), np.float32(s)), "pad x/s")
        assert_same_bits(host(K.pad_fwd(st.expand(A.shape), A, 1.0552)), oracle.pad(np.float32(s), a[:70000].reshape(7, 10000), 1.0552), "pad s/x")
    # non-contiguous input (transposed view): copied like the reference's flatten()
    m = mixed_operands(6 * 50, 51).reshape(6, 50)
    assert_same_bits(host(K.pam_fwd(dev(m).T, dev(m.T.copy()), 1.0)), oracle.pam(m.T, m.T), "transposed view")


# ------------------------------------------------------------------ elementwise vs native.py goldens

def test_goldens_short_mantissa_bit_exact(K):
    g = np.load(GOLDEN / "short_mantissa.npz")
    a, b, d = f32(g["a"]), f32(g["b"]), f32(g["d"])
    assert_same_bits(host(K.pam_fwd(dev(a), dev(b), 1.0)), f32(g["pam"]), "pam vs native.py")
    assert_same_bits(host(K.pad_fwd(dev(a), dev(b), 1.0)), f32(g["pad"]), "pad vs native.py")
    assert_same_bits(host(K.pam_bwd(dev(a), dev(b), dev(d), 1.0)), f32(g["pam_bwd"]), "pam_bwd vs native.py")


def test_goldens_full_mantissa(K, oracle):
    g = np.load(GOLDEN / "normal_fullmant.npz")
    a, b, d = f32(g["a"]), f32(g["b"]), f32(g["d"]); off = float(g["offset"])
    cases = [("pam", K.pam_fwd, oracle.pam_chain, None), ("pad", K.pad_fwd, oracle.pad_chain, None),
             ("pam_off", K.pam_fwd, oracle.pam_chain, off), ("pad_off", K.pad_fwd, oracle.pad_chain, off)]
    for name, fn, chain, o in cases:
        got = host(fn(dev(a), dev(b), _o(o))); want = f32(g[name])
        assert np.allclose(got, want, rtol=1e-5, atol=1e-8), name           # the reference's own bar
        differ = ~same_bits(got, want)
        # every element where the integer add and native.py disagree is one where the model of
        # native.py's float chain reproduces native.py: the difference is its rounding, not ours
        assert same_bits(chain(a, b, o), want)[differ].all(), name
    assert_same_bits(host(K.pam_bwd(dev(a), dev(b), dev(d), 1.0)), f32(g["pam_bwd"]), "pam_bwd")
    assert_same_bits(host(K.pam_bwd(dev(a), dev(b), dev(d), off)), f32(g["pam_bwd_off"]), "pam_bwd offset")
    # how far the kernels are from pam/native.py, per unit of the last place: the recorded histogram
    import json
    from _util import full_mantissa_histograms
    fns = {"pam": lambda x, y, o: host(K.pam_fwd(dev(x), dev(y), _o(o))), "pad": lambda x, y, o: host(K.pad_fwd(dev(x), dev(y), _o(o)))}
    assert full_mantissa_histograms(fns) == json.loads((GOLDEN / "ulp_histogram.json").read_text())


def test_goldens_edge_grid_classes(K):
    g = np.load(GOLDEN / "edge_grid.npz")
    ev = f32(g["values"]); a = np.repeat(ev, len(ev)); b = np.tile(ev, len(ev))
    keep = ~(below_pow2(a) | below_pow2(b))
    for name, fn, o in (("pam", K.pam_fwd, 1.0), ("pad", K.pad_fwd, 1.0),
                        ("pam_off", K.pam_fwd, float(g["offset"])), ("pad_off", K.pad_fwd, float(g["offset"]))):
        got = host(fn(dev(a), dev(b), o))[keep]; want = f32(g[name])[keep]
        assert (fclass(got) == fclass(want)).all(), name
        nn = ~np.isnan(want)
        assert (np.signbit(got[nn]) == np.signbit(want[nn])).all(), name        # signed zeros and infinities
        fin = fclass(want) == 1
        rel = np.abs(got[fin].astype(np.float64) - want[fin]) / np.abs(want[fin].astype(np.float64))
        assert rel.max() <= 2.0 ** -16, name


def test_goldens_exp_log(K, oracle):
    g = np.load(GOLDEN / "exp_log.npz")
    xs, xl = f32(g["x_exp"]), f32(g["x_log"])
    ok_s, ok_l = ~below_pow2(xs), ~below_pow2(xl)
    for name, base in (("e", math.e), ("2", 2.0), ("10", 10.0)):
        got = host(K.pa_exp_fwd(dev(xs), base, 1.0))[ok_s]; want = f32(g[f"exp_{name}"])[ok_s]
        differ = ~same_bits(got, want)
        assert same_bits(oracle.pa_exp_chain(xs, base)[ok_s], want)[differ].all()
        sel = (fclass(want) == 1) & (np.abs(want) > 1e-30)
        assert np.allclose(got[sel], want[sel], rtol=3e-4, atol=1e-6)
        got = host(K.pa_log_fwd(dev(xl), base, 1.0))[ok_l]; want = f32(g[f"log_{name}"])[ok_l]
        differ = ~same_bits(got, want)
        assert same_bits(oracle.pa_log_chain(xl, base)[ok_l], want)[differ].all()
        sel = fclass(want) == 1
        assert np.allclose(got[sel], want[sel], rtol=3e-4, atol=1e-6)


# ------------------------------------------------------------------ matrix products vs oracle

def _layouts(x):
    """row-major, column-major (transposed storage) and a generic-stride view of the same matrix"""
    t = dev(x)
    cm = dev(np.ascontiguousarray(np.swapaxes(x, -1, -2))).transpose(-1, -2)
    wide = torch.zeros(*x.shape[:-1], x.shape[-1] * 2 + 1, device="cuda")
    wide[..., ::2][..., :x.shape[-1]] = t
    return {"rm": t, "cm": cm, "any": wide[..., ::2][..., :x.shape[-1]]}


def _rand(shape, seed, zeros=0.0, specials=False):
    rng = np.random.RandomState(seed)
    x = rng.standard_normal(shape).astype(np.float32)
    if zeros:
        x[rng.rand(*shape) < zeros] = 0.0
    if specials:
        flat = x.reshape(-1)
        idx = rng.choice(flat.size, size=max(4, flat.size // 200), replace=False)
        flat[idx] = np.resize(np.array([np.inf, -0.0, 1e-40, np.nan, 3e38, -1e-39, 2.0 ** -100, 2.0 ** 100], np.float32), idx.size)
    return x


SHAPES = [(5, 4, 3), (64, 16, 64), (70, 33, 45), (130, 100, 257), (128, 197, 128), (33, 1, 9), (257, 64, 192)]


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_matmul_forward_layouts(K, oracle, m, k, n):
    A, B = _rand((m, k), m + k), _rand((k, n), n + k + 1)
    want = ogemm(oracle, A, B)
    for la, ta in _layouts(A).items():
        for lb, tb in _layouts(B).items():
            assert_same_bits(host(K.pam_matmul_fwd(ta, tb, True, True, 1.0)), want, f"{la} x {lb}")
    assert_same_bits(host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0552)), ogemm(oracle, A, B, offset=1.0552), "offset")
    assert_same_bits(host(K.standard_matmul(dev(A), dev(B), True, True, 1.0)), ogemm(oracle, A, B, mode=oracle.MODE_STD), "standard")


@pytest.mark.parametrize("zeros,specials", [(0.5, False), (0.02, True), (1.0, False)])
def test_matmul_zeros_and_specials(K, oracle, zeros, specials):
    A, B = _rand((150, 75), 1, zeros, specials), _rand((75, 90), 2, zeros / 2, specials)
    for la, ta in _layouts(A).items():
        for lb, tb in _layouts(B).items():
            assert_same_bits(host(K.pam_matmul_fwd(ta, tb, True, True, 1.0)), ogemm(oracle, A, B), f"{la} x {lb}")
    assert_same_bits(host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0552)), ogemm(oracle, A, B, offset=1.0552), "offset")


@pytest.mark.parametrize("side", ["left", "right", "mixed"])
def test_matmul_zeros_in_one_operand(K, oracle, side):
    """k-tiles whose zeros sit in one operand only take their own loop (a stand-in for the zero and a
    0 / 1 factor in the accumulating fma): signed zeros, values at both ends of the range that this
    loop accepts, and in the mixed case k-tiles of all four kinds (none, left, right, both) in one product."""
    rng = np.random.RandomState(21)
    A, B = _rand((140, 192), 31), _rand((192, 130), 32)
    edge = np.array([2.0 ** -63, -(2.0 ** -63), np.nextafter(np.float32(2.0 ** 64), np.float32(0)), -1.5 * 2.0 ** 63], np.float32)
    A.reshape(-1)[rng.choice(A.size, 64, replace=False)] = np.resize(edge, 64)
    B.reshape(-1)[rng.choice(B.size, 64, replace=False)] = np.resize(edge, 64)
    za, zb = rng.rand(*A.shape) < 0.4, rng.rand(*B.shape) < 0.4
    if side == "left":
        zb[:] = False
    elif side == "right":
        za[:] = False
    else:                           # k in [0,32) none, [32,64) left, [64,96) right, [96,128) both, then left / right again
        za[:, :32] = False; zb[:32] = False; zb[32:64] = False; za[:, 64:96] = False; zb[128:160] = False; za[:, 160:] = False
    A[za] = np.where(rng.rand(int(za.sum())) < 0.5, 0.0, -0.0)
    B[zb] = np.where(rng.rand(int(zb.sum())) < 0.5, 0.0, -0.0)
    for la, ta in _layouts(A).items():
        for lb, tb in _layouts(B).items():
            assert_same_bits(host(K.pam_matmul_fwd(ta, tb, True, True, 1.0)), ogemm(oracle, A, B), f"{side}: {la} x {lb}")
    assert_same_bits(host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0552)), ogemm(oracle, A, B, offset=1.0552), "offset")
    # an all-zero row / column keeps its +0 sums
    A[3] = 0.0; B[:, 5] = -0.0
    assert_same_bits(host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0)), ogemm(oracle, A, B), "zero row and column")


@pytest.mark.parametrize("delta_l", [True, False])
@pytest.mark.parametrize("zeros,specials", [(0.0, False), (0.3, True)])
def test_matmul_exact_backward(K, oracle, delta_l, zeros, specials):
    L, R, D = _rand((70, 45), 3, zeros, specials), _rand((45, 97), 4, zeros, specials), _rand((70, 97), 5, zeros / 3, specials)
    mode = oracle.MODE_BWD_DELTA_L if delta_l else oracle.MODE_BWD_DELTA_R
    for off in OFFS:
        want = ogemm(oracle, L, R, mode=mode, D=D, offset=off)
        for ll, tl in _layouts(L).items():
            for lr, tr in _layouts(R).items():
                got = host(K.pam_matmul_bwd(tl, tr, dev(D), True, True, delta_l, _o(off)))
                assert_same_bits(got, want, f"{ll} x {lr} off={off}")


def _sparse_specials(shape, seed, every=600, zero_band=None):
    """N(0,1) with one value in `every` outside the plain range (subnormal, inf, NaN, huge, tiny) at seeded places, and
    zeros in a band of the k dimension: k-tiles then hold k-steps of every kind next to each other."""
    rng = np.random.RandomState(seed)
    x = rng.standard_normal(shape).astype(np.float32)
    flat = x.reshape(-1)
    idx = rng.choice(flat.size, size=max(3, flat.size // every), replace=False)
    flat[idx] = np.resize(np.array([1e-40, 2.0 ** 100, -1e-39, np.inf, 2.0 ** -100, 3e38, np.nan], np.float32), idx.size)
    if zero_band is not None:
        axis, lo, hi = zero_band
        band = [slice(None)] * x.ndim; band[axis] = slice(lo, hi)
        sub = x[tuple(band)]
        sub[rng.rand(*sub.shape) < 0.3] = 0.0
    return x


def test_matmul_few_specials_per_k_tile(K, oracle):
    """A value that needs the full definition sends only its own k-step of the k-tile there; the other steps of the tile
    take the plain form, or the zero-replacing one where the tile also holds zeros.  All layouts, forward and both exact
    gradients, k = 256 (32-deep tiles) and 100 (16-deep, ragged)."""
    for k in (256, 100):
        A = _sparse_specials((150, k), 40 + k, zero_band=(1, 40, 90))
        B = _sparse_specials((k, 90), 41 + k, zero_band=(0, 70, 100))
        want = ogemm(oracle, A, B)
        for la, ta in _layouts(A).items():
            for lb, tb in _layouts(B).items():
                assert_same_bits(host(K.pam_matmul_fwd(ta, tb, True, True, 1.0)), want, f"k={k} {la} x {lb}")
        assert_same_bits(host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0552)), ogemm(oracle, A, B, offset=1.0552), "offset")
        D = _sparse_specials((150, 90), 42 + k, every=900)
        for delta_l, mode in ((True, oracle.MODE_BWD_DELTA_L), (False, oracle.MODE_BWD_DELTA_R)):
            want = ogemm(oracle, A, B, mode=mode, D=D)
            for la, ta in _layouts(A).items():
                for lb, tb in _layouts(B).items():
                    assert_same_bits(host(K.pam_matmul_bwd(ta, tb, dev(D), True, True, delta_l, 1.0)), want, f"exact k={k} {la} x {lb}")


def test_matmul_tiny_values_next_to_small_sums(K, oracle):
    """A tiny value (subnormal, or below 2^-63) may pass as a zero in its k-step only where its products cannot change
    the sums they go to.  Here the sums are small themselves (about 2^-57), the tiny values' exponents run from far below
    to just below the plain range, and their products straddle the sums' last place: some k-steps take the full
    definition, some skip, and every sum must still carry the bits of the plain ascending-k order."""
    rng = np.random.RandomState(77)
    for k, scale_b in ((256, 1.0), (96, 2.0 ** -20)):
        A = (rng.standard_normal((150, k)) * 2.0 ** -60).astype(np.float32)
        B = (rng.standard_normal((k, 90)) * scale_b).astype(np.float32)
        flat = A.reshape(-1)
        idx = rng.choice(flat.size, size=flat.size // 150, replace=False)
        flat[idx] = (rng.uniform(1.0, 2.0, idx.size) * 2.0 ** rng.randint(-140, -63, idx.size) * rng.choice([-1.0, 1.0], idx.size)).astype(np.float32)
        fb = B.reshape(-1)
        jdx = rng.choice(fb.size, size=fb.size // 400, replace=False)
        fb[jdx] = (rng.uniform(1.0, 2.0, jdx.size) * 2.0 ** rng.randint(-149, -63, jdx.size)).astype(np.float32)
        want = ogemm(oracle, A, B)
        assert np.isfinite(want).all() and np.count_nonzero(want) > want.size // 2
        for la, ta in _layouts(A).items():
            assert_same_bits(host(K.pam_matmul_fwd(ta, dev(B), True, True, 1.0)), want, f"k={k} {la}")
        assert_same_bits(host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0552)), ogemm(oracle, A, B, offset=1.0552), f"k={k} offset")
        # the same with the roles exchanged (tiny values mostly in the right operand)
        assert_same_bits(host(K.pam_matmul_fwd(dev(B.T.copy()), dev(A.T.copy()), True, True, 1.0)), ogemm(oracle, B.T.copy(), A.T.copy()), f"k={k} exchanged")


def test_bmm_tails_and_strides(K, oracle):
    # the reference's own bmm test shape (pam/test_pam.py:198-205): power-of-two weights => equals bmm
    rng = np.random.RandomState(6)
    X = (rng.randint(-128, 128, (11, 13, 15)) / 64.0).astype(np.float32)
    W = (2.0 ** rng.randint(-8, 8, (11, 15, 19))).astype(np.float32)
    got = host(K.pam_bmm_fwd(dev(X), dev(W), True, True, 1.0))
    assert_same_bits(got, np.matmul(X.astype(np.float64), W.astype(np.float64)).astype(np.float32), "pow2 bmm")
    # attention-shaped operands, K = 197 (prime) and 64, every layout
    Q, Kt = _rand((6, 197, 64), 7), _rand((6, 64, 197), 8)
    P, V = _rand((6, 197, 197), 9, zeros=0.1), _rand((6, 197, 64), 10)
    for L, R in ((Q, Kt), (P, V)):
        want = ogemm(oracle, L, R)
        for ll, tl in _layouts(L).items():
            for lr, tr in _layouts(R).items():
                assert_same_bits(host(K.pam_bmm_fwd(tl, tr, True, True, 1.0)), want, f"bmm {ll} x {lr}")
    D = _rand((6, 197, 64), 11)
    assert_same_bits(host(K.pam_bmm_bwd(dev(P), dev(V), dev(D), True, True, True, 1.0)),
                     ogemm(oracle, P, V, mode=oracle.MODE_BWD_DELTA_L, D=D), "bmm bwd")
    # fairseq-style strided batch: q = x.view(T, B*H, D).transpose(0, 1), batch stride < row stride
    T, BH, Dh = 32, 12, 16
    x = _rand((T, BH, Dh), 12); y = _rand((T, BH, Dh), 13)
    q = dev(x).transpose(0, 1); kt = dev(y).transpose(0, 1).transpose(1, 2)
    assert q.stride() == (Dh, BH * Dh, 1) and kt.stride() == (Dh, 1, BH * Dh)
    want = ogemm(oracle, np.swapaxes(x, 0, 1), np.swapaxes(np.swapaxes(y, 0, 1), 1, 2))
    assert_same_bits(host(K.pam_bmm_fwd(q, kt, True, False, 1.0)), want, "strided batch")
    # the ordinary-multiply products through the batched kernel instances (pam/cuda_kernels.cu:942): every layout,
    # the strided batch, and the autograd wrapper with BMM=True against torch.bmm on exactly representable products
    want = ogemm(oracle, Q, Kt, mode=oracle.MODE_STD)
    for ll, tl in _layouts(Q).items():
        for lr, tr in _layouts(Kt).items():
            assert_same_bits(host(K.standard_bmm(tl, tr, True, True, 1.0)), want, f"standard bmm {ll} x {lr}")
    want = ogemm(oracle, np.swapaxes(x, 0, 1), np.swapaxes(np.swapaxes(y, 0, 1), 1, 2), mode=oracle.MODE_STD)
    assert_same_bits(host(K.standard_bmm(q, kt, True, False, 1.0)), want, "standard bmm, strided batch")
    from pam_amd import cuda_bindings
    rng = np.random.RandomState(16)
    a = dev((rng.randint(-8, 9, (5, 33, 20)) / 4.0).astype(np.float32)).requires_grad_()
    b = dev((2.0 ** rng.randint(-3, 4, (5, 20, 17))).astype(np.float32)).requires_grad_()
    up = dev((2.0 ** rng.randint(-2, 3, (5, 33, 17))).astype(np.float32))
    out = cuda_bindings.standard_matmul(a, b, BMM=True)
    out.backward(up)
    a2, b2 = a.detach().clone().requires_grad_(), b.detach().clone().requires_grad_()
    ref = torch.bmm(a2, b2)
    ref.backward(up)
    assert torch.equal(out, ref) and torch.equal(a.grad, a2.grad) and torch.equal(b.grad, b2.grad)


def test_split_k_fixed_order(K, oracle):
    from pam_amd import _abi
    m, n, k = 96, 160, 8192
    chunk = _abi.gemm_plan(1, m, n, k)
    assert chunk % 16 == 0 and chunk < k, "this shape is expected to split k across work-groups"
    A, B = _rand((m, k), 14), _rand((k, n), 15)
    want = oracle.gemm(A, B, kchunk=chunk)
    assert_same_bits(host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0)), want, "split-K order")
    At = dev(np.ascontiguousarray(A.T)).T                      # the dW layout: column-major left operand
    assert_same_bits(host(K.pam_matmul_fwd(At, dev(B), False, True, 1.0)), want, "split-K, cm x rm")
    # the same call again and again finds the queue and arrival words as the call before left them
    for _ in range(3):
        assert_same_bits(host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0)), want, "repeated call")
    # the sequential order differs from the split order only by fp32 rounding of the sums
    seq = oracle.gemm(A, B)
    assert np.abs(seq - want).max() <= 1e-5 * np.abs(seq).max()


def test_matmul_config0_golden(K, oracle):
    from test_oracle_goldens import c0_operands
    g = np.load(GOLDEN / "matmul_c0.npz")
    A, B, dY = c0_operands()
    Y = host(K.pam_matmul_fwd(dev(A), dev(B), True, True, 1.0)); want = f32(g["y"]).reshape(256, 256)
    assert_same_bits(Y, ogemm(oracle, A, B), "config 0 forward vs oracle")
    assert np.abs(Y - want).max() / np.abs(want).max() <= 1e-5                  # vs native.pam_matmul
    dA = host(K.pam_matmul_fwd(dev(dY), dev(B).T, True, False, 1.0))
    dB = host(K.pam_matmul_fwd(dev(A).T, dev(dY), False, True, 1.0))
    assert np.abs(dA[::8] - f32(g["da_rows"]).reshape(32, 512)).max() / np.abs(f32(g["da_rows"])).max() <= 1e-5
    assert np.abs(dB[::8] - f32(g["db_rows"]).reshape(64, 256)).max() / np.abs(f32(g["db_rows"])).max() <= 1e-5


# ------------------------------------------------------------------ full-size configurations

def test_deit_linear_full_size(K, oracle):
    """12608 x 192 -> 768 forward and both backward products at full size: sampled rows
    against the oracle, and exact scale-invariance of the whole result."""
    rng = np.random.RandomState(100)
    X = rng.standard_normal((12608, 192)).astype(np.float32)
    W = np.clip(rng.standard_normal((768, 192)) * 0.02, -0.04, 0.04).astype(np.float32)
    dY = (rng.standard_normal((12608, 768)) * 1e-2).astype(np.float32)
    tX, tW, tdY = dev(X), dev(W), dev(dY)
    Y = K.pam_matmul_fwd(tX, tW.T, True, False, 1.0)
    dX = K.pam_matmul_fwd(tdY, tW, True, True, 1.0)
    dW = K.pam_matmul_fwd(tX.T, tdY, False, True, 1.0)
    rows = rng.choice(12608, 48, replace=False)
    assert_same_bits(host(Y)[rows], ogemm(oracle, X[rows], W.T, plan_shape=(1, 12608, 768, 192)), "Y rows")
    assert_same_bits(host(dX)[rows], ogemm(oracle, dY[rows], W, plan_shape=(1, 12608, 192, 768)), "dX rows")
    cols = rng.choice(768, 24, replace=False)
    assert_same_bits(host(dW)[:, cols], ogemm(oracle, X.T, dY[:, cols], plan_shape=(1, 192, 768, 12608)), "dW cols")
    # the second layer of the pair, 768 -> 192: row-major times column-major with k = 768 (k split across work-groups)
    X2 = rng.standard_normal((12608, 768)).astype(np.float32)
    W2 = np.clip(rng.standard_normal((192, 768)) * 0.02, -0.04, 0.04).astype(np.float32)
    Y2 = K.pam_matmul_fwd(dev(X2), dev(W2).T, True, False, 1.0)
    assert_same_bits(host(Y2)[rows], ogemm(oracle, X2[rows], W2.T, plan_shape=(1, 12608, 192, 768)), "Y rows, 768 -> 192")
    dY2 = (rng.standard_normal((12608, 192)) * 1e-2).astype(np.float32)
    dW2 = K.pam_matmul_fwd(dev(X2).T, dev(dY2), False, True, 1.0)
    cols2 = rng.choice(192, 16, replace=False)
    assert_same_bits(host(dW2)[:, cols2], ogemm(oracle, X2.T, dY2[:, cols2], plan_shape=(1, 768, 192, 12608)), "dW cols, 768 -> 192")
    # the same layer behind a ReLU (half of the left operand's values are zeros: k-tiles that skip the zero products),
    # then with 30 % of the weights pruned too (zeros in both operands)
    X2r = np.maximum(X2, 0.0).astype(np.float32)
    Y2r = K.pam_matmul_fwd(dev(X2r), dev(W2).T, True, False, 1.0)
    assert_same_bits(host(Y2r)[rows], ogemm(oracle, X2r[rows], W2.T, plan_shape=(1, 12608, 192, 768)), "Y rows, ReLU input")
    dW2r = K.pam_matmul_fwd(dev(X2r).T, dev(dY2), False, True, 1.0)
    assert_same_bits(host(dW2r)[:, cols2], ogemm(oracle, X2r.T, dY2[:, cols2], plan_shape=(1, 768, 192, 12608)), "dW cols, ReLU input")
    W2s = (W2 * (rng.rand(*W2.shape) >= 0.3)).astype(np.float32)
    Y2s = K.pam_matmul_fwd(dev(X2r), dev(W2s).T, True, False, 1.0)
    assert_same_bits(host(Y2s)[rows], ogemm(oracle, X2r[rows], W2s.T, plan_shape=(1, 12608, 192, 768)), "Y rows, ReLU input, pruned weight")
    # the input gradient of the 768 -> 192 layer: row-major times row-major with k = 192
    dX2 = K.pam_matmul_fwd(dev(dY2), dev(W2), True, True, 1.0)
    assert_same_bits(host(dX2)[rows], ogemm(oracle, dY2[rows], W2, plan_shape=(1, 12608, 768, 192)), "dX rows, 768 -> 192")
    # the exact gradients of the 192 -> 768 layer (the calls of pam/cuda_bindings.py:154-164), with and without an offset:
    # dX = bwd(dY, W, X, delta is the left operand), dW^T = bwd(X^T, dY, W^T, delta is the right operand)
    for off in OFFS:
        edX = K.pam_matmul_bwd(tdY, tW, tX, True, True, True, _o(off))
        assert_same_bits(host(edX)[rows], ogemm(oracle, dY[rows], W, plan_shape=(1, 12608, 192, 768), mode=oracle.MODE_BWD_DELTA_L,
                                                D=X[rows], offset=off), f"exact dX rows off={off}")
        edW = K.pam_matmul_bwd(tX.T, tdY, tW.T, False, True, False, _o(off))
        assert_same_bits(host(edW)[:, cols], ogemm(oracle, X.T, dY[:, cols], plan_shape=(1, 192, 768, 12608), mode=oracle.MODE_BWD_DELTA_R,
                                                   D=np.ascontiguousarray(W.T[:, cols]), offset=off), f"exact dW cols off={off}")
    # multiplying an operand by a power of two multiplies every PAM product, hence the sum, exactly
    assert torch.equal(K.pam_matmul_fwd(tX * 4.0, tW.T, True, False, 1.0), Y * 4.0)
    assert torch.equal(K.pam_matmul_fwd(tX, (tW * 0.5).T, True, False, 1.0), Y * 0.5)
    # a row permutation of X permutes the rows of Y
    perm = torch.randperm(12608, device="cuda")
    assert torch.equal(K.pam_matmul_fwd(tX[perm], tW.T, True, False, 1.0), Y[perm])


def test_attention_bmm_full_size(K, oracle):
    """Batched attention products at full size (batch 64 x 3 heads, 197 tokens, head dim 64): Q K^T and
    P V forward plus the approximate backward products on transposed views, sampled batches
    against the oracle; K = 197 (prime) and 64 exercise the k tail and the row tails."""
    g = torch.Generator().manual_seed(300)
    B, T, D = 192, 197, 64
    Q, Kk, V = (torch.randn(B, T, D, generator=g) for _ in range(3))
    P = torch.softmax(torch.randn(B, T, T, generator=g), dim=-1)
    dS, dO = torch.randn(B, T, T, generator=g), torch.randn(B, T, D, generator=g)
    q, k, v, p, ds, do = (t.cuda() for t in (Q, Kk, V, P, dS, dO))
    kt = k.transpose(1, 2)
    S = K.pam_bmm_fwd(q, kt, True, False, 1.0)                   # [B, T, T], K = 64
    O = K.pam_bmm_fwd(p, v, True, True, 1.0)                     # [B, T, D], K = 197
    dQ = K.pam_bmm_fwd(ds, kt.mT, True, True, 1.0)               # dS K
    dKt = K.pam_bmm_fwd(q.mT, ds, False, True, 1.0)              # Q^T dS
    dP = K.pam_bmm_fwd(do, v.mT, True, False, 1.0)               # dO V^T
    dV = K.pam_bmm_fwd(p.mT, do, False, True, 1.0)               # P^T dO
    pick = [0, 77, 191]
    n = lambda t: t[pick].numpy()
    tr = lambda a: np.swapaxes(a, 1, 2)
    cases = [("S", S, n(Q), tr(n(Kk)), (B, T, T, D)), ("O", O, n(P), n(V), (B, T, D, T)),
             ("dQ", dQ, n(dS), n(Kk), (B, T, D, T)), ("dKt", dKt, tr(n(Q)), n(dS), (B, D, T, T)),
             ("dP", dP, n(dO), tr(n(V)), (B, T, T, D)), ("dV", dV, tr(n(P)), n(dO), (B, T, D, T))]
    for name, got, L, R, shape in cases:
        assert_same_bits(host(got)[pick], ogemm(oracle, L, R, plan_shape=shape), name)
    # the autograd layer produces the same six tensors
    import pam_amd as pam
    q2, k2, v2, p2 = (t.clone().requires_grad_() for t in (q, k, v, p))
    s2 = pam.bmm(q2, k2.transpose(1, 2), approx_bwd=True); s2.backward(ds)
    o2 = pam.bmm(p2, v2, approx_bwd=True); o2.backward(do)
    assert torch.equal(s2, S) and torch.equal(o2, O) and torch.equal(q2.grad, dQ) and torch.equal(p2.grad, dP)
    assert torch.equal(k2.grad, dKt.transpose(1, 2)) and torch.equal(v2.grad, dV)


def test_elementwise_full_size(K, oracle):
    """2^26 elements, 98 % N(0,1) and 2 % edge values: slices against the oracle, and the
    round trip (a (*) b) (/) b == a wherever nothing saturates."""
    n = 1 << 26
    a, b = mixed_operands(n, 10), mixed_operands(n, 11)
    ta, tb = dev(a), dev(b)
    prod = K.pam_fwd(ta, tb, 1.0); quot = K.pad_fwd(ta, tb, 1.0)
    hp, hq = host(prod), host(quot)
    for lo in (0, 12345677, n - (1 << 20)):
        sl = slice(lo, lo + (1 << 20))
        assert_same_bits(hp[sl], oracle.pam(a[sl], b[sl]), f"pam slice {lo}")
        assert_same_bits(hq[sl], oracle.pad(a[sl], b[sl]), f"pad slice {lo}")
    back = host(K.pad_fwd(prod, tb, 1.0))
    ea = (a.view(np.uint32) >> 23) & 0xff; eb = (b.view(np.uint32) >> 23) & 0xff
    safe = (ea > 40) & (ea < 210) & (eb > 40) & (eb < 210)
    assert safe.mean() > 0.95 and (back[safe].view(np.uint32) == a[safe].view(np.uint32)).all()
    # checksum of the whole array against the oracle on all host cores
    want = oracle.pam(a, b)
    assert np.bitwise_xor.reduce(hp.view(np.uint32)[~np.isnan(hp)]) == np.bitwise_xor.reduce(want.view(np.uint32)[~np.isnan(want)])
    assert (np.isnan(hp) == np.isnan(want)).all()


# ------------------------------------------------------------------ autograd layer on the device

def test_linear_autograd_matches_oracle(K, oracle):
    import pam_amd as pam
    rng = np.random.RandomState(200)
    X = rng.standard_normal((4, 50, 96)).astype(np.float32); W = (rng.standard_normal((40, 96)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(40).astype(np.float32); dY = rng.standard_normal((4, 50, 40)).astype(np.float32)
    for approx in (True, False):
        lin = pam.Linear(96, 40, approx_bwd=approx).cuda()
        with torch.no_grad():
            lin.weight.copy_(dev(W)); lin.bias.copy_(dev(bias))
        x = dev(X).requires_grad_()
        y = lin(x); y.backward(dev(dY))
        X2, dY2 = X.reshape(200, 96), dY.reshape(200, 40)
        assert_same_bits(host(y).reshape(200, 40), ogemm(oracle, X2, W.T) + bias, "linear forward")
        if approx:
            assert_same_bits(host(x.grad).reshape(200, 96), ogemm(oracle, dY2, W), "dX approx")
            assert_same_bits(host(lin.weight.grad), ogemm(oracle, X2.T, dY2).T, "dW approx")
        else:
            assert_same_bits(host(x.grad).reshape(200, 96), ogemm(oracle, dY2, W, mode=oracle.MODE_BWD_DELTA_L, D=X2), "dX exact")
            assert_same_bits(host(lin.weight.grad), ogemm(oracle, X2.T, dY2, mode=oracle.MODE_BWD_DELTA_R, D=W.T).T, "dW exact")


def test_reference_vectors_on_device(K):
    # pam/test_pam.py:13-45 run against the HIP path, with the reference's comparators
    import pam_amd as pam
    abc = torch.tensor([
        [1.0, 1.0, 1.0], [1.2345, 1.0, 1.2345], [1.2345, 32.0, 32.0 * 1.2345], [-1.2345, 32.0, -32.0 * 1.2345],
        [1.2345, -32.0, -32.0 * 1.2345], [-1.2345, -32.0, 32.0 * 1.2345], [1.0, 0.0, 0.0], [0.0, -1.0, -0.0],
        [1.5, 1.5, 2.0], [1.3, -1.3, -1.6], [4.5, 3.0, 8 * (1 + (4.5 - 4) / 4 + (3.0 - 2) / 2)], [-6.0, 3.0, -16.0],
        [-3.5, -3.5, 8 * (1 + (3.5 - 2) / 2 + (3.5 - 2) / 2 - 1)], [1e-30, 1e-30, 0.0], [1e-30, -1e-30, -0.0]], device="cuda")
    assert torch.allclose(abc[:, 2], pam.mul(abc[:, 0].contiguous(), abc[:, 1].contiguous()))
    ab = torch.tensor([[1e30, 1e30], [1e30, -1e30], [float("-inf"), 1e-20], [float("nan"), -1e-20],
                       [float("inf"), 0.0], [float("nan"), 0.0]], device="cuda")
    assert (~pam.mul(ab[:, 0].contiguous(), ab[:, 1].contiguous()).isfinite()).all()
    # pam/test_pam.py:127-148: approximate backward equals the two transposed products
    A = (torch.arange(20) ** 3 % 7 - 2.0).reshape((5, 4)).cuda().requires_grad_()
    B = (torch.arange(12) ** 2 % 5 - 2.0).reshape((3, 4)).T.cuda().requires_grad_()
    C = pam.matmul(A, B, approx_bwd=True)
    delta = torch.arange(C.numel()).float().reshape_as(C).cuda()
    C.backward(delta)
    assert torch.equal(A.grad, pam.matmul(delta, B.detach().T)) and torch.equal(B.grad, pam.matmul(A.detach().T, delta))
    g = np.load(GOLDEN / "matmul_small.npz")
    assert_same_bits(host(C), f32(g["p20_c"]).reshape(5, 3), "reference 5x4 @ 4x3 forward")
    assert np.allclose(host(A.grad), f32(g["p20_da_approx"]).reshape(5, 4)) and np.allclose(host(B.grad), f32(g["p20_db_approx"]).reshape(4, 3))


@pytest.mark.gpu
def test_linear_with_bias_in_the_epilogue(oracle):
    """pam.linear with a bias: added inside the product kernel (after the chunk sums when k is split),
    bit-identical to the product followed by a separate add; gradients as without the fusion."""
    import pam_amd
    from pam_amd import pam_ops, _abi
    rng = np.random.RandomState(11)
    for (m, k, n) in [(197, 192, 768), (50, 1000, 24), (7, 5, 3), (3000, 4096, 64)]:
        X = rng.standard_normal((m, k)).astype(np.float32); W = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32); dY = rng.standard_normal((m, n)).astype(np.float32)
        want = (ogemm(oracle, X, W.T) + b).astype(np.float32)
        res = {}
        for fused_on in (True, False):
            pam_ops.fused_bias = fused_on
            try:
                x = torch.from_numpy(X).cuda().requires_grad_(); w = torch.from_numpy(W).cuda().requires_grad_()
                bb = torch.from_numpy(b).cuda().requires_grad_()
                y = pam_amd.linear(x, w, bb, approx_bwd=True, offset=None)
                y.backward(torch.from_numpy(dY).cuda())
                res[fused_on] = [t.detach().cpu().numpy() for t in (y, x.grad, w.grad, bb.grad)]
            finally:
                pam_ops.fused_bias = True
        assert_same_bits(res[True][0], want, f"linear+bias {m}x{k}x{n}")
        for a, c, name in zip(res[True], res[False], ("y", "dX", "dW", "db")):
            assert_same_bits(a, c, f"{name} fused vs separate add, {m}x{k}x{n}")
    # leading dimensions and the module
    lin = pam_amd.Linear(192, 96, approx_bwd=True).cuda()
    x3 = torch.randn(4, 197, 192, device="cuda")
    pam_ops.fused_bias = False
    ref = lin(x3)
    pam_ops.fused_bias = True
    assert torch.equal(lin(x3), ref) and lin(x3).shape == (4, 197, 96)


@pytest.mark.parametrize("off", OFFS)
@pytest.mark.parametrize("p", [0.5, 2.0, -1.5, 3])
def test_pow_with_a_number_in_one_pass(K, oracle, p, off):
    """pam.pow(A, number): one kernel against the reference's chain (pam/pam_ops.py:70-79) built from
    the oracle's primitives, and against the same chain of kernels on the GPU -- values and the
    gradient autograd chains through select, exp2, product and log2, bit for bit."""
    import pam_amd
    from pam_amd import pam_ops
    rng = np.random.RandomState(17)
    a = np.abs(rng.standard_normal(5003)).astype(np.float32) * 3 + 0.01
    a[rng.choice(a.size, 40, replace=False)] = np.resize(np.array([0.0, -0.0, 1e-30, 1e30, 1.0, 2.0 ** -126, 1e-40, np.inf], np.float32), 40)
    g = rng.standard_normal(a.shape).astype(np.float32)
    l = oracle.pa_log(a, 2.0, off)
    want = np.where(a == 0, np.float32(0), oracle.pa_exp(oracle.pam(l, np.float32(p), off), 2.0, off)).astype(np.float32)
    res = {}
    for fused_on in (True, False):
        pam_ops.fused_pow = fused_on
        try:
            for approx in (False, True, (True, False), (False, True)):
                at = dev(a).requires_grad_()
                y = pam_amd.pow(at, p, offset=off, approx_bwd=approx)
                y.backward(dev(g))
                res[fused_on, approx] = (host(y.detach()), host(at.grad))
        finally:
            pam_ops.fused_pow = True
    for approx in (False, True, (True, False), (False, True)):
        assert_same_bits(res[True, approx][0], want, f"pow {p} forward")
        assert_same_bits(res[True, approx][0], res[False, approx][0], f"pow {p}: one pass against the chain")
        assert_same_bits(res[True, approx][1], res[False, approx][1], f"pow {p} gradient, approx={approx}: one pass against the chain")
    # the exact gradient from the oracle's primitives
    t = oracle.pam(l, np.float32(p), off)
    gy = np.where(a == 0, np.float32(0), g).astype(np.float32)
    gt = oracle.pa_exp_bwd(t, gy, 2.0, off)
    gl = oracle.pam_bwd(l, np.full_like(l, p), gt, off)
    assert_same_bits(res[True, False][1], oracle.pa_log_bwd(a, gl, 2.0, off), f"pow {p} exact gradient")


@pytest.mark.parametrize("off", OFFS)
def test_both_gradients_in_one_pass(K, oracle, off):
    """(dA, dB) of a product / quotient from one kernel against the oracle's formulas
    (pam/cuda_bindings.py:43-57, 78-97) and, through autograd, against the one-launch-per-gradient path."""
    import pam_amd
    from pam_amd import cuda_bindings
    n = 10007
    a, b, d = _rand((n,), 51, 0.01, True), _rand((n,), 52, 0.01, True), _rand((n,), 53, 0.01, True)
    o = _o(off)
    inv = oracle.pad(np.ones_like(b), b, off)
    want = {
        ("pam", True): (oracle.pam(d, b, off), oracle.pam(d, a, off)),
        ("pam", False): (oracle.pam_bwd(a, b, d, off), oracle.pam_bwd(b, a, d, off)),
        ("pad", True): (oracle.pam(inv, d, off), -oracle.pam(oracle.pad(oracle.pad(a, b, off), b, off), d, off)),
        ("pad", False): (oracle.pam_bwd(a, inv, d, None), oracle.pad_bwd(a, b, d, off)),
    }
    for op in ("pam", "pad"):
        for approx_a in (True, False):
            for approx_b in (True, False):
                da, db = getattr(K, f"{op}_bwd_pair")(dev(a), dev(b), dev(d), o, approx_a, approx_b)
                assert_same_bits(host(da), want[op, approx_a][0], f"{op} dA approx={approx_a}")
                assert_same_bits(host(db), want[op, approx_b][1], f"{op} dB approx={approx_b}")
    # through autograd: paired against single launches, unaligned views included
    for fn in (pam_amd.mul, pam_amd.div):
        res = {}
        for paired in (True, False):
            cuda_bindings.paired_gradients = paired
            try:
                at, bt = dev(a)[1:].requires_grad_(), dev(b)[1:].requires_grad_()
                fn(at, bt, offset=off, approx_bwd=(True, False)).backward(dev(d)[1:])
                res[paired] = (host(at.grad), host(bt.grad))
            finally:
                cuda_bindings.paired_gradients = True
        assert_same_bits(res[True][0], res[False][0], "dA paired against single")
        assert_same_bits(res[True][1], res[False][1], "dB paired against single")


def test_degenerate_shapes(K, oracle):
    """Empty operands and a zero-length inner dimension: no launch faults, outputs of the right shape, and a
    sum over nothing is +0 (the accumulators start there); empty rows for the row-wise kernels."""
    import pam_amd
    from pam_amd import _abi
    z = lambda *s: torch.zeros(*s, device="cuda")
    assert K.pam_matmul_fwd(z(0, 8), z(8, 5), True, True, 1.0).shape == (0, 5)
    assert K.pam_matmul_fwd(z(7, 8), z(8, 0), True, True, 1.0).shape == (7, 0)
    y = K.pam_matmul_fwd(torch.full((7, 0), 3.0, device="cuda"), z(0, 5), True, True, 1.0)
    assert y.shape == (7, 5) and (host(y).view(np.uint32) == 0).all()
    y = K.pam_bmm_fwd(z(3, 4, 0), z(3, 0, 6), True, True, 1.0)
    assert y.shape == (3, 4, 6) and (host(y).view(np.uint32) == 0).all()
    assert K.pam_bmm_fwd(z(0, 4, 5), z(0, 5, 6), True, True, 1.0).shape == (0, 4, 6)
    assert K.pam_matmul_bwd(z(7, 0), z(0, 5), z(7, 5), True, True, True, 1.0).shape == (7, 5)
    R = _abi.HipRowKernels()
    ys, rs, sh = R.softmax_fwd(z(0, 16), 1.0)
    assert ys.shape == (0, 16) and rs.shape == (0,)
    assert R.row_mean_fwd(z(0, 16), 1.0).shape == (0,)
    with pytest.raises(RuntimeError):                    # as in the reference: the global maximum of nothing (pam/pam_ops.py:318)
        pam_amd.softmax(z(4, 0), dim=-1)
    assert _abi.conv2d_fwd(z(0, 3, 8, 8), z(4, 3, 3, 3), (1, 1), (1, 1), 1.0).shape == (0, 4, 8, 8)
    assert K.pam_fwd(z(0), z(0), 1.0).shape == (0,)


def test_more_than_two_to_the_31_elements(K, oracle):
    """64-bit indexing: an elementwise product over 2^31 + 5 elements, a row kernel over 2^31 elements and a product
    with more than 2^31 output elements, checked on slices from both ends."""
    from pam_amd import _abi
    n = (1 << 31) + 5
    gen = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randn(n, device="cuda", generator=gen); b = torch.randn(n, device="cuda", generator=gen)
    c = K.pam_fwd(a, b, 1.0)
    for lo, hi in ((0, 4096), (n - 4101, n)):
        assert_same_bits(host(c[lo:hi]), oracle.pam(host(a[lo:hi]), host(b[lo:hi])), f"elementwise [{lo}:{hi}]")
    del c, b
    rows = a[:1 << 31].view(1 << 21, 1024)
    R = _abi.HipRowKernels()
    y = R.layer_norm_fwd(rows, None, None, 1e-5, 1.0)
    for lo, hi in ((0, 3), ((1 << 21) - 3, 1 << 21)):
        assert_same_bits(host(y[lo:hi]), oracle.layer_norm_fwd(host(rows[lo:hi]), None, None, 1e-5, None), f"layer_norm rows [{lo}:{hi}]")
    del y
    m = (1 << 25) + 64                                  # m x 64 outputs > 2^31
    L = a[:m * 16].view(m, 16); Rm = torch.randn(16, 64, device="cuda", generator=gen)
    Y = K.pam_matmul_fwd(L, Rm, True, True, 1.0)
    for lo, hi in ((0, 70), (m - 70, m)):
        assert_same_bits(host(Y[lo:hi]), ogemm(oracle, host(L[lo:hi]), host(Rm), plan_shape=(1, m, 64, 16)), f"product rows [{lo}:{hi}]")
