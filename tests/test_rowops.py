"""Single-kernel softmax / logsumexp / log_softmax / mean / layer_norm.

CPU: the oracle's fused restatements are pinned against the chain of primitive calls the
reference makes (pam/pam_ops.py:288-378), written out here from the already pinned oracle
primitives with the kernels' row-sum order restated in numpy: bit for bit.  The softmax
gradient is pinned twice: against the primitives' backward formulas chained by hand, and
against torch autograd running the unfused composition over the oracle-backed kernel object
(there the row sums are torch's, so the comparison is to summation-order noise).
GPU: the HIP kernels against the oracle's fused restatements, bit for bit.
"""
import math

import numpy as np
import pytest
import torch

import pam_amd
from pam_amd import composites, cuda_bindings, pam_ops
from _util import assert_same_bits, same_bits
from test_host_api import OracleKernels

C = np.float32(math.log2(math.e))
LN2 = np.float32(math.log(2.0))
OFF = 1.0552


def fixed_sum(v):
    """Row sums in the kernels' order: 64 strided partial sums from +0, then a butterfly.  Rows of
    4097 ... 16384 values: 1024 strided partial sums, the butterfly within each group of 64, then the
    16 group sums in ascending order."""
    v = np.asarray(v, dtype=np.float32)
    rows, n = v.shape
    if 4096 < n <= 16384:
        pad = (-n) % 1024
        if pad:
            v = np.concatenate([v, np.zeros((rows, pad), np.float32)], axis=1)
        p = np.zeros((rows, 1024), np.float32)
        for j in range(v.shape[1] // 1024):
            p = (p + v[:, 1024 * j:1024 * j + 1024]).astype(np.float32)
        p = p.reshape(rows, 16, 64)
        lanes = np.arange(64)
        for s in (32, 16, 8, 4, 2, 1):
            p = (p + p[:, :, lanes ^ s]).astype(np.float32)
        total = p[:, 0, 0]
        for w in range(1, 16):
            total = (total + p[:, w, 0]).astype(np.float32)
        return total
    pad = (-n) % 64
    if pad:
        v = np.concatenate([v, np.zeros((rows, pad), np.float32)], axis=1)     # adding +0 changes nothing
    p = np.zeros((rows, 64), np.float32)
    for j in range(v.shape[1] // 64):
        p = (p + v[:, 64 * j:64 * j + 64]).astype(np.float32)
    lanes = np.arange(64)
    for s in (32, 16, 8, 4, 2, 1):
        p = (p + p[:, lanes ^ s]).astype(np.float32)
    return p[:, 0]


def rows_case(seed, rows, n, scale=3.0, masks=True):
    rng = np.random.RandomState(seed)
    x = (rng.standard_normal((rows, n)) * scale).astype(np.float32)
    if masks and n > 2:
        x[rng.randint(rows), rng.randint(n)] = -np.inf
        x[rng.randint(rows), : n // 2] = -np.inf
    return x


# ------------------------------------------------------------------ the reference's chains, from oracle primitives
def softmax_chain(o, x, off):
    neg = np.isneginf(x)
    s = np.where(neg, -np.inf, o.pam(x, C, off)).astype(np.float32)
    shift = np.floor(s.max())
    t = (s - shift).astype(np.float32)
    e = np.where(neg, 0, o.pa_exp(t, 2.0, off)).astype(np.float32)
    total = fixed_sum(e)[:, None]
    return o.pad(e, total, off), dict(neg=neg, t=t, e=e, total=total, shift=shift)


def softmax_grad_chain(o, x, g, off, approx):
    """pad -> sum -> where -> exp2 -> subtract -> where -> mul, each with the backward formula of
    its autograd Function (pam/cuda_bindings.py:43-57, 78-97, 224-239)."""
    approx_a, approx_b, approx_e = approx
    _, f = softmax_chain(o, x, off)
    neg, t, e, total = f["neg"], f["t"], f["e"], np.broadcast_to(f["total"], x.shape)
    inv = o.pad(np.ones_like(total), total, off)
    d_e = o.pam(inv, g, off) if approx_a else o.pam_bwd(e, inv, g, None)
    if approx_b:
        d_total_full = (-o.pam(o.pad(o.pad(e, total, off), total, off), g, off)).astype(np.float32)
    else:
        d_total_full = o.pad_bwd(e, total, g, off)
    d_total = fixed_sum(d_total_full)[:, None]
    d_e = np.where(neg, 0, (d_e + d_total).astype(np.float32)).astype(np.float32)
    if approx_e:
        d_t = o.pam(o.pam(o.pa_exp(t, 2.0, off), LN2, off), d_e, off)
    else:
        d_t = o.pa_exp_bwd(t, d_e, 2.0, off)
    d_s = np.where(neg, 0, d_t).astype(np.float32)
    return o.pam(d_s, C, off) if approx_a else o.pam_bwd(x, C, d_s, off)


def logsumexp_chain(o, x, off):
    """pam/pam_ops.py:333-342: the offset goes to mul, exp2 and div; log2 of the row total is called bare."""
    s = o.pam(x, C, off)
    shift = np.floor(s.max())
    e = o.pa_exp((s - shift).astype(np.float32), 2.0, off)
    total = fixed_sum(e)
    return o.pad((shift + o.pa_log(total, 2.0, None)).astype(np.float32), C, off)


def logsumexp_grad_chain(o, x, g_out, off, approx):
    """Autograd's walk back through pam/pam_ops.py:333-342 with the backward formula of each Function
    (pam/cuda_bindings.py:43-57, 78-97, 224-239, 262-276): div -> add -> log2 -> sum -> exp2 -> subtract -> mul.
    log2 was called without keyword arguments, so its gradient is pa_log_bwd without an offset, always."""
    approx_a, _, approx_e = approx
    s = o.pam(x, C, off)
    shift = np.floor(s.max())
    t = (s - shift).astype(np.float32)
    e = o.pa_exp(t, 2.0, off)
    total = fixed_sum(e)
    u = (shift + o.pa_log(total, 2.0, None)).astype(np.float32)
    inv = o.pad(np.ones_like(u), np.full_like(u, C), off)
    d_u = o.pam(inv, g_out, off) if approx_a else o.pam_bwd(u, inv, g_out, None)
    d_total = o.pa_log_bwd(total, d_u, 2.0, None)
    d_e = np.broadcast_to(d_total[:, None], x.shape).astype(np.float32)
    if approx_e:
        d_t = o.pam(o.pam(o.pa_exp(t, 2.0, off), LN2, off), d_e, off)
    else:
        d_t = o.pa_exp_bwd(t, d_e, 2.0, off)
    return o.pam(d_t, C, off) if approx_a else o.pam_bwd(x, np.full_like(x, C), d_t, off)


def layer_norm_chain(o, x, w, b, eps, off):
    n = np.float32(x.shape[1])
    mu = o.pad(fixed_sum(x)[:, None], n, off)
    cen = (x - mu).astype(np.float32)
    var = o.pad(fixed_sum(o.pam(cen, cen, off))[:, None], n, off)
    v = (var + np.float32(eps)).astype(np.float32)
    root = np.where(v == 0, 0, o.pa_exp(o.pam(o.pa_log(v, 2.0, off), np.float32(0.5), off), 2.0, off)).astype(np.float32)
    out = o.pad(cen, root, off)
    if w is not None:
        out = o.pam(out, w, off)
    if b is not None:
        out = (out + b).astype(np.float32)
    return out


# ------------------------------------------------------------------ CPU: oracle fused == chain
@pytest.mark.parametrize("off", [None, OFF])
@pytest.mark.parametrize("rows,n", [(1, 1), (3, 5), (4, 63), (4, 64), (5, 65), (6, 197), (2, 1000)])
def test_oracle_softmax_is_the_chain(oracle, rows, n, off):
    x = rows_case(rows * 1000 + n, rows, n)
    y, row_sum, shift = oracle.softmax_fwd(x, off)
    want, f = softmax_chain(oracle, x, off)
    assert_same_bits(y, want, "softmax")
    assert_same_bits(row_sum, f["total"][:, 0], "row sums")
    assert_same_bits(shift, f["shift"], "shift")
    g = np.random.RandomState(7).standard_normal(x.shape).astype(np.float32)
    for approx in [(False, False, False), (True, True, True), (True, False, True), (False, True, True)]:
        got = oracle.softmax_bwd(x, g, row_sum, shift, off, approx)
        assert_same_bits(got, softmax_grad_chain(oracle, x, g, off, approx), f"softmax gradient approx={approx}")


def test_oracle_softmax_special_rows(oracle):
    x = rows_case(3, 6, 40, masks=False)
    x[0, :] = -np.inf                       # fully masked row: 0 (/) 0
    x[1, 3] = np.nan
    y, _, _ = oracle.softmax_fwd(x)
    assert np.isnan(y).all()                # the NaN reaches the global shift, as in the reference's chain
    x[1, 3] = 0.5
    y, row_sum, _ = oracle.softmax_fwd(x)
    assert np.isnan(y[0]).all() and row_sum[0] == 0 and np.isfinite(y[1:]).all()
    assert_same_bits(y, softmax_chain(oracle, x, None)[0], "masked row")
    assert np.abs(y[1:].sum(-1) - 1).max() < 0.1


@pytest.mark.parametrize("off", [None, OFF])
def test_oracle_logsumexp_mean_layer_norm_are_the_chains(oracle, off):
    for rows, n in [(1, 1), (3, 7), (4, 64), (5, 192), (2, 513), (2, 4097), (2, 9000)]:
        x = rows_case(rows * 77 + n, rows, n, masks=False)
        want = logsumexp_chain(oracle, x, off)
        lse, ls = oracle.logsumexp_fwd(x, off, with_log_softmax=True)
        assert_same_bits(lse, want, "logsumexp")
        assert_same_bits(ls, (x - want[:, None]).astype(np.float32), "log_softmax")
        assert_same_bits(oracle.row_mean_fwd(x, off), oracle.pad(fixed_sum(x), np.float32(n), off), "mean")
        rng = np.random.RandomState(n)
        w, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
        for ww, bb in [(None, None), (w, None), (w, b)]:
            assert_same_bits(oracle.layer_norm_fwd(x, ww, bb, 1e-5, off), layer_norm_chain(oracle, x, ww, bb, 1e-5, off),
                             "layer_norm")
    const = np.full((2, 8), 3.0, np.float32)              # zero variance: the power's zero branch is not taken (eps)
    assert np.isfinite(oracle.layer_norm_fwd(const)).all()
    assert_same_bits(oracle.layer_norm_fwd(const, eps=0.0), np.full((2, 8), np.nan, np.float32), "0 (/) 0")


def test_fixed_order_sum_is_exact_where_sums_are(oracle):
    """Rows whose sums are exact in fp32 give the same result in any order: ties the fixed
    order to torch's on such rows."""
    rng = np.random.RandomState(5)
    x = (rng.randint(-64, 64, size=(6, 300)) / 8.0).astype(np.float32)
    assert_same_bits(fixed_sum(x), x.sum(-1, dtype=np.float64).astype(np.float32), "exact sums")
    assert_same_bits(oracle.row_mean_fwd(x), oracle.pad(x.sum(-1, dtype=np.float64).astype(np.float32), np.float32(300)), "mean")


@pytest.fixture()
def on_cpu(oracle, monkeypatch):
    monkeypatch.setattr(cuda_bindings, "cuda_kernels", OracleKernels(oracle))
    monkeypatch.setattr(pam_ops, "_require_kernel", lambda t, use_kernel: None)
    return oracle


@pytest.mark.parametrize("approx", [False, True, (True, False)])
def test_softmax_gradient_chain_is_what_autograd_does(on_cpu, approx):
    """torch autograd over the unfused composition (oracle-backed kernels, CPU) against the
    fused restatement: same formulas, torch's summation order instead of the fixed one."""
    o = on_cpu
    x = rows_case(11, 7, 33)
    g = np.random.RandomState(12).standard_normal(x.shape).astype(np.float32)
    for off in (None, OFF):
        xt = torch.from_numpy(x.copy()).requires_grad_()
        y = composites.softmax(xt, dim=-1, offset=off, approx_bwd=approx)
        y.backward(torch.from_numpy(g))
        flags = (approx, approx, approx) if isinstance(approx, bool) else (approx[0], approx[1], True)
        yo, row_sum, shift = o.softmax_fwd(x, off)
        got = o.softmax_bwd(x, g, row_sum, shift, off, flags)
        want = xt.grad.numpy()
        assert np.allclose(yo, y.detach().numpy(), rtol=2e-6, atol=1e-7)
        scale = np.abs(want).max()
        assert np.isfinite(want).all() and np.abs(got - want).max() <= 5e-6 * scale, (np.abs(got - want).max(), scale)
        assert (got[np.isneginf(x)] == 0).all()


def _flags(approx):
    return (approx, approx, approx) if isinstance(approx, bool) else (approx[0], approx[1], True)


@pytest.mark.parametrize("approx", [False, True, (True, False), (False, True)])
def test_logsumexp_and_layer_norm_gradient_chains_are_what_autograd_does(on_cpu, approx):
    """The oracle's gradient restatements against torch autograd over the unfused compositions
    (oracle-backed kernel object, CPU): same formulas, torch's summation order."""
    o = on_cpu
    x = rows_case(31, 6, 40, masks=False)
    rng = np.random.RandomState(32)
    g_rows = rng.standard_normal(6).astype(np.float32); g_full = rng.standard_normal(x.shape).astype(np.float32)
    w = (rng.standard_normal(40) + 2).astype(np.float32); b = rng.standard_normal(40).astype(np.float32)

    def close(got, want, tol=1e-5):
        scale = np.abs(want).max()
        assert np.isfinite(want).all() and np.abs(got - want).max() <= tol * scale, (np.abs(got - want).max(), scale)

    for off in (None, OFF):
        shift = np.floor(o.pam(x, C, off).max())
        xt = torch.from_numpy(x.copy()).requires_grad_()
        composites.logsumexp(xt, dim=-1, offset=off, approx_bwd=approx).backward(torch.from_numpy(g_rows))
        close(o.logsumexp_bwd(x, g_rows, shift, off, _flags(approx)), xt.grad.numpy())
        xt = torch.from_numpy(x.copy()).requires_grad_()
        composites.log_softmax(xt, dim=-1, offset=off, approx_bwd=approx).backward(torch.from_numpy(g_full))
        close(o.logsumexp_bwd(x, g_full, shift, off, _flags(approx), log_softmax=True), xt.grad.numpy())
        for ww, bb in [(None, None), (w, b)]:
            xt = torch.from_numpy(x.copy()).requires_grad_()
            wt = None if ww is None else torch.from_numpy(ww.copy()).requires_grad_()
            bt = None if bb is None else torch.from_numpy(bb.copy()).requires_grad_()
            composites.layer_norm(xt, 40, wt, bt, offset=off, approx_bwd=approx).backward(torch.from_numpy(g_full))
            dx, terms = o.layer_norm_bwd(x, ww, g_full, 1e-5, off, _flags(approx))
            close(dx, xt.grad.numpy(), 2e-5)
            if ww is not None:
                close(terms.sum(0), wt.grad.numpy())
                close(g_full.sum(0), bt.grad.numpy())


def reference_text_logsumexp(x, dim, keepdim=False, **pam_kwargs):
    """The reference's logsumexp as its source reads (pam/pam_ops.py:333-342), on the op library's primitives: the
    keyword arguments (offset, approx_bwd) go to the product, to exp2 and to the quotient -- the log2 of the summed
    weights gets none of them (:341).  Independent of `composites.logsumexp` on purpose."""
    k = math.log2(math.e)
    scaled = pam_ops.mul(x, k, **pam_kwargs)
    with torch.no_grad():
        shift = torch.floor(torch.max(scaled))
    weights = pam_ops.exp2(scaled - shift, **pam_kwargs)
    total = torch.sum(weights, dim=dim, keepdim=keepdim)
    bare_log2 = pam_ops.log2(total)                       # no offset, exact gradient
    return pam_ops.div(shift + bare_log2, k, **pam_kwargs)


@pytest.mark.parametrize("approx", [False, True, (True, False), (False, True)])
@pytest.mark.parametrize("off", [None, OFF])
def test_logsumexp_is_the_chain_the_reference_text_writes(on_cpu, off, approx):
    """Values and gradients of logsumexp / log_softmax in three restatements -- the unfused composition of this
    package, the oracle's fused restatement (what the HIP row kernels are compared with) and the primitives' backward
    formulas chained by hand -- against the chain as the reference's source text has it.  A restatement that hands the
    offset or approx_bwd to the inner log2 differs by percents (forward with an offset, gradient with approx_bwd) and fails."""
    o = on_cpu
    x = rows_case(31, 6, 40, masks=False)
    rng = np.random.RandomState(32)
    g_rows = rng.standard_normal(6).astype(np.float32); g_full = rng.standard_normal(x.shape).astype(np.float32)

    def close(got, want, what, tol=1e-5):
        scale = np.abs(want).max()
        assert np.isfinite(want).all() and np.abs(got - want).max() <= tol * scale, (what, np.abs(got - want).max(), scale)

    xt = torch.from_numpy(x.copy()).requires_grad_()
    ref = reference_text_logsumexp(xt, -1, offset=off, approx_bwd=approx)
    ref.backward(torch.from_numpy(g_rows))
    ref_val, ref_grad = ref.detach().numpy(), xt.grad.numpy().copy()
    xt = torch.from_numpy(x.copy()).requires_grad_()
    (xt - reference_text_logsumexp(xt, -1, keepdim=True, offset=off, approx_bwd=approx)).backward(torch.from_numpy(g_full))
    ref_ls_grad = xt.grad.numpy().copy()
    shift = np.floor(o.pam(x, C, off).max())

    # this package's unfused composition: the same torch ops, so the same bits
    xt = torch.from_numpy(x.copy()).requires_grad_()
    y = composites.logsumexp(xt, dim=-1, offset=off, approx_bwd=approx)
    y.backward(torch.from_numpy(g_rows))
    assert_same_bits(y.detach().numpy(), ref_val, "composites.logsumexp")
    assert_same_bits(xt.grad.numpy(), ref_grad, "composites.logsumexp gradient")
    xt = torch.from_numpy(x.copy()).requires_grad_()
    composites.log_softmax(xt, dim=-1, offset=off, approx_bwd=approx).backward(torch.from_numpy(g_full))
    assert_same_bits(xt.grad.numpy(), ref_ls_grad, "composites.log_softmax gradient")

    # the oracle's fused restatement and the hand-chained formulas: fixed-order row sums instead of torch's
    lse, ls = o.logsumexp_fwd(x, off, with_log_softmax=True)
    close(lse, ref_val, "oracle logsumexp", 2e-6)
    close(ls, x - ref_val[:, None], "oracle log_softmax", 2e-6)
    assert_same_bits(lse, logsumexp_chain(o, x, off), "oracle logsumexp vs hand chain")
    close(o.logsumexp_bwd(x, g_rows, shift, off, _flags(approx)), ref_grad, "oracle logsumexp gradient")
    close(o.logsumexp_bwd(x, g_full, shift, off, _flags(approx), log_softmax=True), ref_ls_grad, "oracle log_softmax gradient")
    assert_same_bits(o.logsumexp_bwd(x, g_rows, shift, off, _flags(approx)), logsumexp_grad_chain(o, x, g_rows, off, _flags(approx)),
                     "oracle logsumexp gradient vs hand chain")


# ------------------------------------------------------------------ GPU: HIP kernels == oracle fused
def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("off", [None, OFF])
def test_gpu_softmax_forward_backward(oracle, off):
    # 4097 ... 16384 values: a work-group per row
    # (every values-per-lane instance of the register-resident kernels: 64, 65, 192, 197, 300, 512, 768, 1000)
    for rows, n in [(1, 1), (3, 5), (4, 63), (4, 64), (5, 65), (5, 192), (64, 197), (7, 300), (7, 384), (3, 512), (3, 768), (2, 1000), (300, 32), (3, 4096), (5, 4097),
                    (3, 6145), (2, 10000), (2, 12288), (2, 16384), (2, 16385)]:
        x = rows_case(rows * 1000 + n, rows, n)
        g = np.random.RandomState(n).standard_normal(x.shape).astype(np.float32)
        want, row_sum, shift = oracle.softmax_fwd(x, off)
        for approx in (False, True, (True, False), (False, True)):
            xt = _dev(x).requires_grad_()
            y = pam_amd.softmax(xt, dim=-1, offset=off, approx_bwd=approx)
            assert_same_bits(y.detach().cpu().numpy(), want, f"softmax {rows}x{n}")
            y.backward(_dev(g))
            flags = _flags(approx)
            assert_same_bits(xt.grad.cpu().numpy(), oracle.softmax_bwd(x, g, row_sum, shift, off, flags),
                             f"softmax gradient {rows}x{n} approx={approx}")


@pytest.mark.gpu
def test_gpu_softmax_matches_unfused_composition(oracle):
    """The single kernel against the chain of primitive kernels on the same device: equal up to
    the order of the row sums; leading dimensions and the module-level switch."""
    x = rows_case(21, 12 * 7, 50).reshape(12, 7, 50)
    g = np.random.RandomState(3).standard_normal(x.shape).astype(np.float32)
    res = {}
    for fused_on in (True, False):
        composites.fused_rows = fused_on
        try:
            xt = _dev(x).requires_grad_()
            y = pam_amd.softmax(xt, dim=-1, approx_bwd=True)
            y.backward(_dev(g))
            res[fused_on] = (y.detach().cpu().numpy(), xt.grad.cpu().numpy())
        finally:
            composites.fused_rows = True
    assert np.allclose(res[True][0], res[False][0], rtol=2e-6, atol=1e-7)
    scale = np.abs(res[False][1]).max()
    assert np.abs(res[True][1] - res[False][1]).max() <= 5e-6 * scale
    # a reduction over another dimension keeps the unfused chain
    y0 = pam_amd.softmax(_dev(x), dim=1)
    assert y0.shape == x.shape and torch.isfinite(y0[~torch.isnan(y0)]).all()


@pytest.mark.gpu
def test_gpu_softmax_special_values(oracle):
    x = rows_case(3, 6, 40, masks=False)
    x[0, :] = -np.inf
    x[2, 5] = 3.0e38
    x[3, 1] = 1e-40
    x[4, 2] = 0.0
    want, row_sum, shift = oracle.softmax_fwd(x)
    assert_same_bits(pam_amd.softmax(_dev(x), dim=-1).cpu().numpy(), want, "special values")
    x[1, 3] = np.nan
    assert torch.isnan(pam_amd.softmax(_dev(x), dim=-1)).all()


@pytest.mark.gpu
@pytest.mark.parametrize("off", [None, OFF])
@pytest.mark.parametrize("approx", [False, True])
@pytest.mark.parametrize("n", [60, 100, 150, 200, 350, 512, 700, 1000, 2000, 20000])      # (every values-per-lane instance)
def test_gpu_exact_gradients_at_the_edges_of_the_unchecked_forms(oracle, n, approx, off):
    """All-exact (and all-approximate) gradients without an offset first run on unchecked arithmetic: inputs and upstream
    gradients at and beyond the edges of what that accepts (zeros, subnormals, huge and tiny values, inf, NaN, a variance
    of exactly 1)."""
    rng = np.random.RandomState(n)
    x = (rng.standard_normal((12, n)) * 3).astype(np.float32)
    x[1, 3] = 0.0; x[2, 5] = 1e-40; x[3, 7] = 3e38; x[4, 9] = -3e38; x[5, 11] = 2.0 ** -120; x[6, :] = 2.0 ** 100; x[7, 13] = -np.inf
    x[8, :] = np.where(np.arange(n) % 2 == 0, 1.0, -1.0)             # mean 0, variance 1 (n even)
    g = rng.standard_normal(x.shape).astype(np.float32)
    g[0, 1] = 0.0; g[0, 2] = 1e-42; g[1, 4] = np.inf; g[2, 6] = np.nan; g[3, 8] = 3e38; g[9, :] = 0.0; g[10, 3] = 2.0 ** -130
    flags = (approx, approx, approx)
    xt = _dev(x).requires_grad_()
    y = pam_amd.softmax(xt, dim=-1, approx_bwd=approx, offset=off)
    want, row_sum, shift = oracle.softmax_fwd(x, off)
    assert_same_bits(y.detach().cpu().numpy(), want, "softmax")
    y.backward(_dev(g))
    assert_same_bits(xt.grad.cpu().numpy(), oracle.softmax_bwd(x, g, row_sum, shift, off, flags), "softmax gradient")
    xf = np.where(np.isfinite(x), x, np.float32(1.5)).astype(np.float32)
    xt = _dev(xf).requires_grad_()
    y = pam_amd.log_softmax(xt, dim=-1, approx_bwd=approx, offset=off)
    y.backward(_dev(g))
    sh = np.floor(oracle.pam(xf, C, off).max())
    assert_same_bits(xt.grad.cpu().numpy(), oracle.logsumexp_bwd(xf, g, sh, off, flags, log_softmax=True), "log_softmax gradient")
    xt = _dev(xf).requires_grad_()
    pam_amd.logsumexp(xt, dim=-1, approx_bwd=approx, offset=off).backward(_dev(g[:, 0].copy()))
    assert_same_bits(xt.grad.cpu().numpy(), oracle.logsumexp_bwd(xf, g[:, 0].copy(), sh, off, flags), "logsumexp gradient")
    w = (rng.standard_normal(n) + 2).astype(np.float32); w[3] = 0.0; w[5] = 1e-39; w[7] = -2.0
    for ww in (None, w):
        xt = _dev(xf).requires_grad_()
        wt = None if ww is None else _dev(ww).requires_grad_()
        y = pam_amd.layer_norm(xt, n, wt, None, approx_bwd=approx, offset=off)
        y.backward(_dev(g))
        dx, _ = oracle.layer_norm_bwd(xf, ww, g, 1e-5, off, flags)
        assert_same_bits(xt.grad.cpu().numpy(), dx, "layer_norm gradient")


@pytest.mark.gpu
@pytest.mark.parametrize("approx", [True, False])
@pytest.mark.parametrize("off", [None, OFF])
def test_gpu_long_rows_with_special_values(oracle, off, approx):
    """Rows held by a whole work-group: a value outside the normal range anywhere in the row sends every
    thread of the row to the checked arithmetic (forward, all-approximate and all-exact gradients)."""
    n = 9000
    x = rows_case(77, 6, n, masks=False)
    x[1, 8999] = 0.0; x[2, 1024] = 1e-40; x[3, 5000] = np.inf; x[4, 63] = -np.inf; x[5, 4000] = np.nan
    g = np.random.RandomState(8).standard_normal(x.shape).astype(np.float32)
    g[0, 77] = 0.0; g[1, 5] = 1e-41
    w = (np.random.RandomState(9).standard_normal(n) + 2).astype(np.float32); w[17] = 0.0
    xt = _dev(x).requires_grad_()
    y = pam_amd.softmax(xt, dim=-1, offset=off, approx_bwd=approx)
    want, row_sum, shift = oracle.softmax_fwd(x, off)
    assert_same_bits(y.detach().cpu().numpy(), want, "softmax")
    y.backward(_dev(g))
    assert_same_bits(xt.grad.cpu().numpy(), oracle.softmax_bwd(x, g, row_sum, shift, off, (approx, approx, approx)), "softmax gradient")
    xs = x[:3]                                       # finite rows for the shifted ops
    lse, ls = oracle.logsumexp_fwd(xs, off, with_log_softmax=True)
    xt = _dev(xs).requires_grad_()
    y = pam_amd.log_softmax(xt, dim=-1, offset=off, approx_bwd=approx)
    assert_same_bits(y.detach().cpu().numpy(), ls, "log_softmax")
    y.backward(_dev(g[:3]))
    sh = np.floor(oracle.pam(xs, C, off).max())
    assert_same_bits(xt.grad.cpu().numpy(), oracle.logsumexp_bwd(xs, g[:3], sh, off, (approx, approx, approx), log_softmax=True), "log_softmax gradient")
    assert_same_bits(pam_amd.mean(_dev(x), dim=-1, offset=off).cpu().numpy(), oracle.row_mean_fwd(x, off), "mean")
    xt = _dev(x).requires_grad_(); wt = _dev(w).requires_grad_()
    y = pam_amd.layer_norm(xt, n, wt, None, offset=off, approx_bwd=approx)
    assert_same_bits(y.detach().cpu().numpy(), oracle.layer_norm_fwd(x, w, None, 1e-5, off), "layer_norm")
    y.backward(_dev(g))
    dx, _ = oracle.layer_norm_bwd(x, w, g, 1e-5, off, (approx, approx, approx))
    assert_same_bits(xt.grad.cpu().numpy(), dx, "layer_norm gradient")


@pytest.mark.gpu
@pytest.mark.parametrize("rows,n", [(20000, 520), (1100, 4100)])
def test_gpu_more_rows_than_the_launch_holds(oracle, rows, n):
    """More rows than wavefronts (work-groups) in the launch: every wavefront (work-group) walks several rows, the
    forward kernels fetching the next row while they compute the current one."""
    x = rows_case(rows + n, rows, n)
    g = np.random.RandomState(4).standard_normal(x.shape).astype(np.float32)
    xt = _dev(x).requires_grad_()
    y = pam_amd.softmax(xt, dim=-1, approx_bwd=True)
    want, row_sum, shift = oracle.softmax_fwd(x)
    assert_same_bits(y.detach().cpu().numpy(), want, "softmax")
    y.backward(_dev(g))
    assert_same_bits(xt.grad.cpu().numpy(), oracle.softmax_bwd(x, g, row_sum, shift, None, (True, True, True)), "softmax gradient")
    xf = rows_case(rows + n + 1, rows, n, masks=False)
    lse, ls = oracle.logsumexp_fwd(xf, None, with_log_softmax=True)
    xt = _dev(xf).requires_grad_()
    y = pam_amd.log_softmax(xt, dim=-1, approx_bwd=True)
    assert_same_bits(y.detach().cpu().numpy(), ls, "log_softmax")
    y.backward(_dev(g))
    sh = np.floor(oracle.pam(xf, C).max())
    assert_same_bits(xt.grad.cpu().numpy(), oracle.logsumexp_bwd(xf, g, sh, None, (True, True, True), log_softmax=True), "log_softmax gradient")
    assert_same_bits(pam_amd.logsumexp(_dev(xf), dim=-1).cpu().numpy(), lse, "logsumexp")
    w = (np.random.RandomState(6).standard_normal(n) + 2).astype(np.float32); b = np.random.RandomState(7).standard_normal(n).astype(np.float32)
    xt = _dev(xf).requires_grad_()
    y = pam_amd.layer_norm(xt, n, _dev(w), _dev(b), approx_bwd=True)
    assert_same_bits(y.detach().cpu().numpy(), oracle.layer_norm_fwd(xf, w, b, 1e-5), "layer_norm")
    y.backward(_dev(g))
    assert_same_bits(xt.grad.cpu().numpy(), oracle.layer_norm_bwd(xf, w, g, 1e-5, None, (True, True, True))[0], "layer_norm gradient")
    assert_same_bits(pam_amd.mean(_dev(xf), dim=-1).cpu().numpy(), oracle.row_mean_fwd(xf), "mean")


@pytest.mark.gpu
@pytest.mark.parametrize("off", [None, OFF])
def test_gpu_logsumexp_mean_layer_norm(oracle, off):
    for rows, n in [(1, 1), (3, 7), (4, 64), (50, 192), (5, 384), (2, 513), (33, 512), (3, 768), (2, 4096), (3, 4097), (3, 8193), (3, 10000), (2, 12289), (2, 16384), (2, 16385)]:
        x = rows_case(rows * 77 + n, rows, n, masks=False)
        xt = _dev(x)
        lse, ls = oracle.logsumexp_fwd(x, off, with_log_softmax=True)
        assert_same_bits(pam_amd.logsumexp(xt, dim=-1, offset=off).cpu().numpy(), lse, "logsumexp")
        assert pam_amd.logsumexp(xt, dim=-1, keepdim=True, offset=off).shape == (rows, 1)
        assert_same_bits(pam_amd.log_softmax(xt, dim=-1, offset=off).cpu().numpy(), ls, "log_softmax")
        assert_same_bits(pam_amd.mean(xt, dim=-1, offset=off).cpu().numpy(), oracle.row_mean_fwd(x, off), "mean")
        rng = np.random.RandomState(n)
        w, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
        for ww, bb in [(None, None), (w, None), (w, b)]:
            got = pam_amd.layer_norm(xt, n, None if ww is None else _dev(ww), None if bb is None else _dev(bb), offset=off)
            assert_same_bits(got.cpu().numpy(), oracle.layer_norm_fwd(x, ww, bb, 1e-5, off), f"layer_norm {rows}x{n}")


@pytest.mark.gpu
def test_gpu_layer_norm_with_graph_keeps_gradients(oracle):
    """With a graph recorded the unfused chain runs (it carries the gradient); the values agree
    with the single kernel up to the order of the row sums."""
    x = rows_case(9, 40, 192, masks=False)
    ln = pam_amd.LayerNorm(192, approx_bwd=True).cuda()
    xt = _dev(x).requires_grad_()
    y = ln(xt)
    y.sum().backward()
    assert xt.grad is not None and torch.isfinite(xt.grad).all() and ln.weight.grad is not None
    with torch.no_grad():
        y2 = ln(_dev(x))
    assert_same_bits(y2.cpu().numpy(), oracle.layer_norm_fwd(x, np.ones(192, np.float32), np.zeros(192, np.float32)), "no-grad path")
    assert np.allclose(y.detach().cpu().numpy(), y2.cpu().numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_gpu_attention_softmax_full_size(oracle):
    """Attention probabilities at the benchmark's shape, batch 64 x 3 heads x 197 x 197, against the oracle."""
    rng = np.random.RandomState(0)
    x = rng.standard_normal((192, 197, 197)).astype(np.float32)
    g = rng.standard_normal(x.shape).astype(np.float32)
    xt = _dev(x).requires_grad_()
    y = pam_amd.softmax(xt, dim=-1, approx_bwd=True)
    y.backward(_dev(g))
    want, row_sum, shift = oracle.softmax_fwd(x)
    assert_same_bits(y.detach().cpu().numpy(), want, "softmax 192x197x197")
    assert_same_bits(xt.grad.cpu().numpy(), oracle.softmax_bwd(x, g, row_sum, shift, None, (True, True, True)), "its gradient")
    assert np.abs(want.sum(-1) - 1).max() < 0.1


@pytest.mark.gpu
@pytest.mark.parametrize("off", [None, OFF])
def test_gpu_logsumexp_and_layer_norm_gradients(oracle, off):
    # rows beyond 1024 values: the gradient kernels sweep the row several times instead of holding it in registers
    for rows, n in [(1, 1), (3, 7), (5, 64), (40, 192), (6, 384), (9, 513), (4, 768), (6, 1024), (5, 1025), (3, 2500), (2, 4097), (2, 6200), (2, 10000), (2, 12300), (2, 16384), (2, 16385)]:
        x = rows_case(rows * 13 + n, rows, n, masks=False)
        rng = np.random.RandomState(n)
        g_rows = rng.standard_normal(rows).astype(np.float32); g_full = rng.standard_normal(x.shape).astype(np.float32)
        w = (rng.standard_normal(n) + 2).astype(np.float32); b = rng.standard_normal(n).astype(np.float32)
        shift = np.floor(oracle.pam(x, C, off).max())
        for approx in (False, True, (True, False)):
            xt = _dev(x).requires_grad_()
            pam_amd.logsumexp(xt, dim=-1, offset=off, approx_bwd=approx).backward(_dev(g_rows))
            assert_same_bits(xt.grad.cpu().numpy(), oracle.logsumexp_bwd(x, g_rows, shift, off, _flags(approx)), f"logsumexp gradient {rows}x{n}")
            xt = _dev(x).requires_grad_()
            y = pam_amd.log_softmax(xt, dim=-1, offset=off, approx_bwd=approx)
            assert_same_bits(y.detach().cpu().numpy(), oracle.logsumexp_fwd(x, off, with_log_softmax=True)[1], "log_softmax")
            y.backward(_dev(g_full))
            assert_same_bits(xt.grad.cpu().numpy(), oracle.logsumexp_bwd(x, g_full, shift, off, _flags(approx), log_softmax=True),
                             f"log_softmax gradient {rows}x{n}")
            for ww, bb in [(None, None), (w, b)]:
                xt = _dev(x).requires_grad_()
                wt = None if ww is None else _dev(ww).requires_grad_(); bt = None if bb is None else _dev(bb).requires_grad_()
                y = pam_amd.layer_norm(xt, n, wt, bt, offset=off, approx_bwd=approx)
                assert_same_bits(y.detach().cpu().numpy(), oracle.layer_norm_fwd(x, ww, bb, 1e-5, off), "layer_norm")
                y.backward(_dev(g_full))
                dx, terms = oracle.layer_norm_bwd(x, ww, g_full, 1e-5, off, _flags(approx))
                assert_same_bits(xt.grad.cpu().numpy(), dx, f"layer_norm gradient {rows}x{n} approx={approx}")
                if ww is not None:
                    want_w = torch.from_numpy(terms).sum(0).numpy()
                    assert np.abs(wt.grad.cpu().numpy() - want_w).max() <= 1e-5 * np.abs(want_w).max() + 1e-7
                    assert np.allclose(bt.grad.cpu().numpy(), g_full.sum(0), rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
def test_gpu_row_gradients_match_unfused_composition():
    """LayerNorm and log_softmax in training on the GPU: single kernels against the chains of
    primitive kernels, values and all gradients, up to the order of the sums."""
    x = rows_case(41, 8 * 25, 96, masks=False).reshape(8, 25, 96)
    g = np.random.RandomState(5).standard_normal(x.shape).astype(np.float32)
    res = {}
    for fused_on in (True, False):
        composites.fused_rows = fused_on
        try:
            torch.manual_seed(0)
            ln = pam_amd.LayerNorm(96, approx_bwd=True).cuda()
            with torch.no_grad():
                ln.weight.copy_(torch.randn(96).cuda() + 2); ln.bias.copy_(torch.randn(96).cuda())
            xt = _dev(x).requires_grad_()
            y = pam_amd.log_softmax(ln(xt), dim=-1, approx_bwd=True)
            y.backward(_dev(g))
            res[fused_on] = [t.detach().cpu().numpy() for t in (y, xt.grad, ln.weight.grad, ln.bias.grad)]
        finally:
            composites.fused_rows = True
    for a, b in zip(res[True], res[False]):
        assert np.abs(a - b).max() <= 2e-5 * np.abs(b).max()
    # long rows too
    wide = _dev(rows_case(42, 3, 1500, masks=False)).requires_grad_()
    pam_amd.layer_norm(wide, 1500, approx_bwd=True).sum().backward()
    assert torch.isfinite(wide.grad).all()


@pytest.mark.gpu
@pytest.mark.parametrize("off", [None, OFF])
def test_gpu_mean_gradient(oracle, off):
    """mean over the last dimension in training: the single kernel's approximate gradient is the chain's,
    (1 (/) n) (*) g for every element, bit for bit; the exact gradient keeps the chain."""
    x = rows_case(77, 37, 300, masks=False)
    g = np.random.RandomState(8).standard_normal(37).astype(np.float32)
    res = {}
    for fused_on in (True, False):
        composites.fused_rows = fused_on
        try:
            xt = _dev(x).requires_grad_()
            y = pam_amd.mean(xt, dim=-1, offset=off, approx_bwd=True)
            y.backward(_dev(g))
            res[fused_on] = (y.detach().cpu().numpy(), xt.grad.cpu().numpy())
        finally:
            composites.fused_rows = True
    assert_same_bits(res[True][0], oracle.row_mean_fwd(x, off), "mean")
    assert np.abs(res[True][0] - res[False][0]).max() <= 1e-6 * np.abs(res[False][0]).max() + 1e-7      # torch.sum's order
    assert_same_bits(res[True][1], res[False][1], "mean gradient against the chain")
    want = oracle.pam(oracle.pad(np.ones_like(g), np.full_like(g, 300.0), off), g, off)
    assert_same_bits(res[True][1], np.broadcast_to(want[:, None], x.shape), "mean gradient")
    xt = _dev(x).requires_grad_()
    pam_amd.mean(xt, dim=-1, offset=off, approx_bwd=False).backward(_dev(g))                             # exact: the chain
    assert torch.isfinite(xt.grad).all()
