"""The compositions built on the PAM primitives (softmax, layer_norm, conv2d, ...):
on the CPU with the oracle standing in for the kernels (composition logic only), and on the
GPU against the reference's own constructions (pam/test_pam.py:151-193) and the oracle."""
import math

import numpy as np
import pytest
import torch

import pam_amd
from pam_amd import composites, cuda_bindings, pam_ops
from _util import assert_same_bits
from test_host_api import OracleKernels


@pytest.fixture()
def on_cpu(oracle, monkeypatch):
    """Kernel object replaced by the oracle, device check lifted: exercises the Python layer on CPU tensors."""
    monkeypatch.setattr(cuda_bindings, "cuda_kernels", OracleKernels(oracle))
    monkeypatch.setattr(pam_ops, "_require_kernel", lambda t, use_kernel: None)
    return oracle


def _tsum(a, keepdims=False):
    """Row sums with torch's CPU reduction order (what the composition itself uses)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).sum(-1, keepdim=keepdims).numpy()


def _softmax_restated(o, x, off=None):
    c = np.float32(math.log2(math.e))
    s = o.pam(x, c, off)
    s = np.where(np.isneginf(x), -np.inf, s).astype(np.float32)
    shift = np.floor(s.max())
    w = np.where(np.isneginf(x), 0, o.pa_exp((s - shift).astype(np.float32), 2.0, off)).astype(np.float32)
    return o.pad(w, _tsum(w, True), off)


def test_softmax_and_logsumexp_composition(on_cpu):
    o = on_cpu
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 9, generator=g) * 3
    x[1, 2] = float("-inf"); x[3, :4] = float("-inf")
    for off in (None, 1.0552):
        got = pam_amd.softmax(x, dim=-1, offset=off).numpy()
        assert_same_bits(got, _softmax_restated(o, x.numpy(), off), f"softmax offset={off}")
        assert (got[np.isneginf(x.numpy())] == 0).all()
    assert np.abs(pam_amd.softmax(x, dim=-1).numpy().sum(-1) - 1).max() < 0.1      # PAM division is approximate
    y = torch.randn(4, 7, generator=g)
    c = np.float32(math.log2(math.e))
    s = o.pam(y.numpy(), c); shift = np.floor(s.max())
    total = _tsum(o.pa_exp((s - shift).astype(np.float32), 2.0))
    want = o.pad((shift + o.pa_log(total, 2.0)).astype(np.float32), c)
    assert_same_bits(pam_amd.logsumexp(y, dim=-1).numpy(), want, "logsumexp")
    assert_same_bits(pam_amd.log_softmax(y, dim=-1).numpy(), y.numpy() - want[:, None], "log_softmax")
    assert np.allclose(pam_amd.logsumexp(y, dim=-1).numpy(), torch.logsumexp(y, -1).numpy(), atol=0.5)   # piecewise-affine, not exact


def test_mean_and_layer_norm_composition(on_cpu):
    o = on_cpu
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 4, 16, generator=g)
    assert_same_bits(pam_amd.mean(x, dim=-1).numpy(), o.pad(_tsum(x.numpy()), np.float32(16)), "mean")
    assert pam_amd.mean(x).shape == () and pam_amd.mean(x, dim=(0, 2), keepdim=True).shape == (1, 4, 1)
    w, b = torch.randn(16, generator=g), torch.randn(16, generator=g)
    rows = x.numpy().reshape(-1, 16)
    mu = o.pad(_tsum(rows, True), np.float32(16))
    cen = (rows - mu).astype(np.float32)
    var = o.pad(_tsum(o.pam(cen, cen), True), np.float32(16))
    ve = (var + np.float32(1e-5)).astype(np.float32)
    root = np.where(ve == 0, 0, o.pa_exp(o.pam(o.pa_log(ve, 2.0), np.float32(0.5)), 2.0)).astype(np.float32)
    want = (o.pam(o.pad(cen, root).reshape(3, 4, 16), w.numpy()) + b.numpy()).astype(np.float32)
    assert_same_bits(pam_amd.layer_norm(x, 16, w, b).numpy(), want, "layer_norm")
    ln = pam_amd.LayerNorm(16, approx_bwd=True)
    with torch.no_grad():
        ln.weight.copy_(w); ln.bias.copy_(b)
    assert_same_bits(ln(x).detach().numpy(), want, "LayerNorm module")
    assert np.allclose(want, torch.nn.functional.layer_norm(x, (16,), w, b).numpy(), atol=0.35)
    assert set(ln.state_dict()) == set(torch.nn.LayerNorm(16).state_dict()) and "approx_bwd=True" in repr(ln)
    xr = x.clone().requires_grad_(); ln(xr).sum().backward()
    assert xr.grad.shape == x.shape and torch.isfinite(xr.grad).all()


def test_conv2d_composition(on_cpu):
    # weights that are powers of two make every PAM product exact: the convolution equals F.conv2d
    # (the construction of pam/test_pam.py:151-193)
    g = torch.Generator().manual_seed(2)
    X = (torch.randint(-64, 64, (2, 6, 9, 8), generator=g) / 16.0).requires_grad_()
    W = (2.0 ** torch.randint(-3, 3, (4, 6, 3, 3), generator=g).float()).requires_grad_()
    bias = torch.randn(4, generator=g)
    for kwargs in (dict(), dict(padding=1), dict(stride=2, padding="same"), dict(padding="valid")):
        got = pam_amd.conv2d(X, W, bias, approx_bwd=True, **kwargs)
        ref_kwargs = dict(kwargs)
        if ref_kwargs.get("padding") == "same":
            ref_kwargs["padding"] = 1
        want = torch.nn.functional.conv2d(X, W, bias, **ref_kwargs)
        assert got.shape == want.shape and torch.allclose(got, want, atol=1e-5), kwargs
    Xg = (torch.randint(-8, 9, (2, 8, 7, 6), generator=g) / 4.0)
    Wg = 2.0 ** torch.randint(-2, 3, (16, 2, 3, 3), generator=g).float()
    got = pam_amd.conv2d_group(Xg, Wg, None, padding=1, groups=4)
    assert torch.allclose(got, torch.nn.functional.conv2d(Xg, Wg, None, padding=1, groups=4), atol=1e-5)
    conv = pam_amd.Conv2d(8, 16, 3, padding=1, groups=4, bias=False, offset=1.0552)
    assert repr(conv).startswith("pam.Conv2d") and "offset=1.05520" in repr(conv)
    with torch.no_grad():
        conv.weight.copy_(Wg)
    assert conv(Xg).shape == (2, 16, 7, 6)
    with pytest.raises(ValueError):
        pam_amd.conv2d(X, W, padding="circular")
    # a dilation other than 1: the reference sizes its output without it (pam/pam_ops.py:137-138) and its final view
    # of the unfolded product raises; the same here
    with pytest.raises(RuntimeError):
        pam_amd.conv2d(X, W, None, dilation=2)


def _close(a, b):
    """Equal up to fp32 summation order: error small against the largest entry (sums of ~200
    exact products cancel, so an elementwise relative bound does not apply)."""
    return (a - b).abs().max().item() <= 2e-6 * b.abs().max().item()


@pytest.mark.gpu
def test_composites_on_device(oracle):
    from pam_amd._abi import load_library
    load_library()
    torch.manual_seed(0)
    # pam/test_pam.py:151-170 on the HIP path
    X1 = (torch.randint(-1024, 1024, (11, 13, 15, 17), device="cuda") / 64.0).requires_grad_()
    W1 = (2.0 ** torch.randint(-8, 8, (19, 13, 3, 5))).cuda().requires_grad_()
    X2 = X1.detach().clone().requires_grad_(); W2 = W1.detach().clone().requires_grad_()
    Y1 = pam_amd.conv2d(X1, W1, approx_bwd=True); Y1.sum().backward()
    Y2 = torch.nn.functional.conv2d(X2, W2); Y2.sum().backward()
    assert _close(Y1, Y2) and _close(X1.grad, X2.grad) and _close(W1.grad, W2.grad)
    # pam/test_pam.py:173-193
    for G in (1, 8):
        X1 = (torch.randint(-8, 9, (11, 16, 15, 17), device="cuda") / 4.0).requires_grad_()
        W1 = (2.0 ** torch.randint(-2, 3, (128, 16 // G, 3, 5))).cuda().requires_grad_()
        X2 = X1.detach().clone().requires_grad_(); W2 = W1.detach().clone().requires_grad_()
        Y1 = pam_amd.conv2d_group(X1, W1, groups=G, approx_bwd=True); Y1.sum().backward()
        Y2 = torch.nn.functional.conv2d(X2, W2, groups=G); Y2.sum().backward()
        assert _close(Y1, Y2) and _close(X1.grad, X2.grad) and _close(W1.grad, W2.grad)
    # softmax with masking, and layer_norm, against the restatement above on the oracle
    x = torch.randn(64, 197) * 3
    x[5, 10:] = float("-inf")
    got = pam_amd.softmax(x.cuda(), dim=-1, offset=1.0552).cpu().numpy()
    want = _softmax_restated(oracle, x.numpy(), 1.0552)
    assert np.allclose(got, want, rtol=2e-6, atol=1e-9)        # only the row sums differ (reduction order)
    assert (got[5, 10:] == 0).all()
    ln = pam_amd.LayerNorm(192, approx_bwd=True).cuda()
    h = torch.randn(8, 197, 192, device="cuda", requires_grad=True)
    out = ln(h); out.sum().backward()
    assert torch.allclose(out, torch.nn.functional.layer_norm(h, (192,)), atol=0.5) and torch.isfinite(h.grad).all()
