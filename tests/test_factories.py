"""The configuration hooks (counterpart of shared/modules/factories.py), the op-table cross
entropy (pam/pam_opt.py) and the base-2 torch comparison functions (pam/pam_experimental.py).
Host logic only: CPU, no kernel calls except through the oracle-backed kernel object."""
import math
import warnings

import numpy as np
import pytest
import torch
from torch import nn

import pam_amd
from pam_amd import cuda_bindings, factories, pam_experimental, pam_ops
from test_host_api import OracleKernels


def test_linear_and_conv_factories_resolve_names_dicts_and_yaml():
    assert type(factories.get_linear_factory(None)(4, 3)) is nn.Linear
    assert type(factories.get_linear_factory("linear")(4, 3)) is nn.Linear
    assert type(factories.get_linear_factory("custom")(4, 3)) is factories.CustomLinear
    lin = factories.get_linear_factory("pam")(4, 3)
    assert type(lin) is pam_amd.Linear and lin.approx_bwd is False and lin.offset is None
    # defaults lose against call-site arguments, overrides win over them
    make = factories.get_linear_factory({"subtype": "PAM", "dkwargs": {"approx_bwd": True, "bias": True},
                                         "okwargs": {"offset": 1.05}})
    lin = make(4, 3, bias=False, offset=2.0)
    assert lin.approx_bwd is True and lin.bias is None and lin.offset == 1.05
    lin = factories.get_linear_factory("{subtype: pam, dkwargs: {approx_bwd: true}}")(in_features=5, out_features=2)
    assert type(lin) is pam_amd.Linear and lin.approx_bwd is True and lin.weight.shape == (2, 5)
    conv = factories.get_conv_factory("pam")(3, 8, kernel_size=3)
    assert type(conv) is pam_amd.Conv2d
    assert type(factories.get_conv_factory(None)(3, 8, 3)) is nn.Conv2d
    with pytest.raises((ValueError, KeyError, TypeError, AttributeError)):
        factories.get_linear_factory("no_such_layer")(4, 3)
    with pytest.raises(ValueError):
        factories.get_module_factory(3.5, {})


def test_keywords_a_constructor_does_not_take_are_dropped_with_a_warning():
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        lin = factories.get_linear_factory({"subtype": "standard", "dkwargs": {"approx_bwd": True}})(4, 3)
    assert type(lin) is nn.Linear and any("approx_bwd" in str(w.message) for w in seen)
    assert factories.get_valid_kwargs(lambda a, **kw: 0, {"z": 1}) == {"z": 1}
    assert factories.get_valid_kwargs(lambda a, b=1: 0, {"b": 2, "z": 1}) == {"b": 2}


def test_sequential_norm_activation_bias_gain_factories():
    desc = [{"type": "linear", "subtype": "pam", "okwargs": {"approx_bwd": True}},
            {"type": "norm", "subtype": "ln", "dkwargs": {"normalized_shape": 6}},
            {"type": "activation", "subtype": "leaky_relu"}]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        seq = factories.get_linear_factory(desc)(in_features=4, out_features=6)
    assert [type(m) for m in seq] == [pam_amd.Linear, nn.LayerNorm, nn.LeakyReLU] and seq[0].approx_bwd is True
    # pam.LayerNorm takes **kwargs, so nothing is filtered for it (as in the reference): direct use only
    assert type(factories.get_norm_factory({"subtype": "pam_ln", "okwargs": {"approx_bwd": True}})(6)) is pam_amd.LayerNorm
    assert type(factories.get_norm_factory("bn2d")(8)) is nn.BatchNorm2d
    assert type(factories.get_norm_factory("ln")(8)) is nn.LayerNorm
    assert type(factories.get_activation_factory("relu")()) is nn.ReLU
    with pytest.raises(ValueError):
        factories.get_sequential_factory([{"type": "pooling", "subtype": "max"}])
    x = torch.arange(24.0).reshape(2, 3, 4)
    bias = factories.get_bias_factory(None)(3)
    gain = factories.get_gain_factory("gain")(3)
    with torch.no_grad():
        bias.bias.copy_(torch.tensor([1.0, 2.0, 3.0])); gain.gain.copy_(torch.tensor([2.0, 0.5, -1.0]))
    assert torch.equal(bias(x), x + torch.tensor([1.0, 2.0, 3.0]).view(1, 3, 1))
    assert torch.equal(gain(x), x * torch.tensor([2.0, 0.5, -1.0]).view(1, 3, 1))
    assert "3" in repr(bias)
    lazy_b, lazy_g = factories.get_bias_factory("lazy_bias")(), factories.get_gain_factory("lazy_bias")()
    assert torch.equal(lazy_b(x), x) and torch.equal(lazy_g(x), x)          # zeros and ones after materialising
    assert type(lazy_b) is factories.Bias and type(lazy_g) is factories.Gain and lazy_b.bias.shape == (3,)


def test_function_dict_tables():
    names = {"mean", "mul", "div", "softmax", "bmm", "logsumexp", "log_softmax", "pow"}
    std = factories.get_function_dict("standard")
    assert set(std) == names and std["bmm"] is torch.bmm and std["softmax"] is torch.nn.functional.softmax
    assert factories.get_function_dict("torch")["pow"] is torch.pow
    two = factories.get_function_dict("standard2")
    assert two["softmax"] is pam_experimental.torch_softmax2 and two["mul"] is torch.mul
    p = factories.get_function_dict("pam")
    assert set(p) == names and all(p[n] is getattr(pam_amd, n) for n in names)
    assert factories.get_function_dict("pam_bmm_only")["bmm"] is pam_amd.bmm
    assert factories.get_function_dict("pam_bmm_only")["softmax"] is torch.nn.functional.softmax
    assert factories.get_function_dict("pam_softmax_only")["softmax"] is pam_amd.softmax
    std["mul"] = None
    assert factories.get_function_dict("standard")["mul"] is torch.mul          # each call hands out a fresh table
    with pytest.raises((ValueError, AssertionError)):
        factories.get_function_dict("nonsense")
    with pytest.raises(AssertionError):
        factories.get_function_dict({"type": "standard"})


def test_function_dict_form_filters_keywords(oracle, monkeypatch):
    """fairseq hands `dtype=` to the softmax it looks up (fairseq/utils.py:514-518): the plain
    'pam' table passes it on (and pam.softmax rejects it, as in the reference), the dict form drops it."""
    monkeypatch.setattr(cuda_bindings, "cuda_kernels", OracleKernels(oracle))
    monkeypatch.setattr(pam_ops, "_require_kernel", lambda t, use_kernel: None)
    x = torch.randn(3, 5, generator=torch.Generator().manual_seed(0))
    with pytest.raises(TypeError):
        factories.get_function_dict("pam")["softmax"](x, dim=-1, dtype=torch.float32)
    table = factories.get_function_dict("{type: pam, okwargs: {approx_bwd: true}, dkwargs: {offset: 1.0552}}")
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        y = table["softmax"](x, dim=-1, dtype=torch.float32)
    assert torch.equal(y, pam_amd.softmax(x, dim=-1, offset=1.0552, approx_bwd=True))
    assert torch.equal(table["mul"](x, 0.5, offset=None), pam_amd.mul(x, 0.5))        # call-site beats dkwargs
    xr = x.clone().requires_grad_()
    table["mul"](xr, x).sum().backward()
    assert torch.equal(xr.grad, pam_amd.mul(torch.ones_like(x), x, offset=1.0552))    # approx_bwd forced on: dA = delta (*) B


def test_cross_entropy_with_torch_ops_has_torch_gradient():
    """With the ordinary ops the hand-written backward must reproduce autograd's gradient of
    torch's cross entropy: pins the formula (pam/pam_opt.py:29-51) for every option."""
    g = torch.Generator().manual_seed(1)
    X = torch.randn(12, 7, generator=g); Y = torch.randint(0, 7, (12,), generator=g); Y[3] = -100; Y[8] = -100
    w = torch.rand(7, generator=g) + 0.5
    ops = factories.get_function_dict("standard")
    for reduction in ("mean", "sum"):
        for smoothing in (0.0, 0.1):
            for weight in (None, w):
                if weight is not None and (reduction == "mean" or smoothing):
                    continue        # torch normalises weighted means by the weight sum; the reference divides by the row count
                a = X.clone().requires_grad_(); b = X.clone().requires_grad_()
                la = pam_amd.cross_entropy(a, Y, weight, -100, reduction, smoothing, op_dict=ops)
                lb = torch.nn.functional.cross_entropy(b, Y, weight, ignore_index=-100, reduction=reduction, label_smoothing=smoothing)
                assert torch.equal(la, lb)
                (la * 1.5).backward(); (lb * 1.5).backward()
                if reduction == "mean":
                    # the reference divides by all rows, torch by the rows that are not ignored
                    scale = (Y != -100).sum().item() / X.shape[0]
                    assert torch.allclose(a.grad / scale, b.grad, atol=1e-6), (reduction, smoothing)
                else:
                    assert torch.allclose(a.grad, b.grad, atol=1e-6), (reduction, smoothing)
                assert (a.grad[3] == 0).all() and (a.grad[8] == 0).all()
    with pytest.raises(AssertionError):
        pam_amd.cross_entropy(X, Y)


def test_cross_entropy_with_pam_ops(oracle, monkeypatch):
    monkeypatch.setattr(cuda_bindings, "cuda_kernels", OracleKernels(oracle))
    monkeypatch.setattr(pam_ops, "_require_kernel", lambda t, use_kernel: None)
    g = torch.Generator().manual_seed(2)
    X = torch.randn(6, 5, generator=g, requires_grad=True); Y = torch.randint(0, 5, (6,), generator=g)
    loss = pam_amd.cross_entropy(X, Y, None, -100, "mean", 0.0, op_dict=factories.get_function_dict("pam"))
    assert torch.equal(loss, torch.nn.functional.cross_entropy(X.detach(), Y))
    loss.backward()
    want = pam_amd.mul(pam_amd.div(pam_amd.softmax(X.detach(), dim=-1) - torch.nn.functional.one_hot(Y, 5).float(), 6),
                       torch.ones(1, 1))
    assert torch.equal(X.grad, want)
    ref = torch.softmax(X.detach(), -1) - torch.nn.functional.one_hot(Y, 5).float()
    assert torch.allclose(X.grad * 6, ref, atol=0.08)               # PAM softmax and division are approximations


def test_base2_comparison_functions():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 9, generator=g) * 3
    ln2 = math.log(2.0)
    assert torch.allclose(pam_experimental.torch_softmax2(x, dim=-1), torch.softmax(x * ln2, -1), atol=1e-6)
    assert torch.allclose(pam_experimental.torch_logsumexp2(x, dim=-1, keepdim=False), torch.logsumexp(x * ln2, -1) / ln2, atol=1e-5)
    assert torch.allclose(pam_experimental.torch_log_softmax2(x, dim=-1), torch.log_softmax(x * ln2, -1) / ln2, atol=1e-5)
    assert pam_experimental.torch_softmax2(x.double(), dim=0, dtype=torch.float32).dtype == torch.float32
    row = x[0]; t = torch.tensor(4)
    want = -(torch.log_softmax(row * ln2, -1) / ln2)[4]
    assert torch.allclose(pam_experimental.torch_cross_entropy2(row, t, reduction=None).squeeze(), want, atol=1e-5)
    with pytest.raises(ValueError):
        pam_experimental.torch_cross_entropy2(row, t, reduction="median")
