"""The reference is imported as `pam` (and its hook layer as `shared.modules.factories`): every attribute that
shared/modules/factories.py:128-265 and pam/__init__.py:8-10 read must resolve from this repository's root, and the
op tables must be bound to the same objects."""
import inspect

import pytest

import torch

import pam
import pam_amd
from shared.modules import factories


def test_every_attribute_the_hook_layer_reads():
    for name in "Linear Conv2d LayerNorm mean mul div softmax bmm logsumexp log_softmax pow".split():   # factories.py:128,138,176,242-249
        assert getattr(pam, name) is getattr(pam_amd, name), name
    for name in "torch_softmax2 torch_logsumexp2 torch_log_softmax2".split():                           # factories.py:235-238
        assert callable(getattr(pam.pam_experimental, name)), name
    # names of pam/pam_ops.py:16-115, 259-404 and pam/pam_opt.py that `from pam.pam_ops import *` gives
    for name in "exp exp2 log log2 matmul linear conv2d conv2d_group layer_norm cross_entropy".split():
        assert hasattr(pam, name), name
    import importlib
    for sub in "cuda_bindings pam_experimental pam_ops pam_opt utils".split():
        assert importlib.import_module("pam." + sub) is importlib.import_module("pam_amd." + sub), sub
    assert not hasattr(pam, "native")


def test_keyword_interface_of_the_ops():
    # offset / approx_bwd / use_kernel are what the configs pass (README recipes; pam/pam_ops.py:16-67, 82-115)
    for name in "mul div exp exp2 log log2 matmul bmm".split():
        params = inspect.signature(getattr(pam, name)).parameters
        for kw in ("offset", "approx_bwd", "use_kernel"):
            assert kw in params, (name, kw)
    lin = pam.Linear(8, 4, offset=None, approx_bwd=True, use_kernel=True)
    assert isinstance(lin, torch.nn.Linear)


def test_function_dict_binds_to_the_package():
    table = factories.get_function_dict("pam")
    for name in "mean mul div softmax bmm logsumexp log_softmax pow".split():
        assert table[name] is getattr(pam, name), name
    only = factories.get_function_dict("pam_bmm_only")
    assert only["bmm"] is pam.bmm and only["softmax"] is torch.nn.functional.softmax
    two = factories.get_function_dict("standard2")
    assert two["softmax"] is pam.pam_experimental.torch_softmax2
    assert factories.get_linear_factory("pam")(8, 4).__class__ is pam.Linear
    assert factories.get_conv_factory("pam")(3, 4, 3).__class__ is pam.Conv2d
    # the dict form filters keywords the op does not take (fairseq passes dtype= to softmax)
    custom = factories.get_function_dict({"type": "pam", "dkwargs": {"approx_bwd": True}, "okwargs": {}})
    assert set(custom) == set(table)


def test_pam_ops_module_serves_every_name_of_the_reference_module():
    """pam/pam_ops.py defines the primitives and the compositions in one module (its def / class names, :16-404)."""
    import importlib
    ops = importlib.import_module("pam.pam_ops")
    for name in ("mul", "div", "exp", "exp2", "log", "log2", "pow", "matmul", "bmm", "linear", "conv2d", "conv2d_group",
                 "Conv2d", "Linear", "mean", "softmax", "logsumexp", "log_softmax", "layer_norm", "LayerNorm"):
        assert callable(getattr(ops, name)), name
    from pam.pam_ops import softmax, LayerNorm          # noqa: F401
    import pam
    assert ops.softmax is pam.softmax and ops.Conv2d is pam.Conv2d
    with pytest.raises(AttributeError):
        ops.no_such_name
