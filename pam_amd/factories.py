"""Configuration hooks: strings / dicts / YAML snippets to module factories and to the
table of functional ops that the training libraries look up ("linear_cfg",
"functional_cfg").  Counterpart of the reference's shared/modules/factories.py, with
`pam_amd` behind the 'pam' entries; same function names, description formats and
keyword filtering, so a fork that does

    from shared.modules.factories import get_function_dict, get_linear_factory

works with `from pam_amd.factories import ...` instead.

A description is a known name ('pam', 'standard', ...), a dict
{'subtype': name, 'dkwargs': {...}, 'okwargs': {...}} (defaults that call-site arguments
override, and overrides that win over call-site arguments), a YAML string of such a dict,
or, for modules, a list of {'type': ..., 'subtype': ...} entries that becomes a Sequential.
"""
import copy
import inspect
import warnings

import torch
import yaml
from torch import nn
from torch.nn.modules.lazy import LazyModuleMixin
from torch.nn.parameter import Parameter, UninitializedParameter

import pam_amd as pam
from . import pam_experimental


class CustomLinear(nn.Linear):
    """Placeholder subclass used to test that factories reach submodules (shared/modules/factories.py:15-17)."""


class CustomConv2d(nn.Conv2d):
    """shared/modules/factories.py:20-22"""


class _PerChannel(nn.Module):
    """One learnable value per channel (dim 1), broadcast over the other dims."""
    _name = None
    _init = None

    def __init__(self, num_features=None):
        super().__init__()
        self.num_features = num_features
        setattr(self, self._name, Parameter(torch.empty(self.num_features)))
        self.reset_parameters()

    def _shaped(self, x):
        return getattr(self, self._name).view([d if i == 1 else 1 for i, d in enumerate(x.shape)])

    def reset_parameters(self):
        type(self)._init(getattr(self, self._name))

    def extra_repr(self):
        return f"{self.num_features}"


class Bias(_PerChannel):
    """x + bias[channel] (shared/modules/factories.py:25-42)"""
    _name, _init = "bias", staticmethod(nn.init.zeros_)

    def forward(self, x):
        return x + self._shaped(x)


class Gain(_PerChannel):
    """x * gain[channel] (shared/modules/factories.py:65-82)"""
    _name, _init = "gain", staticmethod(nn.init.ones_)

    def forward(self, x):
        return x * self._shaped(x)


class _LazyPerChannel(LazyModuleMixin):
    """Sizes the parameter from the first input (shared/modules/factories.py:45-62, 85-102)."""

    def __init__(self):
        super().__init__(0)
        setattr(self, self._name, UninitializedParameter())

    def reset_parameters(self):
        if not self.has_uninitialized_params() and self.num_features != 0:
            super().reset_parameters()

    def initialize_parameters(self, input):
        if self.has_uninitialized_params():
            with torch.no_grad():
                self.num_features = input.shape[1]
                getattr(self, self._name).materialize((self.num_features,))
                self.reset_parameters()


class LazyBias(_LazyPerChannel, Bias):
    cls_to_become = Bias


class LazyGain(_LazyPerChannel, Gain):
    cls_to_become = Gain


# ---------------------------------------------------------------- keyword filtering
def get_valid_kwargs(func, argdict):
    """The subset of argdict that func accepts; everything if it takes **kwargs
    (shared/modules/factories.py:198-206)."""
    params = inspect.signature(func).parameters
    if any(p.kind == p.VAR_KEYWORD for p in params.values()):
        return argdict
    return {k: v for k, v in argdict.items() if k in params}


def call_valid_kwargs(func, kwargs_dict, args_tuple=tuple()):
    """Calls func with the keywords it accepts and warns about the rest
    (shared/modules/factories.py:209-213)."""
    kwargs = get_valid_kwargs(func, kwargs_dict)
    dropped = sorted(set(kwargs_dict) - set(kwargs))
    if dropped:
        warnings.warn(f"Function {func} ignored extra arguments {dropped}")
    return func(*args_tuple, **kwargs)


# ---------------------------------------------------------------- module factories
def get_module_factory(desc, factories):
    """shared/modules/factories.py:105-125"""
    if isinstance(desc, str):
        if desc in factories:
            desc = {"subtype": desc}
        else:
            try:
                desc = yaml.safe_load(desc)
            except Exception:
                raise ValueError(f"Unknown linear function {desc}")
    if isinstance(desc, dict):
        factory = factories[desc["subtype"].lower()]
        defaults = desc.get("dkwargs", {})      # call-site arguments override these
        overrides = desc.get("okwargs", {})     # these override call-site arguments

        def make(*args, **kwargs):
            return call_valid_kwargs(factory, {**defaults, **kwargs, **overrides}, args)
        return make
    if isinstance(desc, list):
        return get_sequential_factory(desc)
    raise ValueError(f"Unknown configuration {desc=}")


def get_linear_factory(desc):
    """'standard' | 'linear' | 'pam' | 'custom' (shared/modules/factories.py:128-135)"""
    table = {"standard": nn.Linear, "linear": nn.Linear, "pam": pam.Linear, "custom": CustomLinear}
    return get_module_factory(desc or "standard", table)


def get_conv_factory(desc):
    """shared/modules/factories.py:138-145"""
    table = {"standard": nn.Conv2d, "conv2d": nn.Conv2d, "pam": pam.Conv2d, "custom": CustomConv2d}
    return get_module_factory(desc or "standard", table)


def get_bias_factory(desc):
    """shared/modules/factories.py:148-154"""
    return get_module_factory(desc or "standard", {"standard": Bias, "bias": Bias, "lazy_bias": LazyBias})


def get_gain_factory(desc):
    """The lazy variant is registered under 'lazy_bias', as in the reference
    (shared/modules/factories.py:157-163)."""
    return get_module_factory(desc or "standard", {"standard": Gain, "gain": Gain, "lazy_bias": LazyGain})


def get_activation_factory(desc):
    """shared/modules/factories.py:166-172"""
    assert desc is not None, "Must specify activation type"
    return get_module_factory(desc, {"relu": nn.ReLU, "leaky_relu": nn.LeakyReLU})


def get_norm_factory(desc):
    """shared/modules/factories.py:175-182"""
    assert desc is not None, "Must specify norm type"
    table = {"batch_norm_2d": nn.BatchNorm2d, "bn2d": nn.BatchNorm2d, "layer_norm": nn.LayerNorm, "ln": nn.LayerNorm,
             "pam_layer_norm": pam.LayerNorm, "pam_ln": pam.LayerNorm}
    return get_module_factory(desc, table)


_BY_TYPE = {"conv": get_conv_factory, "linear": get_linear_factory, "activation": get_activation_factory,
            "norm": get_norm_factory, "bias": get_bias_factory, "gain": get_gain_factory}


def get_sequential_factory(descriptions):
    """A list of typed descriptions becomes a factory of nn.Sequential; every member factory is
    called with the same keyword arguments and keeps those it accepts
    (shared/modules/factories.py:185-203)."""
    members = []
    for d in descriptions:
        if d["type"] not in _BY_TYPE:
            raise ValueError(f"Unknown factory type for {d}")
        members.append(_BY_TYPE[d["type"]](d))
    return lambda **kwargs: nn.Sequential(*[make(**kwargs) for make in members])


# ---------------------------------------------------------------- functional ops
_NAMES = ("mean", "mul", "div", "softmax", "bmm", "logsumexp", "log_softmax", "pow")


def _torch_ops():
    f = torch.nn.functional
    return dict(mean=torch.mean, mul=torch.mul, div=torch.div, softmax=f.softmax, bmm=torch.bmm,
                logsumexp=torch.logsumexp, log_softmax=f.log_softmax, pow=torch.pow)


def _pam_ops():
    return {name: getattr(pam, name) for name in _NAMES}


def get_function_dict(desc):
    """The table {'mean','mul','div','softmax','bmm','logsumexp','log_softmax','pow'} -> callable
    for 'standard' / 'torch', 'standard2' (base-2 torch), 'pam', 'pam_bmm_only',
    'pam_softmax_only', or a dict / YAML {'type': 'pam...', 'dkwargs': ..., 'okwargs': ...}
    whose entries filter their keywords (shared/modules/factories.py:216-298).  As in the
    reference, the dict form always maps every name to its PAM op."""
    if isinstance(desc, str):
        if desc in ("standard", "torch"):
            return _torch_ops()
        if desc == "standard2":
            return {**_torch_ops(), "softmax": pam_experimental.torch_softmax2,
                    "logsumexp": pam_experimental.torch_logsumexp2, "log_softmax": pam_experimental.torch_log_softmax2}
        if desc == "pam":
            return _pam_ops()
        if desc == "pam_bmm_only":
            return {**_torch_ops(), "bmm": pam.bmm}
        if desc == "pam_softmax_only":
            return {**_torch_ops(), "softmax": pam.softmax}
        try:
            desc = yaml.safe_load(desc)
        except Exception:
            raise ValueError(f"Unknown function config {desc}")
    assert isinstance(desc, dict), f"Unknown function cfg {desc=}"
    assert desc["type"] in ("pam", "pam_bmm_only", "pam_softmax_only"), "Only support custom cfg for pam"
    defaults = copy.copy(desc.get("dkwargs", {}))
    overrides = copy.copy(desc.get("okwargs", {}))

    def bind(func):
        return lambda *args, **kwargs: call_valid_kwargs(func, {**defaults, **kwargs, **overrides}, args)
    return {name: bind(func) for name, func in _pam_ops().items()}
