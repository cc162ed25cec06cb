"""User-facing op library: the part of the reference's pam/pam_ops.py that sits on the
GPU hot path (mul, div, exp, exp2, log, log2, pow, matmul, bmm, linear, Linear), same
names and keyword arguments (`offset`, `approx_bwd`, `use_kernel`).

Everything runs on the HIP kernels.  The reference falls back to a float emulation
built from torch primitives for CPU tensors or `use_kernel=False` (pam/pam_ops.py:18-21);
this package has no such fallback and raises instead.
"""
import math

import torch

from . import cuda_bindings
from . import fused
from . import utils

__all__ = ["mul", "div", "exp", "exp2", "log", "log2", "pow", "matmul", "bmm", "linear", "Linear"]

fused_bias = True        # False: linear() adds the bias with a separate torch add, as the reference does
fused_pow = True         # False: pow() with a number as exponent runs the chain of log2, product, exp2 and select


def _require_kernel(t, use_kernel):
    if not use_kernel:
        raise NotImplementedError("pam_amd runs on the HIP kernels only; use_kernel=False has no implementation here")
    if not t.is_cuda:
        raise RuntimeError("pam_amd computes on the GPU only: move the tensor to the device first")


def mul(A, B, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:16-22"""
    tA, tB = utils.to_tensor(A, B)
    _require_kernel(tA, use_kernel)
    out = cuda_bindings.pam(tA, tB, offset=offset, approx_bwd=approx_bwd)
    return utils.demote_tensor(out, (A, B))


def div(A, B, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:25-31"""
    tA, tB = utils.to_tensor(A, B)
    _require_kernel(tA, use_kernel)
    out = cuda_bindings.pad(tA, tB, offset=offset, approx_bwd=approx_bwd)
    return utils.demote_tensor(out, (A, B))


def exp(A, base=math.e, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:34-40"""
    tA, = utils.to_tensor(A)
    _require_kernel(tA, use_kernel)
    out = cuda_bindings.pa_exp(tA, base=base, offset=offset, approx_bwd=approx_bwd)
    return utils.demote_tensor(out, (A,))


def exp2(A, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:43-49"""
    tA, = utils.to_tensor(A)
    _require_kernel(tA, use_kernel)
    out = cuda_bindings.pa_exp2(tA, offset=offset, approx_bwd=approx_bwd)
    return utils.demote_tensor(out, (A,))


def log(A, base=math.e, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:52-58"""
    tA, = utils.to_tensor(A)
    _require_kernel(tA, use_kernel)
    out = cuda_bindings.pa_log(tA, base=base, offset=offset, approx_bwd=approx_bwd)
    return utils.demote_tensor(out, (A,))


def log2(A, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:61-67"""
    tA, = utils.to_tensor(A)
    _require_kernel(tA, use_kernel)
    out = cuda_bindings.pa_log2(tA, offset=offset, approx_bwd=approx_bwd)
    return utils.demote_tensor(out, (A,))


def pow(A, B, *, offset=None, approx_bwd=False, use_kernel=True):
    """A ** B as exp2(log2(A) (*) B), zero where A is zero (pam/pam_ops.py:70-79)."""
    if fused_pow and use_kernel and fused.pow_in_place(A, B):
        return fused.pow_scalar(A, B, offset, approx_bwd)             # one pass, and one for the gradient
    tA, tB = utils.to_tensor(A, B)
    kw = dict(offset=offset, approx_bwd=approx_bwd, use_kernel=use_kernel)
    out = torch.where(tA == 0, 0, exp2(mul(log2(tA, **kw), tB, **kw), **kw))
    return utils.demote_tensor(out, (A, B))


def matmul(A, B, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:82-86"""
    _require_kernel(A, use_kernel)
    return cuda_bindings.pam_matmul(A, B, offset=offset, approx_bwd=approx_bwd)


def bmm(A, B, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:89-104"""
    assert A.dim() == B.dim() == 3
    assert A.shape[0] == B.shape[0]
    assert A.shape[2] == B.shape[1]
    _require_kernel(A, use_kernel)
    return cuda_bindings.pam_bmm(A, B, offset=offset, approx_bwd=approx_bwd)


def linear(X, W, bias=None, *, offset=None, approx_bwd=False, use_kernel=True):
    """X W^T + bias with PAM products; leading dims are flattened like torch.nn.Linear
    (pam/pam_ops.py:107-115).  W.T is passed as a view: the kernel reads W in place."""
    lead = X.shape[:-1]
    rows = X.reshape(-1, X.shape[-1])
    if (fused_bias and bias is not None and use_kernel and rows.is_cuda and rows.numel() and bias.dim() == 1
            and all(t.dtype == torch.float32 for t in (rows, W, bias))):
        # the bias is added to the finished sums inside the product kernel: the same add, one pass less
        out = fused.linear_with_bias(rows, W, bias, offset, approx_bwd)
        return out.reshape(*lead, out.shape[-1])
    out = matmul(rows, W.T, offset=offset, approx_bwd=approx_bwd, use_kernel=use_kernel)
    out = out.reshape(*lead, out.shape[-1])
    return out if bias is None else out + bias


class Linear(torch.nn.Linear):
    """torch.nn.Linear with PAM products; same parameters and state_dict
    (pam/pam_ops.py:259-285)."""

    def __init__(self, *args, offset=None, approx_bwd=False, use_kernel=True, **kwargs):
        super().__init__(*args, **kwargs)
        self.offset = offset
        self.approx_bwd = approx_bwd
        self.use_kernel = use_kernel

    def forward(self, input):
        return linear(input, self.weight, self.bias,
                      offset=self.offset, approx_bwd=self.approx_bwd, use_kernel=self.use_kernel)

    def _get_name(self):
        return "pam." + type(self).__name__

    def extra_repr(self):
        parts = [f"in_features={self.in_features}", f"out_features={self.out_features}",
                 f"bias={self.bias is not None}"]
        if self.offset is not None:
            parts.append(f"offset={self.offset:0.5f}")
        parts.append(f"approx_bwd={self.approx_bwd}")
        return ", ".join(parts)


def __getattr__(name):
    # The reference keeps conv2d, conv2d_group, Conv2d, mean, softmax, logsumexp, log_softmax, layer_norm and LayerNorm in
    # this module too (pam/pam_ops.py:118-404); here they live in `composites`, which imports this module, so they are
    # looked up on first use: `pam.pam_ops.softmax` and `from pam.pam_ops import LayerNorm` work as they do there.
    from . import composites
    if name in composites.__all__:
        return getattr(composites, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
