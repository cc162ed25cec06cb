"""Compositions of the PAM primitives: mean, softmax, logsumexp, log_softmax, layer_norm,
LayerNorm, conv2d, conv2d_group, Conv2d -- the rest of the reference's pam/pam_ops.py
(:118-257, 288-404).  Every multiply, divide, exp and log inside them is a PAM kernel call;
additions, subtractions, maxima and sums are ordinary fp32 torch operations, as in the
reference.  Same names and keyword arguments.

Reductions over the last dimension of a contiguous GPU tensor take the single-kernel path of
`pam_amd.fused` (softmax, logsumexp, log_softmax and layer_norm always, their gradients are single
kernels too; mean with the approximate gradient, or when no autograd graph is recorded); every other call runs the chain of primitive kernels written out below.  `fused_rows = False` switches
the single-kernel path off.  conv2d on GPU tensors runs on the matrix kernel with the image
patches read in place instead of unfolded (`implicit_conv = False` switches that off).
"""
import math

import torch

from . import fused
from .pam_ops import bmm, div, exp2, linear, log2, mul, pow

__all__ = ["mean", "softmax", "logsumexp", "log_softmax", "layer_norm", "LayerNorm",
           "conv2d", "conv2d_group", "Conv2d"]

_LOG2_E = math.log2(math.e)
fused_rows = True
implicit_conv = True


def _fused(x, dim, use_kernel, *grad_sources, kernel_gradient=True):
    """True when the call can run as one kernel: always if that kernel has its gradient, else only
    when none of grad_sources asks for one."""
    if not (fused_rows and use_kernel and fused.fusable(x, dim)):
        return False
    return kernel_gradient or not fused.needs_graph(*grad_sources)


def _pam_kwargs(offset, approx_bwd, use_kernel):
    return dict(offset=offset, approx_bwd=approx_bwd, use_kernel=use_kernel)


def mean(input, dim=None, keepdim=False, *, dtype=None, offset=None, approx_bwd=False, use_kernel=True):
    """Sum, then a PAM division by the element count (pam/pam_ops.py:288-302)."""
    if dim is None:
        dim = tuple(range(input.dim()))
    elif isinstance(dim, int):
        dim = (dim,)
    if dtype in (None, torch.float32) and _fused(input, dim, use_kernel, input, kernel_gradient=fused.mean_gradient_in_place(approx_bwd)):
        return fused.mean_last(input, keepdim, offset)
    count = math.prod(input.shape[d] for d in dim)
    total = torch.sum(input, dim=dim, keepdim=keepdim, dtype=dtype)
    return div(total, count, **_pam_kwargs(offset, approx_bwd, use_kernel))


def _scaled_exp2(x, kw, masked):
    """2 ** (x log2(e) - floor(max)), the shared front half of softmax and logsumexp."""
    scaled = mul(x, _LOG2_E, **kw)
    if masked is not None:
        # PAM products of infinities are NaN; -inf is what attention masks use
        scaled = torch.where(masked, float("-inf"), scaled)
    with torch.no_grad():
        shift = torch.floor(torch.max(scaled))          # one global shift, an integer: exact in exp2
    return exp2(scaled - shift, **kw), shift


def softmax(x, dim=None, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:305-328; -inf inputs give exactly zero weight."""
    if _fused(x, dim, use_kernel):
        return fused.softmax(x, offset, approx_bwd)
    kw = _pam_kwargs(offset, approx_bwd, use_kernel)
    masked = x == float("-inf")
    weights, _ = _scaled_exp2(x, kw, masked)
    weights = torch.where(masked, 0, weights)
    return div(weights, torch.sum(weights, dim=dim, keepdim=True), **kw)


def logsumexp(x, dim, keepdim=False, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:331-342; inputs must be finite."""
    kw = _pam_kwargs(offset, approx_bwd, use_kernel)
    assert x.isfinite().all()
    if _fused(x, dim, use_kernel, x):
        return fused.logsumexp(x, keepdim, offset, approx_bwd)
    weights, shift = _scaled_exp2(x, kw, None)
    total = torch.sum(weights, dim=dim, keepdim=keepdim)
    # the reference takes log2 of the total without its keyword arguments (pam/pam_ops.py:341): no offset there, and
    # that log2's gradient is the exact one whatever approx_bwd says
    return div(shift + log2(total), _LOG2_E, **kw)


def log_softmax(x, dim=None, *, offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:345-347"""
    if _fused(x, dim, use_kernel, x):
        assert x.isfinite().all()
        return fused.log_softmax(x, offset, approx_bwd)
    return x - logsumexp(x, dim=dim, keepdim=True, **_pam_kwargs(offset, approx_bwd, use_kernel))


def layer_norm(x, normalized_shape, weight=None, bias=None, eps=1e-05, *,
               offset=None, approx_bwd=False, use_kernel=True):
    """pam/pam_ops.py:350-378: mean and variance by PAM division, the square root as a PAM
    power, scaling by PAM products."""
    kw = _pam_kwargs(offset, approx_bwd, use_kernel)
    if isinstance(normalized_shape, int):
        normalized_shape = (normalized_shape,)
    assert x.shape[-len(normalized_shape):] == normalized_shape
    if _fused(x, -1, use_kernel, x, weight, bias) and all(
            t is None or (t.is_cuda and t.dtype == torch.float32) for t in (weight, bias)):
        return fused.layer_norm(x, math.prod(normalized_shape), weight, bias, eps, offset, approx_bwd)
    rows = x.reshape((-1, math.prod(normalized_shape)))
    centred = rows - mean(rows, dim=-1, keepdim=True, **kw)
    variance = mean(mul(centred, centred, **kw), dim=-1, keepdim=True, **kw)
    out = div(centred, pow(variance + eps, 0.5, **kw), **kw).reshape_as(x)
    if weight is not None:
        out = mul(out, weight, **kw)
    if bias is not None:
        out = out + bias
    return out


class LayerNorm(torch.nn.LayerNorm):
    """torch.nn.LayerNorm computed with PAM arithmetic; same parameters (pam/pam_ops.py:381-404)."""

    def __init__(self, *args, offset=None, approx_bwd=False, use_kernel=True, **kwargs):
        super().__init__(*args, **kwargs)
        self.offset = offset
        self.approx_bwd = approx_bwd
        self.use_kernel = use_kernel

    def forward(self, input):
        return layer_norm(input, self.normalized_shape, self.weight, self.bias, self.eps,
                          offset=self.offset, approx_bwd=self.approx_bwd, use_kernel=self.use_kernel)

    def _get_name(self):
        return "pam." + type(self).__name__

    def extra_repr(self):
        text = super().extra_repr()
        if self.offset is not None:
            text += f", offset={self.offset:0.5f}"
        text += f", approx_bwd={self.approx_bwd}"
        if self.use_kernel is not None:
            text += f", use_kernel={self.use_kernel}"
        return text


def _conv_geometry(in_hw, kernel_hw, stride, padding):
    """Resolves 'same'/'valid'/int padding and int stride; returns (padding, stride, out_hw)."""
    kh, kw = kernel_hw
    if isinstance(padding, str):
        if padding == "same":
            assert kh % 2 == 1 and kw % 2 == 1
            padding = ((kh - 1) // 2, (kw - 1) // 2)
        elif padding == "valid":
            padding = 0
        else:
            raise ValueError(f"Unknown {padding=}")
    if isinstance(padding, int):
        padding = (padding, padding)
    if isinstance(stride, int):
        stride = (stride, stride)
    out_hw = tuple((in_hw[i] + 2 * padding[i] - (kernel_hw[i] - 1) - 1) // stride[i] + 1 for i in (0, 1))
    return padding, stride, out_hw


def conv2d(X, W, bias=None, stride=1, padding=0, dilation=1, *, offset=None, approx_bwd=False, use_kernel=True):
    """Convolution as unfold + PAM linear (pam/pam_ops.py:118-160).  The output size assumes
    dilation 1, as the reference's does."""
    batch = X.shape[0]
    c_out, _, kh, kw = W.shape
    padding, stride, (h_out, w_out) = _conv_geometry(X.shape[2:], (kh, kw), stride, padding)
    if implicit_conv and use_kernel and fused.conv_in_place(X, W, dilation, approx_bwd, stride, padding):
        out = fused.conv2d(X, W, stride, padding, offset, approx_bwd)        # patches read in place
        return out if bias is None else out + bias.view((1, -1, 1, 1))
    patches = torch.nn.functional.unfold(X, (kh, kw), padding=padding, stride=stride, dilation=dilation)
    _, patch_len, locations = patches.shape                    # [N, C kh kw, L]
    rows = patches.transpose(1, 2).contiguous().view(-1, patch_len)
    out = linear(rows, W.view(c_out, -1), offset=offset, approx_bwd=approx_bwd, use_kernel=use_kernel)
    out = out.view(batch, locations, c_out).transpose(1, 2).view(batch, c_out, h_out, w_out)
    return out if bias is None else out + bias.view((1, -1, 1, 1))


def conv2d_group(X, W, bias=None, stride=1, padding=0, dilation=1, groups=1, *,
                 offset=None, approx_bwd=False, use_kernel=True):
    """Grouped convolution (pam/pam_ops.py:163-198: unfold + one PAM bmm over the groups); on the matrix kernel
    with the patches read in place where `fused.conv_in_place` allows."""
    batch, c_in = X.shape[:2]
    c_out, _, kh, kw = W.shape
    padding, stride, (h_out, w_out) = _conv_geometry(X.shape[2:], (kh, kw), stride, padding)
    if implicit_conv and use_kernel and c_in % groups == 0 and c_out % groups == 0 and fused.conv_in_place(
            X, W, dilation, approx_bwd, stride, padding, groups):
        out = fused.conv2d(X, W, stride, padding, offset, approx_bwd, groups)        # patches read in place, one product per group
        return out if bias is None else out + bias.view((1, -1, 1, 1))
    per_group = c_in // groups * kh * kw
    patches = torch.nn.functional.unfold(X, kernel_size=(kh, kw), padding=padding, stride=stride, dilation=dilation)
    patches = patches.view(batch, groups, per_group, -1).permute(1, 2, 0, 3).reshape(groups, per_group, -1)
    out = bmm(W.view(groups, c_out // groups, per_group), patches,
              offset=offset, approx_bwd=approx_bwd, use_kernel=use_kernel)
    out = out.view(c_out, batch, h_out, w_out).transpose(0, 1)
    return out if bias is None else out + bias.view((1, -1, 1, 1))


class Conv2d(torch.nn.Conv2d):
    """torch.nn.Conv2d computed with PAM products; same parameters (pam/pam_ops.py:201-257)."""

    def __init__(self, *args, offset=None, approx_bwd=False, use_kernel=True, **kwargs):
        super().__init__(*args, **kwargs)
        self.offset = offset
        self.approx_bwd = approx_bwd
        self.use_kernel = use_kernel

    def forward(self, input):
        kw = _pam_kwargs(self.offset, self.approx_bwd, self.use_kernel)
        if self.groups != 1:
            return conv2d_group(input, self.weight, self.bias, self.stride, self.padding, self.dilation,
                                self.groups, **kw)
        return conv2d(input, self.weight, self.bias, self.stride, self.padding, self.dilation, **kw)

    def _get_name(self):
        return "pam." + type(self).__name__

    def extra_repr(self):
        text = super().extra_repr()
        if self.offset is not None:
            text += f", offset={self.offset:0.5f}"
        return text + f", approx_bwd={self.approx_bwd}"
