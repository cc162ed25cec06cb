"""Row-wise compositions as single kernels: softmax (with its gradient), logsumexp,
log_softmax, the mean over the last dimension and layer_norm.

Each computes, element for element, what the compositions of `pam_amd.composites` compute
from the primitive kernels (the reference's pam/pam_ops.py:288-378), in one sweep over the
rows instead of five to fifteen elementwise launches.  The only difference is the order of
the row sums, which the reference leaves to torch.sum and the kernels fix.

`row_kernels` is the kernel object; tests may swap it for another object with the same
five methods.  `fusable` says whether a call can take this path: float32 GPU tensor,
contiguous, reduced dimension last, not empty.
"""
import torch

from . import _abi
from . import cuda_bindings
from ._abi import HipRowKernels
from .cuda_bindings import _both, _offset_value

row_kernels = HipRowKernels()


def fusable(x, dim):
    if not (isinstance(x, torch.Tensor) and x.is_cuda and x.dtype == torch.float32):
        return False
    if x.dim() < 1 or x.numel() == 0 or not x.is_contiguous():
        return False
    if isinstance(dim, (tuple, list)):
        if len(dim) != 1:
            return False
        dim = dim[0]
    return isinstance(dim, int) and dim in (-1, x.dim() - 1)


def _wants_grad(*tensors):
    return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


class softmax_autograd(torch.autograd.Function):
    """softmax over the last dimension; the gradient is the chain of the primitives'
    gradients (pam/cuda_bindings.py:43-57, 78-97, 224-239) in one kernel."""

    @staticmethod
    def forward(ctx, x, offset=None, approx_bwd=False):
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        rows = x.reshape(-1, x.shape[-1])
        y, row_sum, shift = row_kernels.softmax_fwd(rows, ctx.offset)
        ctx.save_for_backward(rows, row_sum, shift)
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, grad):
        rows, row_sum, shift = ctx.saved_tensors
        g = grad.contiguous().view(rows.shape)
        dx = row_kernels.softmax_bwd(rows, g, row_sum, shift, ctx.offset, *_flags(ctx.approx_bwd))
        return dx.view(grad.shape), None, None


def softmax(x, offset=None, approx_bwd=False):
    return softmax_autograd.apply(x, offset, approx_bwd)


def _flags(approx_bwd):
    """(first operands, second operands, exp / log): the last tests the flag's truth value, so a
    pair counts as set (pam/cuda_bindings.py:227, 267)."""
    a, b = _both(approx_bwd)
    return a, b, bool(approx_bwd)


def needs_graph(*tensors):
    return _wants_grad(*tensors)


class logsumexp_autograd(torch.autograd.Function):
    """logsumexp (as_log_softmax False) or log_softmax = x - logsumexp(x) over the last dimension."""

    @staticmethod
    def forward(ctx, x, offset, approx_bwd, as_log_softmax, keepdim):
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        ctx.as_log_softmax = as_log_softmax
        rows = x.reshape(-1, x.shape[-1])
        lse, y, shift = row_kernels.logsumexp_fwd(rows, ctx.offset, not as_log_softmax, as_log_softmax)
        ctx.save_for_backward(rows, shift)
        if as_log_softmax:
            return y.view(x.shape)
        return lse.view(x.shape[:-1] + ((1,) if keepdim else ()))

    @staticmethod
    def backward(ctx, grad):
        rows, shift = ctx.saved_tensors
        g = grad.contiguous().view(rows.shape if ctx.as_log_softmax else (rows.shape[0],))
        dx = row_kernels.logsumexp_bwd(rows, g, shift, ctx.offset, *_flags(ctx.approx_bwd), ctx.as_log_softmax)
        return dx, None, None, None, None


def logsumexp(x, keepdim, offset=None, approx_bwd=False):
    out = logsumexp_autograd.apply(x.reshape(-1, x.shape[-1]), offset, approx_bwd, False, True)
    return out.view(x.shape[:-1] + ((1,) if keepdim else ()))


def log_softmax(x, offset=None, approx_bwd=False):
    return logsumexp_autograd.apply(x.reshape(-1, x.shape[-1]), offset, approx_bwd, True, True).view(x.shape)


class mean_autograd(torch.autograd.Function):
    """Row mean = (fixed-order row sum) (/) n with the approximate gradient of the quotient
    (pam/cuda_bindings.py:86-87): every element of a row receives (1 (/) n) (*) g."""

    @staticmethod
    def forward(ctx, rows, offset):
        ctx.offset, ctx.n = _offset_value(offset), rows.shape[1]
        return row_kernels.row_mean_fwd(rows, ctx.offset)

    @staticmethod
    def backward(ctx, g):
        k = cuda_bindings.cuda_kernels
        g = g.contiguous().view(-1)
        count = torch.full((1,), float(ctx.n), dtype=torch.float32, device=g.device).expand_as(g)
        inv = k.pad_fwd(torch.ones((1,), dtype=torch.float32, device=g.device).expand_as(g), count, ctx.offset)
        return k.pam_fwd(inv, g, ctx.offset).unsqueeze(1).expand(-1, ctx.n), None


def mean_gradient_in_place(approx_bwd):
    """The single-kernel mean carries the approximate gradient only (the exact one needs the row sum as the
    forward pass rounded it)."""
    return bool(_both(approx_bwd)[0])


def mean_last(x, keepdim, offset=None):
    y = mean_autograd.apply(x.reshape(-1, x.shape[-1]), offset)
    return y.view(x.shape[:-1] + ((1,) if keepdim else ()))


class layer_norm_autograd(torch.autograd.Function):
    """layer_norm over the last n values of each row; weight and bias of n values or None."""

    @staticmethod
    def forward(ctx, rows, weight, bias, eps, offset, approx_bwd):
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        ctx.eps = eps
        ctx.has_bias = bias is not None
        w = None if weight is None else weight.contiguous().view(-1)
        b = None if bias is None else bias.contiguous().view(-1)
        ctx.save_for_backward(rows, w)
        return row_kernels.layer_norm_fwd(rows, w, b, eps, ctx.offset)

    @staticmethod
    def backward(ctx, grad):
        rows, w = ctx.saved_tensors
        g = grad.contiguous()
        want_w = w is not None and ctx.needs_input_grad[1]
        dx, terms = row_kernels.layer_norm_bwd(rows, w, g, ctx.eps, ctx.offset, *_flags(ctx.approx_bwd), want_w)
        # the broadcast weight and bias collect their gradients by a sum over the rows, as autograd's expand does
        dw = terms.sum(0) if want_w else None
        db = g.sum(0) if (ctx.has_bias and ctx.needs_input_grad[2]) else None
        return dx, dw, db, None, None, None


def layer_norm(x, n, weight, bias, eps, offset=None, approx_bwd=False):
    w = None if weight is None else weight.reshape(-1)
    b = None if bias is None else bias.reshape(-1)
    out = layer_norm_autograd.apply(x.reshape(-1, n), w, b, eps, offset, approx_bwd)
    return out.view(x.shape)


# ---------------------------------------------------------------- power with a scalar exponent

class pow_autograd(torch.autograd.Function):
    """A ** p for a number p: log2, product, exp2 and the select of zeros (pam/pam_ops.py:70-79)
    in one pass, and the gradient those ops' backward formulas chain to in another."""

    @staticmethod
    def forward(ctx, A, exponent, offset, approx_bwd):
        ctx.exponent, ctx.offset, ctx.approx_bwd = float(exponent), _offset_value(offset), approx_bwd
        ctx.save_for_backward(A)
        return _abi.pow_fwd(A, ctx.exponent, ctx.offset)

    @staticmethod
    def backward(ctx, dY):
        A, = ctx.saved_tensors
        approx_a, _, approx_exp = _flags(ctx.approx_bwd)
        return _abi.pow_bwd(A, dY.contiguous(), ctx.exponent, ctx.offset, approx_a, approx_exp), None, None, None


def pow_in_place(A, B):
    """fp32 GPU tensor to the power of a plain number."""
    return (isinstance(A, torch.Tensor) and A.is_cuda and A.dtype == torch.float32
            and isinstance(B, (int, float)) and not isinstance(B, bool))


def pow_scalar(A, exponent, offset=None, approx_bwd=False):
    return pow_autograd.apply(A, exponent, offset, approx_bwd)


# ---------------------------------------------------------------- convolution on image patches read in place

def input_gradient_in_place(W, stride, padding):
    """The gradient of the input is a stride-1 convolution of the upstream gradient when the
    forward stride is 1 and the padding does not exceed kernel - 1."""
    return tuple(stride) == (1, 1) and padding[0] <= W.shape[2] - 1 and padding[1] <= W.shape[3] - 1


def conv_in_place(X, W, dilation, approx_bwd, stride=(1, 1), padding=(0, 0), groups=1):
    """True when conv2d can run on the matrix kernel without unfolding X: fp32 GPU tensors,
    dilation 1, and, if the exact gradient with respect to X is wanted, a geometry for which that
    gradient is a convolution in place too (otherwise it needs the patches as a stored operand)."""
    if not (isinstance(X, torch.Tensor) and isinstance(W, torch.Tensor) and X.is_cuda and W.is_cuda):
        return False
    if X.dtype != torch.float32 or W.dtype != torch.float32 or X.dim() != 4 or W.dim() != 4 or X.numel() == 0:
        return False
    if dilation not in (1, (1, 1), [1, 1]):
        return False
    wants_dx = torch.is_grad_enabled() and X.requires_grad
    if groups != 1:          # grouped: the input gradient has no unfolded fallback here, it must be a convolution itself
        return not wants_dx or input_gradient_in_place(W, stride, padding)
    approx_x, _ = _both(approx_bwd)
    return approx_x or not wants_dx or input_gradient_in_place(W, stride, padding)


class conv2d_autograd(torch.autograd.Function):
    """conv2d as W (x) patches(X) per image.  The reference's product is patches (x) W^T
    (pam/pam_ops.py:118-160); PAM products commute, and the offset, which the reference folds
    into the weights, is applied to them before the product, so every term is the same."""

    @staticmethod
    def forward(ctx, X, W, stride, padding, offset, approx_bwd, groups=1):
        ctx.stride, ctx.padding, ctx.groups = stride, padding, groups
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        ctx.save_for_backward(X, W)
        return _abi.conv2d_fwd(X, W, stride, padding, ctx.offset, groups)

    @staticmethod
    def backward(ctx, dY):
        X, W = ctx.saved_tensors
        approx_x, approx_w = _both(ctx.approx_bwd)       # the reference's A is the patch matrix, its B the weights
        k, off = cuda_bindings.cuda_kernels, ctx.offset
        dY = dY.contiguous()
        dX = dW = None
        if ctx.needs_input_grad[1]:
            per_image = _abi.conv2d_bwd_weight(X, dY, W, ctx.stride, ctx.padding, not approx_w, off, ctx.groups)
            dW = per_image.sum(0).view(W.shape)
        if ctx.needs_input_grad[0] and input_gradient_in_place(W, ctx.stride, ctx.padding):
            dX = _abi.conv2d_bwd_input(dY, W, X, ctx.padding, not approx_x, off, ctx.groups)
        elif ctx.needs_input_grad[0]:
            if not approx_x or ctx.groups != 1:
                raise RuntimeError("this gradient with respect to the convolution input needs the unfolded path")
            batch, co = dY.shape[:2]
            W2 = W.reshape(co, -1)
            if off != 1.0:
                W2 = k.pam_fwd(W2, torch.tensor(off, dtype=torch.float32, device=W.device).expand_as(W2), 1.0)
            # gradient of the patch matrix, then the overlap-add that is unfold's gradient
            d_patches = k.pam_bmm_fwd(W2.t().unsqueeze(0).expand(batch, -1, -1), dY.view(batch, co, -1), False, True, 1.0)
            dX = torch.nn.functional.fold(d_patches, X.shape[2:], W.shape[2:], padding=ctx.padding, stride=ctx.stride)
        return dX, dW, None, None, None, None, None


def conv2d(X, W, stride, padding, offset=None, approx_bwd=False, groups=1):
    return conv2d_autograd.apply(X, W, tuple(stride), tuple(padding), offset, approx_bwd, groups)


# ---------------------------------------------------------------- linear with the bias added in the product's epilogue

class linear_autograd(torch.autograd.Function):
    """X W^T + bias in one kernel; the gradients are those of the product
    (pam/cuda_bindings.py:132-166) and, for the bias, the sum of the upstream gradient over the rows."""

    @staticmethod
    def forward(ctx, X, W, bias, offset, approx_bwd):
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        X2, _ = cuda_bindings.check_row_major(X, 2)
        Wt, _ = cuda_bindings.check_row_major(W.t(), 2)
        ctx.save_for_backward(X2, Wt)
        return _abi.linear_fwd(X2, Wt, bias.contiguous(), ctx.offset)

    @staticmethod
    def backward(ctx, dY):
        A, B = ctx.saved_tensors                      # A = X, B = W^T as the product saw them
        k, off = cuda_bindings.cuda_kernels, ctx.offset
        approx_a, approx_b = _both(ctx.approx_bwd)
        crm = cuda_bindings.check_row_major
        dY2, dY_rm = crm(dY, 2)
        At, At_rm = crm(A.mT, 2)
        Bt, Bt_rm = crm(B.mT, 2)
        dX = dW = db = None
        if ctx.needs_input_grad[0]:
            dX = k.pam_matmul_fwd(dY2, Bt, dY_rm, Bt_rm, off) if approx_a else k.pam_matmul_bwd(dY2, Bt, A, dY_rm, Bt_rm, True, off)
        if ctx.needs_input_grad[1]:
            dB = k.pam_matmul_fwd(At, dY2, At_rm, dY_rm, off) if approx_b else k.pam_matmul_bwd(At, dY2, B, At_rm, dY_rm, False, off)
            dW = dB.t()
        if ctx.needs_input_grad[2]:
            db = dY2.sum(0)
        return dX, dW, db, None, None


def linear_with_bias(X2d, W, bias, offset=None, approx_bwd=False):
    return linear_autograd.apply(X2d, W, bias, offset, approx_bwd)
