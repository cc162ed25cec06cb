"""Autograd layer over the HIP kernels.

Public names, signatures and gradient formulas are those of the reference's
pam/cuda_bindings.py, so `pam_ops` and the linear/functional hooks of the training
libraries bind to it unchanged.  `cuda_kernels` is the kernel object (the reference
JIT-compiles a CUDA extension at import, pam/cuda_bindings.py:15-25; here a prebuilt
shared library is loaded on first use).  Tests may swap `cuda_kernels` for another
object with the same fourteen methods.
"""
import math

import torch

from . import utils
from ._abi import HipKernels

cuda_kernels = HipKernels()


def _offset_value(offset):
    # None switches the offset off: multiplying by 1.0 adds nothing to the bit pattern
    # (pam/cuda_bindings.py:31-32)
    return 1.0 if offset is None else offset


def _both(approx_bwd):
    # one flag for both operands, or one per operand (pam/cuda_bindings.py:43-45)
    return (approx_bwd, approx_bwd) if isinstance(approx_bwd, bool) else tuple(approx_bwd)


paired_gradients = True      # False: one launch per gradient, as the reference's autograd functions do


def _pair_kernel(k, name, A, B):
    """Both gradients in one pass when the kernel object has that entry point and neither operand is a
    broadcast view (flattening it would materialise the copy the single-gradient path avoids)."""
    return paired_gradients and hasattr(k, name) and A.is_contiguous() and B.is_contiguous()


class pam_autograd(torch.autograd.Function):
    """C = A (*) B elementwise (pam/cuda_bindings.py:27-57)."""

    @staticmethod
    def forward(ctx, A, B, offset=None, approx_bwd=False):
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        ctx.save_for_backward(A, B)
        return cuda_kernels.pam_fwd(A, B, ctx.offset)

    @staticmethod
    def backward(ctx, delta_Y):
        A, B = ctx.saved_tensors
        k, off = cuda_kernels, ctx.offset
        approx_A, approx_B = _both(ctx.approx_bwd)
        dY = delta_Y.contiguous()
        need_A, need_B = ctx.needs_input_grad[:2]
        if need_A and need_B and _pair_kernel(k, "pam_bwd_pair", A, B):
            return (*k.pam_bwd_pair(A, B, dY, off, approx_A, approx_B), None, None)
        # approximate: treat PAM as a product, d/dA = B; exact: the slope of the affine piece
        delta_A = delta_B = None
        if need_A:
            delta_A = k.pam_fwd(dY, B, off) if approx_A else k.pam_bwd(A, B, dY, off)
        if need_B:
            delta_B = k.pam_fwd(dY, A, off) if approx_B else k.pam_bwd(B, A, dY, off)
        return delta_A, delta_B, None, None


def pam(A, B, *, offset=None, approx_bwd=False):
    A, B = utils.broadcast_tensors(A, B)
    return pam_autograd.apply(A, B, offset, approx_bwd)


class pad_autograd(torch.autograd.Function):
    """C = A (/) B elementwise (pam/cuda_bindings.py:66-97)."""

    @staticmethod
    def forward(ctx, A, B, offset=None, approx_bwd=False):
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        ctx.save_for_backward(A, B)
        return cuda_kernels.pad_fwd(A, B, ctx.offset)

    @staticmethod
    def backward(ctx, delta_Y):
        A, B = ctx.saved_tensors
        k, off = cuda_kernels, ctx.offset
        approx_A, approx_B = _both(ctx.approx_bwd)
        dY = delta_Y.contiguous()
        need_A, need_B = ctx.needs_input_grad[:2]
        if need_A and need_B and _pair_kernel(k, "pad_bwd_pair", A, B):
            return (*k.pad_bwd_pair(A, B, dY, off, approx_A, approx_B), None, None)

        delta_A = delta_B = None
        if need_A:
            inv_B = k.pad_fwd(torch.ones_like(B), B, off)        # 1 (/) B
            if approx_A:
                delta_A = k.pam_fwd(inv_B, dY, off)
            else:
                delta_A = k.pam_bwd(A, inv_B, dY, 1.0)
        if need_B:
            if approx_B:
                slope = k.pad_fwd(k.pad_fwd(A, B, off), B, off)  # (A (/) B) (/) B
                delta_B = -k.pam_fwd(slope, dY, off)
            else:
                delta_B = k.pad_bwd(A, B, dY, off)
        return delta_A, delta_B, None, None


def pad(A, B, *, offset=None, approx_bwd=False):
    A, B = utils.broadcast_tensors(A, B)
    return pad_autograd.apply(A, B, offset, approx_bwd)


def check_row_major(tensor, target_dim):
    """(tensor, True) if the last dim is contiguous, (tensor, False) if the one before it
    is, else a contiguous copy (pam/cuda_bindings.py:106-115).  No copy is made for
    transposed views, which is what keeps the backward products copy-free."""
    if tensor.dim() != target_dim:
        raise ValueError(f"{tensor.dim()=} is not equal to {target_dim=}")
    strides = tensor.stride()
    if strides[-1] == 1:
        return tensor, True
    if strides[-2] == 1:
        return tensor, False
    return tensor.contiguous(), True


class pam_matmul_autograd(torch.autograd.Function):
    """Y = A (x) B with PAM products, 2-D or batched (pam/cuda_bindings.py:118-166)."""

    @staticmethod
    def forward(ctx, A, B, offset=None, approx_bwd=False, BMM=False):
        nd = 3 if BMM else 2
        A, A_rm = check_row_major(A, nd)
        B, B_rm = check_row_major(B, nd)
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        ctx.BMM = BMM
        ctx.save_for_backward(A, B)
        fwd = cuda_kernels.pam_bmm_fwd if BMM else cuda_kernels.pam_matmul_fwd
        return fwd(A, B, A_rm, B_rm, ctx.offset)

    @staticmethod
    def backward(ctx, delta_Y):
        A, B = ctx.saved_tensors
        off, BMM = ctx.offset, ctx.BMM
        approx_A, approx_B = _both(ctx.approx_bwd)
        nd = 3 if BMM else 2
        fwd = cuda_kernels.pam_bmm_fwd if BMM else cuda_kernels.pam_matmul_fwd
        bwd = cuda_kernels.pam_bmm_bwd if BMM else cuda_kernels.pam_matmul_bwd

        dY, dY_rm = check_row_major(delta_Y, nd)
        At, At_rm = check_row_major(A.mT, nd)        # transposed views, not copies
        Bt, Bt_rm = check_row_major(B.mT, nd)

        # dA = dY (x) B^T and dB = A^T (x) dY; the exact variant weighs each product by the
        # slope of the forward operand's affine piece instead of multiplying
        if approx_A:
            delta_A = fwd(dY, Bt, dY_rm, Bt_rm, off)
        else:
            delta_A = bwd(dY, Bt, A, dY_rm, Bt_rm, True, off)
        if approx_B:
            delta_B = fwd(At, dY, At_rm, dY_rm, off)
        else:
            delta_B = bwd(At, dY, B, At_rm, dY_rm, False, off)
        return delta_A, delta_B, None, None, None


def pam_matmul(A, B, *, offset=None, approx_bwd=False):
    return pam_matmul_autograd.apply(A, B, offset, approx_bwd, False)


def pam_bmm(A, B, *, offset=None, approx_bwd=False):
    return pam_matmul_autograd.apply(A, B, offset, approx_bwd, True)


class standard_matmul_autograd(torch.autograd.Function):
    """Ordinary fp32 product through the same kernel, for calibration
    (pam/cuda_bindings.py:177-202)."""

    @staticmethod
    def forward(ctx, A, B, BMM=False):
        nd = 3 if BMM else 2
        A, A_rm = check_row_major(A, nd)
        B, B_rm = check_row_major(B, nd)
        ctx.BMM = BMM
        ctx.save_for_backward(A, B)
        fwd = cuda_kernels.standard_bmm if BMM else cuda_kernels.standard_matmul
        return fwd(A, B, A_rm, B_rm, 1.0)

    @staticmethod
    def backward(ctx, delta_Y):
        A, B = ctx.saved_tensors
        nd = 3 if ctx.BMM else 2
        fwd = cuda_kernels.standard_bmm if ctx.BMM else cuda_kernels.standard_matmul
        dY, dY_rm = check_row_major(delta_Y, nd)
        At, At_rm = check_row_major(A.mT, nd)
        Bt, Bt_rm = check_row_major(B.mT, nd)
        return fwd(dY, Bt, dY_rm, Bt_rm, 1.0), fwd(At, dY, At_rm, dY_rm, 1.0), None


def standard_matmul(A, B, *, offset=None, approx_bwd=None, BMM=False):
    # offset and approx_bwd are accepted and ignored (pam/cuda_bindings.py:205-207)
    return standard_matmul_autograd.apply(A, B, BMM)


class pa_exp_autograd(torch.autograd.Function):
    """Y = base ** X, piecewise affine (pam/cuda_bindings.py:210-239)."""

    @staticmethod
    def forward(ctx, X, base, offset=None, approx_bwd=False):
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        ctx.base = base
        ctx.save_for_backward(X)
        return cuda_kernels.pa_exp_fwd(X, base, ctx.offset)

    @staticmethod
    def backward(ctx, delta_Y):
        X, = ctx.saved_tensors
        k, off, base = cuda_kernels, ctx.offset, ctx.base
        if not ctx.approx_bwd:
            return k.pa_exp_bwd(X, delta_Y, base, off), None, None, None
        # d/dx base**x = base**x ln(base), every product a PAM product
        grad = k.pa_exp_fwd(X, base, off)
        if base != math.e:
            grad = k.pam_fwd(grad, torch.full_like(X, math.log(base)), off)
        return k.pam_fwd(grad, delta_Y, off), None, None, None


def pa_exp(X, *, base=math.e, offset=None, approx_bwd=False):
    return pa_exp_autograd.apply(X, base, offset, approx_bwd)


def pa_exp2(X, *, offset=None, approx_bwd=False):
    return pa_exp_autograd.apply(X, 2.0, offset, approx_bwd)


class pa_log_autograd(torch.autograd.Function):
    """Y = log_base X, piecewise affine (pam/cuda_bindings.py:250-276)."""

    @staticmethod
    def forward(ctx, X, base, offset=None, approx_bwd=False):
        ctx.offset = _offset_value(offset)
        ctx.approx_bwd = approx_bwd
        ctx.base = base
        ctx.save_for_backward(X)
        return cuda_kernels.pa_log_fwd(X, base, ctx.offset)

    @staticmethod
    def backward(ctx, delta_Y):
        X, = ctx.saved_tensors
        k, off, base = cuda_kernels, ctx.offset, ctx.base
        if not ctx.approx_bwd:
            return k.pa_log_bwd(X, delta_Y, base, off), None, None, None
        # d/dx log_base x = 1 / (x ln(base)), every quotient a PAM quotient
        grad = k.pad_fwd(delta_Y, X, off)
        if base != math.e:
            grad = k.pad_fwd(grad, torch.full_like(X, math.log(base)), off)
        return grad, None, None, None


def pa_log(X, *, base=math.e, offset=None, approx_bwd=False):
    return pa_log_autograd.apply(X, base, offset, approx_bwd)


def pa_log2(X, *, offset=None, approx_bwd=False):
    return pa_log_autograd.apply(X, 2.0, offset, approx_bwd)
