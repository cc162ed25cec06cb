"""Cross entropy whose gradient is computed with a configurable set of ops
(the reference's pam/pam_opt.py:6-63): the forward value is always the ordinary
torch cross entropy, so that losses stay comparable between runs; the backward pass is
softmax(X) - target, scaled, with `softmax`, `mul` and `div` taken from `op_dict`
(for instance the PAM set of `pam_amd.factories.get_function_dict('pam')`).
"""
import torch

__all__ = ["cross_entropy", "cross_entropy_autograd"]


class cross_entropy_autograd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, X, Y, weight=None, ignore_index=None, reduction="mean", label_smoothing=0.0, op_dict=None):
        assert op_dict is not None, "OP dict must be explicitly specified"
        ctx.save_for_backward(X, Y, weight)
        ctx.settings = (ignore_index, reduction, label_smoothing, op_dict)
        return torch.nn.functional.cross_entropy(input=X, target=Y, weight=weight, ignore_index=ignore_index,
                                                 reduction=reduction, label_smoothing=label_smoothing)

    @staticmethod
    def backward(ctx, delta_output):
        X, Y, weight = ctx.saved_tensors
        ignore_index, reduction, label_smoothing, ops = ctx.settings
        prob = ops["softmax"](X, dim=-1)
        ignored = None
        if ignore_index is not None:
            ignored = Y.eq(ignore_index)
            Y = Y.masked_fill(ignored, 0)                   # a valid class; its rows are zeroed below
        target = torch.nn.functional.one_hot(Y, num_classes=X.shape[-1]).float()
        if label_smoothing:
            target = target * (1 - label_smoothing)
            target = target + (label_smoothing / X.shape[-1]) * torch.ones_like(target)
        delta = prob - target
        if weight is not None:
            delta = ops["mul"](delta, weight[Y].view(-1, 1))
        if ignored is not None:
            delta = delta * (~ignored.view(-1, 1))          # times 0 or 1: exact
        if reduction == "mean":
            delta = ops["div"](delta, X.shape[0])
        delta = ops["mul"](delta, delta_output.view(-1, 1))
        return (delta,) + (None,) * 6


def cross_entropy(X, Y, weight=None, ignore_index=None, reduction="mean", label_smoothing=0.0, *, op_dict=None):
    """Always the approximate backward: the gradient formula is the analytic one (pam/pam_opt.py:54-63)."""
    return cross_entropy_autograd.apply(X, Y, weight, ignore_index, reduction, label_smoothing, op_dict)
