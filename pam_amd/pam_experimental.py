"""Base-2 softmax / logsumexp / log_softmax / cross entropy in ordinary torch arithmetic:
the "standard2" comparison functions of the reference (pam/pam_experimental.py:4-59).  They
use the same global floor(max) shift as the PAM versions but exact exp2, log2 and division,
which isolates the effect of the change of base from the effect of PAM.  No PAM kernel is
involved; they run wherever their tensors live.
"""
import torch

__all__ = ["torch_softmax2", "torch_logsumexp2", "torch_log_softmax2", "torch_cross_entropy2"]


def _shifted_exp2(x, dtype):
    if dtype is not None:
        x = x.to(dtype=dtype)
    with torch.no_grad():
        shift = torch.max(x).floor()
    return x, torch.exp2(x - shift), shift


def torch_softmax2(x, dim=None, dtype=None):
    """pam/pam_experimental.py:4-14"""
    _, weights, _ = _shifted_exp2(x, dtype)
    return weights / weights.sum(dim=dim, keepdim=True)


def torch_logsumexp2(x, dim=None, keepdim=None, dtype=None):
    """pam/pam_experimental.py:17-25; keepdim=None (the reference's default, which torch.sum
    rejects) counts as False."""
    _, weights, shift = _shifted_exp2(x, dtype)
    return torch.log2(weights.sum(dim=dim, keepdim=bool(keepdim))) + shift


def torch_log_softmax2(x, dim=None, dtype=None):
    """pam/pam_experimental.py:28-31"""
    if dtype is not None:
        x = x.to(dtype=dtype)
    return x - torch_logsumexp2(x, dim=dim, keepdim=True)


def torch_cross_entropy2(x, target, weight=None, ignore_index=-100, reduction="mean", label_smoothing=0.0):
    """Cross entropy on base-2 log-probabilities from a dense (smoothed) one-hot target
    (pam/pam_experimental.py:34-59).  As in the reference the logsumexp is taken without
    keepdim, so the input is expected as [classes] or with a broadcastable leading shape."""
    log_prob = x - torch_logsumexp2(x, dim=-1)
    ignored = None
    if ignore_index is not None:
        ignored = target.eq(ignore_index)
        target = target.masked_fill(ignored, 0)            # any valid class: the term is zeroed below
    dense = torch.nn.functional.one_hot(target, num_classes=x.shape[-1]).float()
    if label_smoothing:
        dense = dense * (1 - label_smoothing)
        dense = dense + (label_smoothing / x.shape[-1]) * torch.ones_like(dense)
    terms = -log_prob * dense
    if ignored is not None:
        terms = terms * (~ignored.view(-1, 1))
    if weight is not None:
        terms = terms * weight.view(-1, 1)
    loss = terms.sum(dim=-1)
    if reduction == "mean":
        return loss.mean()
    if reduction == "sum":
        return loss.sum()
    if reduction is not None:
        raise ValueError("Unknown reduction")
    return loss
