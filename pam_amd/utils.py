"""Scalar/tensor plumbing of the op library (counterpart of the reference's pam/utils.py)."""
import torch


def to_tensor(*values, device=None):
    """Python numbers become fp32 tensors on the device the tensor arguments live on
    (pam/utils.py:3-16).  Tensors pass through; mixing devices is an error."""
    for v in values:
        if isinstance(v, torch.Tensor):
            if device is not None and device != v.device:
                raise AssertionError(f"Mismatching devices {device=}, {v.device=}")
            device = v.device
    return [torch.tensor(v, device=device, dtype=torch.float32) if isinstance(v, (int, float)) else v
            for v in values]


def broadcast_tensors(*tensors):
    """pam/utils.py:19-20"""
    return torch.broadcast_tensors(*to_tensor(*tensors))


def demote_tensor(out_value, in_values):
    """A result computed from Python numbers only goes back to a Python number (pam/utils.py:23-27)."""
    if all(isinstance(v, (float, int)) for v in in_values):
        return out_value.item()
    return out_value
