"""Adam whose arithmetic comes from a functional op table, so that every product, the
quotient and the square root of the update can be PAM ops: the optimizer of the reference's
fully multiplication-free training recipe (the `Adam` class of
submodules/fairseq/fairseq/optim/adam.py:113-254 in the reference tree, selected there by
`opt_functional_cfg`).

With a PAM table and fp32 GPU tensors the whole update of a parameter is one kernel
(28 B/element instead of eleven elementwise launches); with any other table, or tensors
the kernel does not take, the same formulas run op by op through the table.  Both paths
give identical bits: the update has no reductions.
"""
import math

import torch
import yaml

from . import _abi
from .factories import get_function_dict

__all__ = ["Adam", "multiply_grads"]


def _pam_table_offset(cfg):
    """(True, offset) if cfg selects the PAM ops for 'mul', 'div' and 'pow'; else (False, None).
    The dict / YAML form maps every op to PAM whatever its 'type' says
    (shared/modules/factories.py:290-298)."""
    if isinstance(cfg, str):
        if cfg == "pam":
            return True, None
        if cfg in ("standard", "torch", "standard2", "pam_bmm_only", "pam_softmax_only"):
            return False, None
        try:
            cfg = yaml.safe_load(cfg)
        except Exception:
            return False, None
    if isinstance(cfg, dict) and str(cfg.get("type", "")).startswith("pam"):
        merged = {**cfg.get("dkwargs", {}), **cfg.get("okwargs", {})}
        if merged.get("use_kernel", True) is not True:
            return False, None
        return True, merged.get("offset")
    return False, None


class Adam(torch.optim.Optimizer):
    """Same constructor and state layout as the reference's class: state per parameter is
    {'step', 'exp_avg', 'exp_avg_sq'}; `amsgrad` is accepted and unsupported, as there."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, amsgrad=False,
                 opt_functional_cfg=None):
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad)
        self.op_dict = get_function_dict(opt_functional_cfg)
        self.fused, self.offset = _pam_table_offset(opt_functional_cfg)
        super().__init__(params, defaults)

    @property
    def supports_memory_efficient_fp16(self):
        return True

    @property
    def supports_flat_params(self):
        return True

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        ops = self.op_dict
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            for p in group["params"]:
                if p.grad is None:
                    continue
                grad = p.grad.data
                if grad.dtype in (torch.float16, torch.bfloat16):
                    grad = grad.float()
                if grad.is_sparse:
                    raise RuntimeError("Adam does not support sparse gradients, please consider SparseAdam instead")
                assert not group.get("amsgrad", False), "Not supported"
                half = p.data.dtype in (torch.float16, torch.bfloat16)
                p32 = p.data.float() if half else p.data

                state = self.state[p]
                if len(state) == 0:
                    state["step"] = 0
                    state["exp_avg"] = torch.zeros_like(p32)
                    state["exp_avg_sq"] = torch.zeros_like(p32)
                else:
                    state["exp_avg"] = state["exp_avg"].to(p32)
                    state["exp_avg_sq"] = state["exp_avg_sq"].to(p32)
                exp_avg, exp_avg_sq = state["exp_avg"], state["exp_avg_sq"]
                state["step"] += 1

                # scalar work on the host, in double precision
                correction1 = 1 - beta1 ** state["step"]
                correction2 = 1 - beta2 ** state["step"]
                step_size = group["lr"] * math.sqrt(correction2) / correction1
                decay = group["weight_decay"] * group["lr"] if group["weight_decay"] != 0 else None

                if (self.fused and p32.is_cuda and p32.dtype == torch.float32 and grad.dtype == torch.float32
                        and all(t.is_contiguous() for t in (p32, grad, exp_avg, exp_avg_sq))):
                    _abi.adam_step(p32, grad, exp_avg, exp_avg_sq, beta1, 1 - beta1, beta2, 1 - beta2, group["eps"],
                                   decay, step_size, 1.0 if self.offset is None else self.offset)
                else:
                    exp_avg.copy_(ops["mul"](exp_avg, beta1) + ops["mul"](grad, 1 - beta1))
                    exp_avg_sq.copy_(ops["mul"](exp_avg_sq, beta2))
                    exp_avg_sq += ops["mul"](ops["mul"](grad, grad), 1 - beta2)
                    denom = ops["pow"](exp_avg_sq, 0.5) + group["eps"]
                    if decay is not None:
                        p32 -= ops["mul"](p32, decay)
                    p32 -= ops["mul"](ops["div"](exp_avg, denom), step_size)
                if half:
                    p.data.copy_(p32)
        return loss


def multiply_grads(params, c, op_dict):
    """The gradient-scaling hook of the reference's optimizer wrapper
    (submodules/fairseq/fairseq/optim/fairseq_optimizer.py:103-119 in the reference tree): calls
    op_dict['mul'](grad, c) for every dense gradient and, like the reference, drops the result (its
    loop rebinds a local name), so dense gradients keep their values; sparse gradients are scaled in
    place with an ordinary multiply.  Kept for callers that rely on exactly that behaviour."""
    for p in params:
        if p.grad is None:
            continue
        cc = c.to(p.grad.device) if torch.is_tensor(c) else c
        if p.grad.is_sparse:
            p.grad.data.mul_(cc)
        else:
            op_dict["mul"](p.grad.data, cc)
