"""Adam with PAM arithmetic: the oracle's restatement against the chain of primitive calls
(bit for bit: the update has no reductions), the optimizer's op-by-op path on the CPU with
the oracle-backed kernel object, and on the GPU the single kernel against both."""
import math

import numpy as np
import pytest
import torch

import pam_amd
from pam_amd import cuda_bindings, optim, pam_ops
from _util import assert_same_bits, mixed_operands
from test_host_api import OracleKernels

OFF = 1.0552


def chain(o, p, g, m, v, b1, b2, eps, decay, step_size, off=None):
    """fairseq/optim/adam.py:226-252 of the reference tree, from the oracle primitives."""
    f = np.float32
    m1 = (o.pam(m, f(b1), off) + o.pam(g, f(1 - b1), off)).astype(f)
    v1 = o.pam(v, f(b2), off)
    v1 = (v1 + o.pam(o.pam(g, g, off), f(1 - b2), off)).astype(f)
    root = np.where(v1 == 0, 0, o.pa_exp(o.pam(o.pa_log(v1, 2.0, off), f(0.5), off), 2.0, off)).astype(f)
    denom = (root + f(eps)).astype(f)
    if decay:
        p = (p - o.pam(p, f(decay), off)).astype(f)
    p1 = (p - o.pam(o.pad(m1, denom, off), f(step_size), off)).astype(f)
    return p1, m1, v1


def operands(n, seed):
    rng = np.random.RandomState(seed)
    p = rng.standard_normal(n).astype(np.float32)
    g = (rng.standard_normal(n) * 1e-2).astype(np.float32)
    m = (rng.standard_normal(n) * 1e-2).astype(np.float32)
    v = (rng.standard_normal(n) ** 2 * 1e-4).astype(np.float32)
    g[:8] = [0.0, -0.0, 1e-30, 1e-41, 3e38, -3e38, np.inf, np.nan]     # zero, tiny, subnormal, huge, non-finite gradients
    v[8:12] = 0.0; g[8:12] = 0.0                                           # untouched moments: pow's zero branch
    return p, g, m, v


@pytest.mark.parametrize("off", [None, OFF])
@pytest.mark.parametrize("decay", [None, 1e-4 * 5e-4])
def test_oracle_adam_is_the_chain(oracle, off, decay):
    p, g, m, v = operands(4099, 0)
    step_size = 5e-4 * math.sqrt(1 - 0.98 ** 3) / (1 - 0.9 ** 3)
    got = oracle.adam_step(p, g, m, v, 0.9, 1 - 0.9, 0.98, 1 - 0.98, 1e-8, decay, step_size, off)
    want = chain(oracle, p, g, m, v, 0.9, 0.98, 1e-8, decay, step_size, off)
    for a, b, name in zip(got, want, ("p", "exp_avg", "exp_avg_sq")):
        assert_same_bits(a, b, name)
    assert np.isfinite(got[0][12:]).all()


def test_adam_moves_towards_the_ordinary_adam(oracle):
    """PAM products are within -11.1 % of true products, so one step stays close to torch's Adam."""
    p, g, m, v = operands(1000, 1)
    p, g, m, v = p[12:], g[12:], m[12:], v[12:]
    step_size = 1e-3 * math.sqrt(1 - 0.999) / (1 - 0.9)
    got, _, _ = oracle.adam_step(p, g, m, v, 0.9, 0.1, 0.999, 0.001, 1e-8, None, step_size)
    m1 = 0.9 * m + 0.1 * g; v1 = 0.999 * v + 0.001 * g * g
    want = p - step_size * m1 / (np.sqrt(v1) + 1e-8)
    assert np.abs((got - p) - (want - p)).max() <= 0.35 * np.abs(want - p).max()


@pytest.fixture()
def on_cpu(oracle, monkeypatch):
    monkeypatch.setattr(cuda_bindings, "cuda_kernels", OracleKernels(oracle))
    monkeypatch.setattr(pam_ops, "_require_kernel", lambda t, use_kernel: None)
    return oracle


@pytest.mark.parametrize("cfg,off", [("pam", None), ("{type: pam, okwargs: {offset: 1.0552}}", OFF)])
def test_optimizer_op_by_op_path_is_the_chain(on_cpu, cfg, off):
    o = on_cpu
    p0, g, m, v = operands(300, 2)
    p0, g = p0[12:], g[12:]
    w = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    opt = optim.Adam([w], lr=5e-4, betas=(0.9, 0.98), eps=1e-8, weight_decay=1e-4, opt_functional_cfg=cfg)
    assert opt.fused and opt.offset == off and opt.supports_flat_params and opt.supports_memory_efficient_fp16
    pn, mn, vn = p0, np.zeros_like(p0), np.zeros_like(p0)
    for t in (1, 2, 3):
        gt = (g * t).astype(np.float32)
        w.grad = torch.from_numpy(gt.copy())
        opt.step()
        step_size = 5e-4 * math.sqrt(1 - 0.98 ** t) / (1 - 0.9 ** t)
        pn, mn, vn = chain(o, pn, gt, mn, vn, 0.9, 0.98, 1e-8, 1e-4 * 5e-4, step_size, off)
        assert_same_bits(w.detach().numpy(), pn, f"parameter after step {t}")
        assert_same_bits(opt.state[w]["exp_avg"].numpy(), mn, "exp_avg")
        assert_same_bits(opt.state[w]["exp_avg_sq"].numpy(), vn, "exp_avg_sq")
    assert opt.state[w]["step"] == 3


def test_optimizer_with_ordinary_ops_is_adam():
    g = torch.Generator().manual_seed(0)
    w = torch.nn.Parameter(torch.randn(50, generator=g)); w2 = torch.nn.Parameter(w.detach().clone())
    a = optim.Adam([w], lr=1e-2, betas=(0.9, 0.999), eps=1e-8, opt_functional_cfg="standard")
    b = torch.optim.Adam([w2], lr=1e-2, betas=(0.9, 0.999), eps=1e-8)
    assert not a.fused
    for t in range(3):
        grad = torch.randn(50, generator=g)
        w.grad = grad.clone(); w2.grad = grad.clone()
        a.step(); b.step()
    # same algorithm up to where eps is added (to sqrt(v) here, to sqrt(v / correction) in torch)
    assert torch.allclose(w, w2, atol=1e-4)
    assert a.step(lambda: torch.tensor(1.5)) == 1.5
    with pytest.raises(AssertionError):
        optim.Adam([w], amsgrad=True, opt_functional_cfg="standard").step()


@pytest.mark.gpu
@pytest.mark.parametrize("off", [None, OFF])
def test_gpu_adam_kernel(oracle, off):
    for n in (1, 5, 4099, 1 << 20):
        p, g, m, v = operands(max(n, 16), n)
        p, g, m, v = p[:n], g[:n], m[:n], v[:n]
        for decay in (None, 3e-7):
            step_size = 5e-4 * math.sqrt(1 - 0.98 ** 2) / (1 - 0.9 ** 2)
            want = oracle.adam_step(p, g, m, v, 0.9, 0.1, 0.98, 0.02, 1e-8, decay, step_size, off)
            tp, tg, tm, tv = (torch.from_numpy(t.copy()).cuda() for t in (p, g, m, v))
            pam_amd._abi.adam_step(tp, tg, tm, tv, 0.9, 0.1, 0.98, 0.02, 1e-8, decay, step_size, 1.0 if off is None else off)
            for got, w, name in zip((tp, tm, tv), want, ("p", "exp_avg", "exp_avg_sq")):
                assert_same_bits(got.cpu().numpy(), w, f"{name} n={n}")
            assert_same_bits(tg.cpu().numpy(), g, "gradient untouched")
    # unaligned views take the scalar kernel
    base = torch.zeros(4 * 1001 + 1, device="cuda")
    p, g, m, v = operands(1001, 9)
    views = [base[1 + i * 1001: 1 + (i + 1) * 1001] for i in range(4)]
    for view, a in zip(views, (p, g, m, v)):
        view.copy_(torch.from_numpy(a))
    pam_amd._abi.adam_step(*views, 0.9, 0.1, 0.98, 0.02, 1e-8, None, 1e-3, 1.0)
    want = oracle.adam_step(p, g, m, v, 0.9, 0.1, 0.98, 0.02, 1e-8, None, 1e-3)
    assert_same_bits(views[0].cpu().numpy(), want[0], "unaligned")


@pytest.mark.gpu
def test_gpu_optimizer_kernel_equals_op_by_op():
    """The single kernel and the same update run op by op through the PAM table give the same bits."""
    g = torch.Generator().manual_seed(3)
    shapes = [(192, 768), (768,), (33, 7)]
    init = [torch.randn(s, generator=g) for s in shapes]
    grads = [[torch.randn(s, generator=g) * 1e-2 for s in shapes] for _ in range(3)]
    results = []
    for fused in (True, False):
        params = [torch.nn.Parameter(t.clone().cuda()) for t in init]
        opt = optim.Adam(params, lr=5e-4, betas=(0.9, 0.98), eps=1e-8, weight_decay=1e-4, opt_functional_cfg="pam")
        opt.fused = fused
        for step in grads:
            for p_, g_ in zip(params, step):
                p_.grad = g_.clone().cuda()
            opt.step()
        results.append([p_.detach().cpu().numpy() for p_ in params] + [opt.state[p_]["exp_avg_sq"].cpu().numpy() for p_ in params])
    for a, b in zip(*results):
        assert_same_bits(a, b, "kernel vs op-by-op")


def test_multiply_grads_keeps_dense_gradients_like_the_reference():
    """fairseq_optimizer.py:103-119 computes mul(grad, c) and drops it; dense gradients stay as they are."""
    from pam_amd.optim import multiply_grads
    p = torch.nn.Parameter(torch.ones(4)); p.grad = torch.full((4,), 3.0)
    q = torch.nn.Parameter(torch.ones(4))                      # no gradient
    calls = []
    multiply_grads([p, q], 0.5, {"mul": lambda a, b: calls.append((a.clone(), b)) or a * b})
    assert len(calls) == 1 and calls[0][1] == 0.5 and torch.equal(p.grad, torch.full((4,), 3.0))
