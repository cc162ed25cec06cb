"""One training step of an encoder-decoder transformer whose linear layers and attention
products are PAM (the shape of the reference's fairseq recipe: every nn.Linear replaced by
pam.Linear, attention through pam.bmm, approximate backward).  The model is plain PyTorch
written for this test; only its products go through the package."""
import numpy as np
import pytest
import torch

import pam_amd
from pam_amd import cuda_bindings, pam_ops


FULLY_PAM = False        # softmax and LayerNorm through the package too (the reference's multiplication-free recipe)


def _softmax(s):
    return pam_amd.softmax(s, dim=-1, approx_bwd=True) if FULLY_PAM else torch.softmax(s, -1)


def _norm(d):
    return pam_amd.LayerNorm(d, approx_bwd=True) if FULLY_PAM else torch.nn.LayerNorm(d)


class Attention(torch.nn.Module):
    def __init__(self, d, heads):
        super().__init__()
        self.h = heads
        self.q, self.k, self.v, self.o = (pam_amd.Linear(d, d, approx_bwd=True) for _ in range(4))

    def forward(self, x, mem, causal):
        B, T, D = x.shape; S = mem.shape[1]; H = self.h; dh = D // H
        q = self.q(x).view(B, T, H, dh).transpose(1, 2).reshape(B * H, T, dh) * dh ** -0.5
        k = self.k(mem).view(B, S, H, dh).transpose(1, 2).reshape(B * H, S, dh)
        v = self.v(mem).view(B, S, H, dh).transpose(1, 2).reshape(B * H, S, dh)
        s = pam_amd.bmm(q, k.transpose(1, 2), approx_bwd=True)
        if causal:
            s = s.masked_fill(torch.ones(T, S, dtype=torch.bool, device=x.device).triu(1), float("-inf"))
        o = pam_amd.bmm(_softmax(s), v, approx_bwd=True)
        return self.o(o.view(B, H, T, dh).transpose(1, 2).reshape(B, T, D))


class Layer(torch.nn.Module):
    def __init__(self, d, ffn, heads, cross):
        super().__init__()
        self.sa = Attention(d, heads); self.n1 = _norm(d)
        self.ca = Attention(d, heads) if cross else None
        self.n2 = _norm(d) if cross else None
        self.f1 = pam_amd.Linear(d, ffn, approx_bwd=True); self.f2 = pam_amd.Linear(ffn, d, approx_bwd=True)
        self.n3 = _norm(d)

    def forward(self, x, mem=None):
        x = self.n1(x + self.sa(x, x, causal=mem is not None))
        if self.ca is not None:
            x = self.n2(x + self.ca(x, mem, causal=False))
        return self.n3(x + self.f2(torch.relu(self.f1(x))))            # ReLU: exact zeros reach the next product


class EncDec(torch.nn.Module):
    def __init__(self, vocab, d, ffn, heads, layers):
        super().__init__()
        self.emb = torch.nn.Embedding(vocab, d)
        torch.nn.init.normal_(self.emb.weight, std=d ** -0.5)
        self.enc = torch.nn.ModuleList(Layer(d, ffn, heads, False) for _ in range(layers))
        self.dec = torch.nn.ModuleList(Layer(d, ffn, heads, True) for _ in range(layers))
        self.d = d

    def forward(self, src, tgt):
        m = self.emb(src) * self.d ** 0.5
        for l in self.enc:
            m = l(m)
        y = self.emb(tgt) * self.d ** 0.5
        for l in self.dec:
            y = l(y, m)
        B, T, D = y.shape
        logits = pam_amd.linear(y, self.emb.weight, approx_bwd=True)    # tied output projection
        return logits


def _step(model, src, tgt, labels):
    model.zero_grad(set_to_none=True)
    logits = model(src, tgt)
    loss = torch.nn.functional.cross_entropy(logits.view(-1, logits.shape[-1]), labels.view(-1))
    loss.backward()
    return loss.detach(), {n: p.grad.detach().clone() for n, p in model.named_parameters()}


def _data(vocab, batch, length, seed):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randint(0, vocab, (batch, length), generator=g) for _ in range(3))


@pytest.mark.gpu
def test_small_model_matches_oracle_backed_run(oracle, monkeypatch):
    """GPU step vs the same step with every PAM product computed by the CPU oracle: the PAM parts
    are bit-identical, so what is left is the CPU/GPU difference of softmax, LayerNorm and
    cross-entropy."""
    from test_host_api import OracleKernels
    torch.manual_seed(0)
    model = EncDec(vocab=101, d=64, ffn=128, heads=4, layers=2)
    src, tgt, lab = _data(101, 8, 12, 1)
    gpu_model = EncDec(101, 64, 128, 4, 2).cuda(); gpu_model.load_state_dict(model.state_dict())
    loss_g, grads_g = _step(gpu_model, src.cuda(), tgt.cuda(), lab.cuda())
    loss_g2, grads_g2 = _step(gpu_model, src.cuda(), tgt.cuda(), lab.cuda())
    assert torch.equal(loss_g, loss_g2) and all(torch.equal(grads_g[n], grads_g2[n]) for n in grads_g)   # deterministic
    monkeypatch.setattr(cuda_bindings, "cuda_kernels", OracleKernels(oracle))
    monkeypatch.setattr(pam_ops, "_require_kernel", lambda t, use_kernel: None)
    loss_c, grads_c = _step(model, src, tgt, lab)
    assert abs(loss_g.item() - loss_c.item()) <= 1e-4 * abs(loss_c.item())
    for n, gc in grads_c.items():
        gg = grads_g[n].cpu()
        assert (gg - gc).abs().max() <= 2e-3 * gc.abs().max() + 1e-7, n


@pytest.mark.gpu
def test_full_size_step_runs():
    """6 + 6 layers, d_model 512, FFN 1024, 4 heads, 10k shared vocabulary, 128 sequences of 32 tokens."""
    from pam_amd._abi import load_library
    load_library()
    torch.manual_seed(0)
    model = EncDec(vocab=10000, d=512, ffn=1024, heads=4, layers=6).cuda()
    src, tgt, lab = (t.cuda() for t in _data(10000, 128, 32, 2))
    loss, grads = _step(model, src, tgt, lab)
    assert torch.isfinite(loss) and 5.0 < loss.item() < 30.0          # the order of log(10000) at initialisation
    assert all(torch.isfinite(g).all() for g in grads.values())
    assert sum(float(g.abs().sum()) for g in grads.values()) > 0
    loss2, grads2 = _step(model, src, tgt, lab)
    assert torch.equal(loss, loss2) and all(torch.equal(grads[n], grads2[n]) for n in grads)


@pytest.mark.gpu
def test_fully_pam_recipe_trains(oracle, monkeypatch):
    """The multiplication-free recipe end to end: PAM linears and attention products, PAM softmax
    (single kernel with its gradient) and LayerNorm, the op-table cross entropy and the PAM Adam
    kernel, wired through the configuration hooks.  A few steps on a small model: the first step
    agrees with an oracle-backed CPU run, the loss falls, and a rerun gives identical bits."""
    from pam_amd import factories, optim
    from test_host_api import OracleKernels
    import sys
    mod = sys.modules[__name__]
    monkeypatch.setattr(mod, "FULLY_PAM", True)
    ops = factories.get_function_dict("pam")
    src, tgt, lab = _data(101, 8, 12, 3)

    def run(device, steps):
        torch.manual_seed(0)
        model = EncDec(vocab=101, d=64, ffn=128, heads=4, layers=2).to(device)
        opt = optim.Adam(model.parameters(), lr=2e-3, betas=(0.9, 0.98), eps=1e-8, opt_functional_cfg="pam")
        losses, first_grads = [], None
        for _ in range(steps):
            model.zero_grad(set_to_none=True)
            logits = model(src.to(device), tgt.to(device))
            loss = pam_amd.cross_entropy(logits.view(-1, logits.shape[-1]), lab.to(device).view(-1), None, -100, "mean", 0.0,
                                         op_dict=ops)
            loss.backward()
            if first_grads is None:
                first_grads = {n: p.grad.detach().cpu().clone() for n, p in model.named_parameters()}
            opt.step()
            losses.append(loss.item())
        return losses, first_grads, {n: p.detach().cpu().clone() for n, p in model.named_parameters()}

    losses, grads, params = run("cuda", 8)
    assert all(np.isfinite(losses)) and losses[-1] < losses[0] - 0.05, losses
    losses2, _, params2 = run("cuda", 8)
    assert losses == losses2 and all(torch.equal(params[n], params2[n]) for n in params)
    monkeypatch.setattr(cuda_bindings, "cuda_kernels", OracleKernels(oracle))
    monkeypatch.setattr(pam_ops, "_require_kernel", lambda t, use_kernel: None)
    losses_c, grads_c, _ = run("cpu", 1)
    assert abs(losses[0] - losses_c[0]) <= 1e-4 * abs(losses_c[0])
    for n, gc in grads_c.items():
        assert (grads[n] - gc).abs().max() <= 2e-3 * gc.abs().max() + 1e-7, n
