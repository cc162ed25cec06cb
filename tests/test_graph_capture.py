"""The kernels under HIP graph capture: a PAM training step (linear layers, softmax, LayerNorm, Adam)
recorded once into a torch.cuda.CUDAGraph and replayed with new inputs gives, on every replay, the bits
of the same step run eagerly.  Calls only enqueue kernels on the capturing stream; nothing in the
library allocates, synchronises or clears memory with a memset."""
import pytest
import torch

import pam_amd
from pam_amd import optim

pytestmark = pytest.mark.gpu


class Block(torch.nn.Module):
    def __init__(self, d, ffn):
        super().__init__()
        self.norm = pam_amd.LayerNorm(d, approx_bwd=True)
        self.f1 = pam_amd.Linear(d, ffn, approx_bwd=True)
        self.f2 = pam_amd.Linear(ffn, d, approx_bwd=True)

    def forward(self, x):
        h = self.f2(torch.relu(self.f1(self.norm(x))))
        return pam_amd.softmax(x + h, dim=-1, approx_bwd=True)


def _make(seed):
    torch.manual_seed(seed)
    model = Block(64, 160).cuda()
    opt = optim.Adam(model.parameters(), lr=1e-2, betas=(0.9, 0.98), opt_functional_cfg="pam")
    return model, opt


def _train_step(model, opt, x, target):
    opt.zero_grad(set_to_none=False)
    loss = ((model(x) - target) ** 2).sum()
    loss.backward()
    opt.step()
    return loss


def test_training_step_replays_bit_for_bit():
    g = torch.Generator().manual_seed(0)
    batches = [(torch.randn(96, 64, generator=g).cuda(), torch.rand(96, 64, generator=g).cuda()) for _ in range(4)]

    # eager run
    model, opt = _make(1)
    # Adam creates its state on the first step and advances a Python step counter; capture needs fixed
    # scalars, so both runs take one eager step first and the graph replays the second step's scalars
    eager_losses = []
    for x, t in batches:
        eager_losses.append(_train_step(model, opt, x, t).item())
    eager_params = [p.detach().clone() for p in model.parameters()]

    # captured run: first step eager (state creation), then one step captured and replayed
    model, opt = _make(1)
    sx, st = batches[0][0].clone(), batches[0][1].clone()
    first = _train_step(model, opt, sx, st).item()
    assert first == eager_losses[0]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up on a side stream, as capture requires
        snapshot = [p.detach().clone() for p in model.parameters()]
        state = {k: {n: (v.clone() if torch.is_tensor(v) else v) for n, v in s.items()} for k, s in opt.state.items()}
        _train_step(model, opt, sx, st)
        with torch.no_grad():                           # undo the warm-up step
            for p, q in zip(model.parameters(), snapshot):
                p.copy_(q)
            for k, s in state.items():
                for n, v in s.items():
                    if torch.is_tensor(v):
                        opt.state[k][n].copy_(v)
                    else:
                        opt.state[k][n] = v
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    # every replayed step must use its own bias-correction scalars: capture one graph per step index
    losses = [first]
    for step, (x, t) in enumerate(batches[1:], start=2):
        sx.copy_(x); st.copy_(t)
        graph = torch.cuda.CUDAGraph()
        for k in opt.state:
            opt.state[k]["step"] = step - 1
        with torch.cuda.graph(graph):
            loss = _train_step(model, opt, sx, st)
        # capture only records; run it, with eager work and synchronisation around the replay
        probe = (sx * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        losses.append(loss.item())
        assert probe == (sx * 2).sum().item()
    assert losses == eager_losses
    for p, q in zip(model.parameters(), eager_params):
        assert torch.equal(p.detach(), q)


def test_one_graph_replayed_many_times():
    """A forward + backward recorded once and replayed on changing inputs, eager work in between."""
    torch.manual_seed(3)
    model = Block(64, 160).cuda()
    g = torch.Generator().manual_seed(4)
    sx = torch.randn(50, 64, generator=g).cuda().requires_grad_()
    sg = torch.randn(50, 64, generator=g).cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        model(sx).backward(sg)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    sx.grad = None
    for p in model.parameters():
        p.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = model(sx)
        y.backward(sg)
    for i in range(4):
        x = torch.randn(50, 64, generator=g).cuda(); gr = torch.randn(50, 64, generator=g).cuda()
        with torch.no_grad():
            sx.copy_(x); sg.copy_(gr)
        graph.replay()
        torch.cuda.synchronize()
        xe = x.clone().requires_grad_()
        ref = Block(64, 160).cuda(); ref.load_state_dict(model.state_dict())
        ye = ref(xe); ye.backward(gr)
        assert torch.equal(y.detach(), ye.detach()), f"replay {i}: forward"
        assert torch.equal(sx.grad, xe.grad), f"replay {i}: input gradient"
        for (n, p), q in zip(model.named_parameters(), ref.parameters()):
            assert torch.equal(p.grad, q.grad), f"replay {i}: gradient of {n}"
