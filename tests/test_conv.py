"""conv2d on the matrix kernel with the image patches read in place: against the oracle's
product on the unfolded matrix (bit for bit, same accumulation plan), against the unfolded
composition on the same GPU (same terms, other summation grouping), and its gradients."""
import numpy as np
import pytest
import torch

import pam_amd
from pam_amd import _abi, composites
from _util import assert_same_bits

pytestmark = pytest.mark.gpu
OFF = 1.0552

CASES = [
    # batch, c, h, w, co, kh, kw, stride, padding
    (2, 3, 9, 8, 5, 3, 3, (1, 1), (1, 1)),
    (3, 6, 12, 10, 70, 3, 5, (2, 1), (0, 2)),
    (2, 4, 16, 16, 8, 4, 4, (4, 4), (0, 0)),          # non-overlapping patches (patch embedding): 128-bit patch loads
    (2, 3, 32, 40, 70, 8, 8, (8, 8), (0, 0)),         # ... with k = 192 (32-deep k-tiles), ragged in both outputs
    (1, 2, 20, 24, 5, 8, 8, (4, 4), (0, 0)),          # ... overlapping patches, k = 128
    (1, 20, 7, 7, 33, 1, 1, (1, 1), (0, 0)),
    (2, 16, 32, 32, 64, 3, 3, (1, 1), (1, 1)),          # horizontal stride 1, output width a multiple of 4: position quads
    (2, 32, 12, 16, 40, 3, 3, (1, 1), (1, 1)),          # ... with k = 288 (32-deep k-tiles)
    (1, 8, 11, 12, 9, 3, 5, (2, 1), (1, 2)),            # ... vertical stride 2, padding 2 at the row ends
    (1, 4, 16, 32, 6, 3, 3, (1, 1), (1, 1)),            # ... 512 output positions (32-deep k-tiles in the weight gradient)
]


def _inputs(case, seed, specials=False):
    batch, c, h, w, co, kh, kw, stride, padding = case
    rng = np.random.RandomState(seed)
    X = rng.standard_normal((batch, c, h, w)).astype(np.float32)
    W = (rng.standard_normal((co, c, kh, kw)) * 0.1).astype(np.float32)
    if specials:
        flat = X.reshape(-1)
        flat[rng.choice(flat.size, 6, replace=False)] = [0.0, -0.0, 1e-40, -3e38, np.inf, np.nan]
        # (and weights whose products with a padding zero are not zeros: inf, NaN, and 2^127 and more, whose slope is inf)
        W.reshape(-1)[rng.choice(W.size, 5, replace=False)] = [np.inf, np.nan, 3.3e38, 0.0, -1e-40]
    return X, W


def _unfold(X, case):
    _, _, _, _, _, kh, kw, stride, padding = case
    return torch.nn.functional.unfold(torch.from_numpy(X), (kh, kw), padding=padding, stride=stride).numpy()   # [B, K, L]


def _plan(batch, m, n, k):
    return _abi.gemm_plan(batch, m, n, k)


@pytest.mark.parametrize("off", [None, OFF])
@pytest.mark.parametrize("case", CASES)
def test_forward_against_oracle(oracle, case, off):
    batch, c, h, w, co, kh, kw, stride, padding = case
    for specials in (False, True):
        X, W = _inputs(case, 1, specials)
        P = _unfold(X, case)
        K, L = P.shape[1:]
        W2 = W.reshape(co, K)
        Wl = W2 if off is None else oracle.pam(W2, np.float32(off))         # the offset goes with the weights
        want = oracle.gemm(np.broadcast_to(Wl, (batch, co, K)), P, kchunk=_plan(batch, co, L, K))
        got = _abi.conv2d_fwd(torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda(), stride, padding, 1.0 if off is None else off)
        assert got.shape[2] * got.shape[3] == L
        assert_same_bits(got.cpu().numpy().reshape(batch, co, L), want, f"conv forward {case} specials={specials}")


@pytest.mark.parametrize("off", [None, OFF])
@pytest.mark.parametrize("case", [c for c in CASES if c[4] <= 70 and c[1] <= 8])
def test_weight_gradient_against_oracle(oracle, case, off):
    batch, c, h, w, co, kh, kw, stride, padding = case
    X, W = _inputs(case, 2)
    P = _unfold(X, case)
    K, L = P.shape[1:]
    dY = (np.random.RandomState(3).standard_normal((batch, co, L)) * 1e-2).astype(np.float32)
    Xd, Wd = torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda()
    dYd = torch.from_numpy(dY).cuda().view(batch, co, *_abi.conv2d_fwd(Xd, Wd, stride, padding, 1.0).shape[2:])
    Pt = np.ascontiguousarray(P.transpose(0, 2, 1))                          # [B, L, K]
    plan = _plan(batch, co, K, L)
    dl = dY if off is None else oracle.pam(dY, np.float32(off))
    want = oracle.gemm(dl, Pt, kchunk=plan)
    got = _abi.conv2d_bwd_weight(Xd, dYd, Wd, stride, padding, False, 1.0 if off is None else off)
    assert_same_bits(got.cpu().numpy(), want, f"approximate weight gradient {case}")
    want = oracle.gemm(dY, Pt, mode=oracle.MODE_BWD_DELTA_L, D=np.broadcast_to(W.reshape(co, K), (batch, co, K)), offset=off, kchunk=plan)
    got = _abi.conv2d_bwd_weight(Xd, dYd, Wd, stride, padding, True, 1.0 if off is None else off)
    assert_same_bits(got.cpu().numpy(), want, f"exact weight gradient {case}")


STRIDE_ONE = [c for c in CASES if c[7] == (1, 1)] + [
              (2, 5, 10, 13, 7, 3, 5, (1, 1), (2, 0)),        # padding k - 1 on one axis, none on the other
              (1, 3, 6, 6, 4, 2, 2, (1, 1), (0, 0))]          # even kernel


@pytest.mark.parametrize("off", [None, OFF])
@pytest.mark.parametrize("case", STRIDE_ONE)
def test_input_gradient_against_oracle(oracle, case, off):
    """Stride 1: dX is the convolution of dY, padded by k - 1 - pad, with the flipped weights; the
    oracle computes that product on the unfolded gradient with the library's accumulation plan."""
    batch, c, h, w, co, kh, kw, stride, (ph, pw) = case
    X, W = _inputs(case, 4)
    ho, wo = h + 2 * ph - kh + 1, w + 2 * pw - kw + 1
    rng = np.random.RandomState(5)
    dY = (rng.standard_normal((batch, co, ho, wo)) * 1e-2).astype(np.float32)
    dY.reshape(-1)[rng.choice(dY.size, max(2, dY.size // 50), replace=False)] = 0.0
    P = torch.nn.functional.unfold(torch.from_numpy(dY), (kh, kw), padding=(kh - 1 - ph, kw - 1 - pw)).numpy()   # [B, co kh kw, h w]
    K, L = P.shape[1:]
    assert L == h * w
    Wf = np.ascontiguousarray(W.transpose(1, 0, 2, 3)[:, :, ::-1, ::-1]).reshape(c, K)
    plan = _plan(batch, c, L, K)
    Xd, Wd, dYd = torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda(), torch.from_numpy(dY).cuda()
    o = 1.0 if off is None else off
    Wl = Wf if off is None else oracle.pam(Wf, np.float32(off))
    want = oracle.gemm(np.broadcast_to(Wl, (batch, c, K)), P, kchunk=plan)
    got = _abi.conv2d_bwd_input(dYd, Wd, Xd, (ph, pw), False, o)
    assert_same_bits(got.cpu().numpy().reshape(batch, c, L), want, f"approximate input gradient {case}")
    want = oracle.gemm(np.broadcast_to(Wf, (batch, c, K)), P, mode=oracle.MODE_BWD_DELTA_R, D=X.reshape(batch, c, L), offset=off, kchunk=plan)
    got = _abi.conv2d_bwd_input(dYd, Wd, Xd, (ph, pw), True, o)
    assert_same_bits(got.cpu().numpy().reshape(batch, c, L), want, f"exact input gradient {case}")


def test_input_gradient_rejects_other_strides():
    X = torch.randn(1, 2, 8, 8, device="cuda"); W = torch.randn(3, 2, 3, 3, device="cuda")
    lib = _abi.load_library()
    assert lib.pam_hip_conv2d_workspace_bytes(1, 2, 8, 8, 3, 3, 3, 2, 2, 1, 1, 1, 2, 1.0) == 0
    dY = torch.randn(1, 3, 4, 4, device="cuda"); dX = torch.empty_like(X); ws = torch.empty(1 << 16, device="cuda")
    rc = lib.pam_hip_conv2d_bwd_input(dY.data_ptr(), W.data_ptr(), X.data_ptr(), dX.data_ptr(), 1, 2, 8, 8, 3, 3, 3, 2, 2, 1, 1, 1,
                                      0, 1.0, ws.data_ptr(), ws.numel() * 4, None)
    assert rc == -1 and b"stride 1" in lib.pam_hip_last_error()
    assert not pam_amd.fused.input_gradient_in_place(W, (2, 2), (1, 1)) and pam_amd.fused.input_gradient_in_place(W, (1, 1), (2, 2))
    assert not pam_amd.fused.input_gradient_in_place(W, (1, 1), (3, 1))


def _close(a, b, tol=3e-6):
    return (a - b).abs().max().item() <= tol * b.abs().max().item()


@pytest.mark.parametrize("stride", [(2, 1), (1, 1)])
@pytest.mark.parametrize("approx", [True, (True, False), False, (False, True)])
def test_module_path_matches_unfolded_composition(approx, stride):
    """pam.conv2d / pam.Conv2d with patches read in place against the unfold + linear chain on the
    same GPU: values and both gradients agree up to the grouping of the sums.  With stride 1 the
    input gradient runs in place as well, the exact one included; with another stride the exact
    input gradient sends the whole call down the unfolded path."""
    torch.manual_seed(0)
    X = torch.randn(4, 6, 14, 11, device="cuda"); W = torch.randn(10, 6, 3, 3, device="cuda") * 0.2; b = torch.randn(10, device="cuda")
    g = torch.randn(4, 10, 7 if stride[0] == 2 else 14, 11, device="cuda")
    res = {}
    for implicit in (True, False):
        composites.implicit_conv = implicit
        try:
            Xr, Wr = X.clone().requires_grad_(), W.clone().requires_grad_()
            Y = pam_amd.conv2d(Xr, Wr, b, stride=stride, padding=1, offset=OFF, approx_bwd=approx)
            Y.backward(g)
            res[implicit] = (Y.detach(), Xr.grad, Wr.grad)
        finally:
            composites.implicit_conv = True
    in_place = stride == (1, 1) or approx is True or (isinstance(approx, tuple) and approx[0])
    assert res[True][0].is_contiguous() == in_place
    for a, c in zip(res[True], res[False]):
        assert a.shape == c.shape and _close(a, c)
    # an exact gradient with respect to the input: in place for stride 1, else the unfolded path
    Xr = X.clone().requires_grad_()
    pam_amd.conv2d(Xr, W, None, padding=1, stride=stride, approx_bwd=False).sum().backward()
    assert Xr.grad is not None and torch.isfinite(Xr.grad).all()
    # no gradient wanted for the input (first layer): in place whatever the flags
    Wr = W.clone().requires_grad_()
    pam_amd.conv2d(X, Wr, None, padding=1, approx_bwd=False).sum().backward()
    assert Wr.grad is not None and torch.isfinite(Wr.grad).all()


def test_conv_module_against_torch_on_exact_products():
    """Power-of-two weights make every PAM product exact (pam/test_pam.py:151-170): the layer equals F.conv2d."""
    torch.manual_seed(1)
    X1 = (torch.randint(-1024, 1024, (5, 13, 15, 17), device="cuda") / 64.0).requires_grad_()
    _against_torch(X1, (1, 2))
    _against_torch(X1.detach().clone().requires_grad_(), (1, 1))        # the input gradient in place


def _against_torch(X1, stride):
    conv = pam_amd.Conv2d(13, 19, (3, 5), padding=(1, 2), stride=stride, approx_bwd=True).cuda()
    with torch.no_grad():
        conv.weight.copy_(2.0 ** torch.randint(-8, 8, conv.weight.shape, device="cuda").float())
    X2 = X1.detach().clone().requires_grad_()
    Y1 = conv(X1); Y1.sum().backward()
    Y2 = torch.nn.functional.conv2d(X2, conv.weight.detach(), conv.bias.detach(), padding=(1, 2), stride=stride); Y2.sum().backward()
    assert _close(Y1, Y2, 2e-6) and _close(X1.grad, X2.grad, 2e-6)
    Wt = conv.weight.detach().clone().requires_grad_()
    torch.nn.functional.conv2d(X2.detach(), Wt, None, padding=(1, 2), stride=stride).sum().backward()
    assert _close(conv.weight.grad, Wt.grad, 2e-6)


GROUPED = [
    # batch, c, h, w, co, kh, kw, stride, padding, groups
    (2, 8, 9, 8, 12, 3, 3, (1, 1), (1, 1), 4),
    (3, 6, 12, 10, 140, 3, 5, (2, 1), (0, 2), 2),        # 70 filters per group: more than one row tile
    (2, 16, 7, 7, 16, 3, 3, (1, 1), (1, 1), 16),         # depthwise
    (3, 8, 12, 10, 8, 3, 5, (2, 1), (0, 2), 8),          # depthwise, strided, a 3 x 5 kernel
    (1, 4, 40, 40, 4, 3, 3, (1, 1), (1, 1), 4),          # depthwise with few channels: the weight gradient's sum over 1600 positions is cut
    (2, 6, 9, 9, 6, 5, 5, (1, 1), (4, 4), 6),            # depthwise, padding = kernel - 1
    (2, 4, 10, 9, 12, 3, 3, (1, 1), (1, 1), 4),          # one channel, three filters per group
]


@pytest.mark.parametrize("off", [None, OFF])
@pytest.mark.parametrize("case", GROUPED)
def test_grouped_convolution_against_oracle(oracle, case, off):
    """pam.conv2d_group's arithmetic (pam/pam_ops.py:163-198) per group: forward, both weight gradients and, for
    stride 1, both input gradients against the oracle's products on the unfolded slices."""
    batch, c, h, w, co, kh, kw, stride, padding, G = case
    cg, cog = c // G, co // G
    _grouped_case(oracle, case, off, odd_weights=False)
    if G == c == co:
        # depthwise kernels leave out the terms of padding positions, which are zeros -- unless a weight or an upstream
        # gradient is inf or NaN (or becomes inf with the offset): then the term is NaN, as in the matrix kernel
        _grouped_case(oracle, case, off, odd_weights=True)


def _grouped_case(oracle, case, off, odd_weights):
    batch, c, h, w, co, kh, kw, stride, padding, G = case
    cg, cog = c // G, co // G
    rng = np.random.RandomState(11)
    X = rng.standard_normal((batch, c, h, w)).astype(np.float32)
    W = (rng.standard_normal((co, cg, kh, kw)) * 0.1).astype(np.float32)
    X.reshape(-1)[rng.choice(X.size, 5, replace=False)] = [0.0, -0.0, 1e-40, -3e38, 7.0]
    if odd_weights:
        W.reshape(-1)[rng.choice(W.size, 4, replace=False)] = [np.inf, np.nan, 3.3e38, 0.0]
    o = 1.0 if off is None else off
    Xd, Wd = torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda()
    Y = _abi.conv2d_fwd(Xd, Wd, stride, padding, o, G)
    ho, wo = Y.shape[2:]
    L = ho * wo
    dY = (rng.standard_normal((batch, co, ho, wo)) * 1e-2).astype(np.float32)
    if odd_weights:
        dY.reshape(-1)[rng.choice(dY.size, 4, replace=False)] = [np.inf, np.nan, -3.3e38, 0.0]
    dYd = torch.from_numpy(dY).cuda()
    dW_a = _abi.conv2d_bwd_weight(Xd, dYd, Wd, stride, padding, False, o, G).cpu().numpy()
    dW_e = _abi.conv2d_bwd_weight(Xd, dYd, Wd, stride, padding, True, o, G).cpu().numpy()
    stride_one = stride == (1, 1)
    if stride_one:
        dX_a = _abi.conv2d_bwd_input(dYd, Wd, Xd, padding, False, o, G).cpu().numpy()
        dX_e = _abi.conv2d_bwd_input(dYd, Wd, Xd, padding, True, o, G).cpu().numpy()
    for g in range(G):
        Xg = np.ascontiguousarray(X[:, g * cg:(g + 1) * cg]); Wg = W[g * cog:(g + 1) * cog]; dYg = np.ascontiguousarray(dY[:, g * cog:(g + 1) * cog])
        P = torch.nn.functional.unfold(torch.from_numpy(Xg), (kh, kw), padding=padding, stride=stride).numpy()        # [B, K, L]
        K = P.shape[1]
        W2 = Wg.reshape(cog, K)
        Wl = W2 if off is None else oracle.pam(W2, np.float32(off))
        want = oracle.gemm(np.broadcast_to(Wl, (batch, cog, K)), P, kchunk=_plan(batch * G, cog, L, K))          # one launch over (image, group) pairs
        assert_same_bits(Y[:, g * cog:(g + 1) * cog].cpu().numpy().reshape(batch, cog, L), want, f"grouped forward, group {g}")
        Pt = np.ascontiguousarray(P.transpose(0, 2, 1)); d2 = dYg.reshape(batch, cog, L); plan = _plan(batch * G, cog, K, L)
        dl = d2 if off is None else oracle.pam(d2, np.float32(off))
        assert_same_bits(dW_a[:, g * cog:(g + 1) * cog], oracle.gemm(dl, Pt, kchunk=plan), f"grouped weight gradient, group {g}")
        want = oracle.gemm(d2, Pt, mode=oracle.MODE_BWD_DELTA_L, D=np.broadcast_to(W2, (batch, cog, K)), offset=off, kchunk=plan)
        assert_same_bits(dW_e[:, g * cog:(g + 1) * cog], want, f"grouped exact weight gradient, group {g}")
        if stride_one:
            Pd = torch.nn.functional.unfold(torch.from_numpy(dYg), (kh, kw), padding=(kh - 1 - padding[0], kw - 1 - padding[1])).numpy()
            Kt = Pd.shape[1]
            Wf = np.ascontiguousarray(Wg.transpose(1, 0, 2, 3)[:, :, ::-1, ::-1]).reshape(cg, Kt)
            plan = _plan(batch * G, cg, h * w, Kt)
            Wfl = Wf if off is None else oracle.pam(Wf, np.float32(off))
            assert_same_bits(dX_a[:, g * cg:(g + 1) * cg].reshape(batch, cg, h * w), oracle.gemm(np.broadcast_to(Wfl, (batch, cg, Kt)), Pd, kchunk=plan),
                             f"grouped input gradient, group {g}")
            want = oracle.gemm(np.broadcast_to(Wf, (batch, cg, Kt)), Pd, mode=oracle.MODE_BWD_DELTA_R, D=Xg.reshape(batch, cg, h * w), offset=off, kchunk=plan)
            assert_same_bits(dX_e[:, g * cg:(g + 1) * cg].reshape(batch, cg, h * w), want, f"grouped exact input gradient, group {g}")


@pytest.mark.parametrize("stride", [(1, 1), (2, 2)])
@pytest.mark.parametrize("approx", [True, False])
def test_grouped_module_matches_unfolded_composition(approx, stride):
    """pam.Conv2d with groups: patches in place against unfold + bmm on the same GPU, values and gradients."""
    torch.manual_seed(3)
    X = torch.randn(3, 8, 10, 9, device="cuda"); g = None
    res = {}
    for implicit in (True, False):
        composites.implicit_conv = implicit
        try:
            torch.manual_seed(4)
            conv = pam_amd.Conv2d(8, 12, 3, padding=1, stride=stride, groups=4, approx_bwd=approx, offset=OFF).cuda()
            Xr = X.clone().requires_grad_()
            Y = conv(Xr)
            g = torch.randn_like(Y) if g is None else g
            Y.backward(g)
            res[implicit] = (Y.detach(), Xr.grad, conv.weight.grad, conv.bias.grad)
        finally:
            composites.implicit_conv = True
    for a, c in zip(res[True], res[False]):
        assert a.shape == c.shape and _close(a, c)
