"""Host-side logic without a GPU: the C ABI exports what include/pam_hip.h declares, and the
autograd layer (same formulas as the reference's pam/cuda_bindings.py) composes kernel calls
correctly.  The kernels are replaced by a stand-in built on the CPU oracle, so only the
plumbing is under test here; the kernels themselves are checked on the GPU."""
import ctypes
import math
import pathlib
import re

import numpy as np
import pytest
import torch

import pam_amd
from pam_amd import _abi, cuda_bindings, pam_ops
from _util import assert_same_bits

ROOT = pathlib.Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "pam_hip.h").read_text()
    declared = set(re.findall(r"\b(pam_hip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) == 42
    # measurement probes and the tuning hook live in a header of their own, not in the drop-in interface
    probes = set(re.findall(r"\b(pam_hip_[a-z0-9_]+)\s*\(", (ROOT / "include" / "pam_hip_probe.h").read_text()))
    assert probes == {"pam_hip_issue_probe", "pam_hip_issue_probe_lds", "pam_hip_set_tuning"} and not (probes & declared)
    declared |= probes
    lib = ctypes.CDLL(str(_abi.library_path()))
    missing = [name for name in sorted(declared) if not hasattr(lib, name)]
    assert not missing, f"declared in pam_hip.h but not exported: {missing}"
    # the fourteen entry points of the reference's extension module, one to one (pam/cuda_kernels.cu:932-947)
    for name in ("pam_fwd pam_bwd pad_fwd pad_bwd pam_matmul_fwd pam_bmm_fwd pam_matmul_bwd pam_bmm_bwd "
                 "standard_matmul standard_bmm pa_exp_fwd pa_exp_bwd pa_log_fwd pa_log_bwd").split():
        assert "pam_hip_" + name in declared and hasattr(_abi.HipKernels, name)
    assert set(_abi.exported_symbols()) <= declared
    assert _abi.load_library().pam_hip_abi_version() == 2
    # the library under test was built from the sources of this tree
    from pam_amd import build as builder
    assert _abi.load_library().pam_hip_source_hash().decode() == builder.source_hash()


def test_log2_of_the_usual_bases_is_pinned():
    """pa_exp / pa_log scale by the fp32 constant log2(base); one unit of the last place in it moves every result.
    The goldens of tests/golden/exp_log.npz were written with torch.log2(torch.tensor(base)) on the CPU: the
    library's constant, the oracle's and torch's must be these bit patterns."""
    import numpy as np
    import torch
    from oracle import pam_oracle
    lib = _abi.load_library()
    for base, want in ((math.e, 0x3fb8aa3b), (10.0, 0x40549a78), (0.5, 0xbf800000), (2.0, 0x3f800000), (3.0, 0x3fcae00d)):
        for got in (lib.pam_hip_log2_base(base), pam_oracle.log2_base(base), torch.log2(torch.tensor(base, dtype=torch.float32)).item()):
            assert np.float32(got).view(np.uint32) == want, (base, got)


def test_argument_errors_come_back_as_status_codes():
    lib = _abi.load_library()
    assert lib.pam_hip_pam_fwd(None, None, None, 16, 1.0, None) == -1
    assert b"null pointer" in lib.pam_hip_last_error()
    assert lib.pam_hip_pam_fwd(None, None, None, 0, 1.0, None) == 0          # empty input is fine
    assert lib.pam_hip_pam_matmul_fwd(None, 1, 1, None, 1, 1, None, 1, 1, -1, 4, 4, 1.0, None, 0, None) == -1
    assert lib.pam_hip_pam_matmul_fwd(None, 1, 1, None, 1, 1, None, 1, 1, 0, 4, 4, 1.0, None, 0, None) == 0
    c = _abi.gemm_plan(1, 12608, 768, 192)
    assert c % 32 == 0 and c >= 192
    c = _abi.gemm_plan(1, 192, 768, 12608)
    assert c % 32 == 0 and 128 <= c < 12608     # long k, few outputs: every tile's k range is cut into pieces of 128 k or more
    pieces = -(-12608 // c)
    assert _abi.load_library().pam_hip_gemm_workspace_bytes(1, 192, 768, 12608) == (64 << 10) + pieces * 36 * 64 * 64 * 4     # arrival words + a piece per unit
    assert _abi.load_library().pam_hip_gemm_workspace_bytes(1, 12608, 768, 192) == 0        # whole tiles: no scratch


class OracleKernels:
    """Same fourteen methods as the kernel object, computed by the CPU oracle on CPU tensors."""

    def __init__(self, oracle):
        self.o = oracle
        self.calls = []

    @staticmethod
    def _np(t):
        return t.detach().numpy()

    def _ret(self, a):
        return torch.from_numpy(np.array(a, dtype=np.float32, order="C"))      # keeps 0-d results 0-d

    def _off(self, offset):
        return None if offset == 1.0 else offset

    def pam_fwd(self, A, B, offset):
        self.calls.append(("pam_fwd", A.stride(), B.stride()))
        return self._ret(self.o.pam(self._np(A), self._np(B), self._off(offset)).reshape(A.shape))

    def pad_fwd(self, A, B, offset):
        return self._ret(self.o.pad(self._np(A), self._np(B), self._off(offset)).reshape(A.shape))

    def pam_bwd(self, A, B, dC, offset):
        return self._ret(self.o.pam_bwd(self._np(A), self._np(B), self._np(dC), self._off(offset)).reshape(A.shape))

    def pad_bwd(self, A, B, dC, offset):
        return self._ret(self.o.pad_bwd(self._np(A), self._np(B), self._np(dC), self._off(offset)).reshape(A.shape))

    def pa_exp_fwd(self, X, base, offset):
        return self._ret(self.o.pa_exp(self._np(X), base, self._off(offset)).reshape(X.shape))

    def pa_log_fwd(self, X, base, offset):
        return self._ret(self.o.pa_log(self._np(X), base, self._off(offset)).reshape(X.shape))

    def pa_exp_bwd(self, X, dY, base, offset):
        return self._ret(self.o.pa_exp_bwd(self._np(X), self._np(dY), base, self._off(offset)).reshape(X.shape))

    def pa_log_bwd(self, X, dY, base, offset):
        return self._ret(self.o.pa_log_bwd(self._np(X), self._np(dY), base, self._off(offset)).reshape(X.shape))

    def _mm(self, name, L, R, lrm, rrm, offset, mode=0, D=None):
        self.calls.append((name, tuple(L.stride()), tuple(R.stride()), lrm, rrm))
        # the flags must describe the strides they come with (pam/cuda_bindings.py:106-115)
        assert (L.stride()[-1] == 1) == lrm or L.stride()[-2] == 1
        assert (R.stride()[-1] == 1) == rrm or R.stride()[-2] == 1
        return self._ret(self.o.gemm(self._np(L), self._np(R), mode=mode, D=None if D is None else self._np(D),
                                     offset=self._off(offset)))

    def pam_matmul_fwd(self, A, B, arm, brm, offset):
        return self._mm("pam_matmul_fwd", A, B, arm, brm, offset)

    def pam_bmm_fwd(self, A, B, arm, brm, offset):
        return self._mm("pam_bmm_fwd", A, B, arm, brm, offset)

    def standard_matmul(self, A, B, arm, brm, offset):
        return self._mm("standard_matmul", A, B, arm, brm, offset, mode=1)

    def standard_bmm(self, A, B, arm, brm, offset):
        return self._mm("standard_bmm", A, B, arm, brm, offset, mode=1)

    def pam_matmul_bwd(self, L, R, M, lrm, rrm, delta_L, offset):
        return self._mm("pam_matmul_bwd", L, R, lrm, rrm, offset, mode=2 if delta_L else 3, D=M)

    def pam_bmm_bwd(self, L, R, M, lrm, rrm, delta_L, offset):
        return self._mm("pam_bmm_bwd", L, R, lrm, rrm, offset, mode=2 if delta_L else 3, D=M)


@pytest.fixture()
def fake(oracle, monkeypatch):
    k = OracleKernels(oracle)
    monkeypatch.setattr(cuda_bindings, "cuda_kernels", k)
    return k


def _t(shape, seed, grad=True):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).requires_grad_(grad)


def test_elementwise_autograd_formulas(fake, oracle):
    A, B = _t((7, 5), 1), _t((7, 5), 2)
    dY = _t((7, 5), 3, grad=False)
    for off in (None, 1.0552):
        for approx in (True, False, (True, False), (False, True)):
            A.grad = B.grad = None
            cuda_bindings.pam(A, B, offset=off, approx_bwd=approx).backward(dY)
            ap = (approx, approx) if isinstance(approx, bool) else approx
            a, b, d = A.detach().numpy(), B.detach().numpy(), dY.numpy()
            want_a = oracle.pam(d, b, off) if ap[0] else oracle.pam_bwd(a, b, d, off)      # pam/cuda_bindings.py:47-55
            want_b = oracle.pam(d, a, off) if ap[1] else oracle.pam_bwd(b, a, d, off)
            assert_same_bits(A.grad.numpy(), want_a, f"dA {off} {approx}")
            assert_same_bits(B.grad.numpy(), want_b, f"dB {off} {approx}")
    # division: the GPU flavour of the formulas (pam/cuda_bindings.py:86-95)
    A.grad = B.grad = None
    cuda_bindings.pad(A, B, approx_bwd=True).backward(dY)
    a, b, d = A.detach().numpy(), B.detach().numpy(), dY.numpy()
    assert_same_bits(A.grad.numpy(), oracle.pam(oracle.pad(np.ones_like(b), b), d), "pad dA approx")
    assert_same_bits(B.grad.numpy(), -oracle.pam(oracle.pad(oracle.pad(a, b), b), d), "pad dB approx")
    A.grad = B.grad = None
    cuda_bindings.pad(A, B, approx_bwd=False).backward(dY)
    assert_same_bits(A.grad.numpy(), oracle.pam_bwd(a, oracle.pad(np.ones_like(b), b), d), "pad dA exact")
    assert_same_bits(B.grad.numpy(), oracle.pad_bwd(a, b, d), "pad dB exact")


def test_broadcast_and_scalars(fake, oracle):
    A = _t((4, 3), 5)
    out = cuda_bindings.pam(A, 2.0)
    assert_same_bits(out.detach().numpy(), A.detach().numpy() * 2.0, "x * 2")
    out.sum().backward()
    assert A.grad.shape == A.shape
    row = _t((3,), 6)
    out = cuda_bindings.pam(A, row, approx_bwd=True)
    out.backward(torch.ones_like(out))
    assert row.grad.shape == (3,)                 # autograd sums over the broadcast dimension
    assert_same_bits(row.grad.numpy(), oracle.pam(np.ones((4, 3), np.float32), A.detach().numpy()).sum(0), "broadcast grad")


def test_exp_log_autograd_formulas(fake, oracle):
    X = _t((6, 4), 7); dY = _t((6, 4), 8, grad=False)
    x, d = X.detach().numpy(), dY.numpy()
    for base in (math.e, 2.0, 10.0):
        X.grad = None
        y = cuda_bindings.pa_exp(X, base=base, approx_bwd=True); y.backward(dY)
        grad = oracle.pa_exp(x, base)
        if base != math.e:
            grad = oracle.pam(grad, np.full_like(x, math.log(base)))
        assert_same_bits(X.grad.numpy(), oracle.pam(grad, d), f"exp approx {base}")        # pam/cuda_bindings.py:228-235
        X.grad = None
        cuda_bindings.pa_exp(X, base=base, approx_bwd=False).backward(dY)
        assert_same_bits(X.grad.numpy(), oracle.pa_exp_bwd(x, d, base), f"exp exact {base}")
        Xp = X.detach().abs().requires_grad_()
        cuda_bindings.pa_log(Xp, base=base, approx_bwd=True).backward(dY)
        grad = oracle.pad(d, Xp.detach().numpy())
        if base != math.e:
            grad = oracle.pad(grad, np.full_like(x, math.log(base)))
        assert_same_bits(Xp.grad.numpy(), grad, f"log approx {base}")                    # pam/cuda_bindings.py:268-272
    assert_same_bits(cuda_bindings.pa_exp2(X).detach().numpy(), oracle.pa_exp(x, 2.0), "exp2")
    assert_same_bits(cuda_bindings.pa_log2(X.detach().abs()).numpy(), oracle.pa_log(np.abs(x), 2.0), "log2")


def test_check_row_major():
    t = torch.zeros(4, 6)
    assert cuda_bindings.check_row_major(t, 2)[1] is True
    v, rm = cuda_bindings.check_row_major(t.T, 2)
    assert rm is False and v.data_ptr() == t.data_ptr()              # a transposed view is passed on, not copied
    s = torch.zeros(4, 12)[:, ::2]
    c, rm = cuda_bindings.check_row_major(s, 2)
    assert rm is True and c.is_contiguous() and c.data_ptr() != s.data_ptr()
    with pytest.raises(ValueError):
        cuda_bindings.check_row_major(t, 3)
    q = torch.zeros(8, 6, 4).transpose(0, 1)                          # fairseq-style (B*H, T, D) view of (T, B*H, D)
    assert cuda_bindings.check_row_major(q, 3)[1] is True and cuda_bindings.check_row_major(q.transpose(1, 2), 3)[1] is False


def test_matmul_autograd_uses_views(fake, oracle):
    A = _t((9, 6), 9); Bt = _t((5, 6), 10)                 # B given as W.T, the nn.Linear case
    dY = _t((9, 5), 11, grad=False)
    a, b, d = A.detach().numpy(), Bt.detach().numpy().T, dY.numpy()
    Y = cuda_bindings.pam_matmul(A, Bt.T, approx_bwd=True)
    assert_same_bits(Y.detach().numpy(), oracle.gemm(a, b), "forward")
    Y.backward(dY)
    assert_same_bits(A.grad.numpy(), oracle.gemm(d, b.T), "dA = dY B^T")               # pam/cuda_bindings.py:155
    assert_same_bits(Bt.grad.numpy().T, oracle.gemm(a.T, d), "dB = A^T dY")            # pam/cuda_bindings.py:161
    fwd = [c for c in fake.calls if c[0] == "pam_matmul_fwd"]
    assert fwd[0][1:] == ((6, 1), (1, 6), True, False)       # X row-major, W.T column-major view
    assert fwd[1][1:] == ((5, 1), (6, 1), True, True)        # dY row-major, (W.T).mT = W row-major: no copy
    assert fwd[2][1:] == ((1, 6), (5, 1), False, True)       # X.mT column-major view, dY row-major
    A.grad = Bt.grad = None
    cuda_bindings.pam_matmul(A, Bt.T, approx_bwd=False).backward(dY)
    assert_same_bits(A.grad.numpy(), oracle.gemm(d, b.T, mode=oracle.MODE_BWD_DELTA_L, D=a), "exact dA")
    assert_same_bits(Bt.grad.numpy().T, oracle.gemm(a.T, d, mode=oracle.MODE_BWD_DELTA_R, D=b), "exact dB")
    # batched, tuple flag, standard product
    P, V = _t((3, 7, 4), 12), _t((3, 4, 6), 13); dO = _t((3, 7, 6), 14, grad=False)
    cuda_bindings.pam_bmm(P, V, approx_bwd=(True, False)).backward(dO)
    p, v, do = P.detach().numpy(), V.detach().numpy(), dO.numpy()
    assert_same_bits(P.grad.numpy(), oracle.gemm(do, np.swapaxes(v, 1, 2)), "bmm dA approx")
    assert_same_bits(V.grad.numpy(), oracle.gemm(np.swapaxes(p, 1, 2), do, mode=oracle.MODE_BWD_DELTA_R, D=v), "bmm dB exact")
    S = cuda_bindings.standard_matmul(A.detach(), Bt.detach().T, offset=1.5, approx_bwd=True)
    assert np.allclose(S.numpy(), a @ b, rtol=1e-5, atol=1e-6)


def test_op_library_surface(fake):
    for name in ("mul", "div", "exp", "exp2", "log", "log2", "pow", "matmul", "bmm", "linear", "Linear"):
        assert hasattr(pam_amd, name)
    x = torch.randn(3, 4)
    with pytest.raises(RuntimeError, match="GPU only"):
        pam_ops.mul(x, x)                                   # no CPU fallback in this package
    with pytest.raises(NotImplementedError):
        pam_ops.matmul(x, x.T, use_kernel=False)
    with pytest.raises(AssertionError):
        pam_ops.bmm(torch.zeros(2, 3, 4), torch.zeros(3, 4, 5))
    lin = pam_amd.Linear(8, 3, offset=1.0552, approx_bwd=True)
    ref = torch.nn.Linear(8, 3)
    lin.load_state_dict(ref.state_dict())                   # same parameters as torch.nn.Linear (pam/pam_ops.py:259-264)
    assert set(lin.state_dict()) == set(ref.state_dict())
    assert "offset=1.05520" in repr(lin) and "approx_bwd=True" in repr(lin) and repr(lin).startswith("pam.Linear")


def test_kernel_object_rejects_host_tensors():
    k = _abi.HipKernels()
    x = torch.randn(4, 4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):           # CHECK_CUDA, pam/cuda_kernels.cu:8
        k.pam_fwd(x, x, 1.0)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        k.pam_matmul_fwd(x, x, True, True, 1.0)


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU; asking for more ends with a message instead of a silent single-GPU run."""
    import pathlib
    import subprocess
    import sys
    root = pathlib.Path(__file__).resolve().parents[1]
    res = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode != 0 and "one GPU" in res.stderr and res.stdout.strip() == ""
