"""ctypes front end of libpam_oracle.so (numpy in, numpy out).

Test infrastructure only: the product never imports this module.
"""
import ctypes
import math
import pathlib
import subprocess

import numpy as np

_HERE = pathlib.Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libpam_oracle.so"


def build(force=False):
    """Compile the oracle with gcc (a second or two)."""
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < (_HERE / "pam_oracle.c").stat().st_mtime:
        subprocess.run(["make", "-s", "-B", "-C", str(_HERE)], check=True)
    return _LIB_PATH


_lib = None
_fp = ctypes.POINTER(ctypes.c_float)


def lib():
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        _lib = ctypes.CDLL(str(_LIB_PATH))
        L = _lib
        for name in ("pamo_pam", "pamo_pad", "pamo_pam_chain", "pamo_pad_chain",
                     "pamo_pam_chain_off", "pamo_pad_chain_off"):
            getattr(L, name).argtypes = [_fp, _fp, _fp, ctypes.c_size_t, ctypes.c_float]
            getattr(L, name).restype = None
        for name in ("pamo_pam_bwd", "pamo_pad_bwd"):
            getattr(L, name).argtypes = [_fp, _fp, _fp, _fp, ctypes.c_size_t, ctypes.c_float]
            getattr(L, name).restype = None
        for name in ("pamo_pa_log2", "pamo_pa_exp2"):
            getattr(L, name).argtypes = [_fp, _fp, ctypes.c_size_t]
            getattr(L, name).restype = None
        for name in ("pamo_pa_exp", "pamo_pa_log"):
            getattr(L, name).argtypes = [_fp, _fp, ctypes.c_size_t, ctypes.c_float, ctypes.c_float]
            getattr(L, name).restype = None
        for name in ("pamo_pa_exp_chain", "pamo_pa_log_chain"):
            getattr(L, name).argtypes = [_fp, _fp, ctypes.c_size_t, ctypes.c_float, ctypes.c_float, ctypes.c_int]
            getattr(L, name).restype = None
        for name in ("pamo_pa_exp_bwd", "pamo_pa_log_bwd"):
            getattr(L, name).argtypes = [_fp, _fp, _fp, ctypes.c_size_t, ctypes.c_float, ctypes.c_float]
            getattr(L, name).restype = None
        cl = ctypes.c_long
        L.pamo_gemm.argtypes = [ctypes.c_int, cl, cl, cl, cl,
                                _fp, cl, cl, cl, _fp, cl, cl, cl, _fp, cl, cl, cl, _fp, cl, cl, cl,
                                ctypes.c_float, cl, cl]
        L.pamo_gemm.restype = None
        L.pamo_gemm_fast.argtypes = [cl, cl, cl, _fp, _fp, _fp]
        L.pamo_gemm_fast.restype = None
        cf, ci = ctypes.c_float, ctypes.c_int
        L.pamo_softmax_fwd.argtypes = [_fp, _fp, _fp, _fp, cl, cl, cf]
        L.pamo_softmax_bwd.argtypes = [_fp, _fp, _fp, cf, _fp, cl, cl, cf, ci, ci, ci]
        L.pamo_logsumexp_fwd.argtypes = [_fp, _fp, _fp, cl, cl, cf]
        L.pamo_row_mean_fwd.argtypes = [_fp, _fp, cl, cl, cf]
        L.pamo_layer_norm_fwd.argtypes = [_fp, _fp, _fp, _fp, cl, cl, cf, cf]
        L.pamo_logsumexp_bwd.argtypes = [_fp, _fp, cf, _fp, cl, cl, ci, cf, ci, ci, ci]
        L.pamo_layer_norm_bwd.argtypes = [_fp, _fp, _fp, _fp, _fp, cl, cl, cf, cf, ci, ci, ci]
        L.pamo_logsumexp_bwd.restype = None; L.pamo_layer_norm_bwd.restype = None
        L.pamo_adam_step.argtypes = [_fp, _fp, _fp, _fp, ctypes.c_size_t, cf, cf, cf, cf, cf, cf, ci, cf, cf]
        L.pamo_adam_step.restype = None
        for name in ("pamo_softmax_fwd", "pamo_softmax_bwd", "pamo_logsumexp_fwd", "pamo_row_mean_fwd",
                     "pamo_layer_norm_fwd"):
            getattr(L, name).restype = None
    return _lib


def _f32(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32))


def _p(a):
    return a.ctypes.data_as(_fp)


def log2_base(base):
    """log2 of the base in fp32, as torch.log2(torch.tensor(base)) gives it."""
    return float(np.log2(np.float32(base), dtype=np.float32))


def _off(offset):
    return 1.0 if offset is None else float(np.float32(offset))


def _binary(fn, a, b, offset):
    a, b = np.broadcast_arrays(_f32(a), _f32(b))
    a, b = _f32(a), _f32(b)
    c = np.empty_like(a)
    getattr(lib(), fn)(_p(a), _p(b), _p(c), a.size, _off(offset))
    return c


def pam(a, b, offset=None):
    return _binary("pamo_pam", a, b, offset)


def pad(a, b, offset=None):
    return _binary("pamo_pad", a, b, offset)


def pam_chain(a, b, offset=None):
    return _binary("pamo_pam_chain" if offset is None else "pamo_pam_chain_off", a, b, offset)


def pad_chain(a, b, offset=None):
    return _binary("pamo_pad_chain" if offset is None else "pamo_pad_chain_off", a, b, offset)


def _ternary(fn, a, b, d, offset):
    a, b, d = np.broadcast_arrays(_f32(a), _f32(b), _f32(d))
    a, b, d = _f32(a), _f32(b), _f32(d)
    c = np.empty_like(a)
    getattr(lib(), fn)(_p(a), _p(b), _p(d), _p(c), a.size, _off(offset))
    return c


def pam_bwd(a, b, delta, offset=None):
    return _ternary("pamo_pam_bwd", a, b, delta, offset)


def pad_bwd(a, b, delta, offset=None):
    return _ternary("pamo_pad_bwd", a, b, delta, offset)


def pad_grads_native(a, b, delta, offset=None, flavour="chain"):
    """(dA, dB) of C = A (/) B as the reference's CPU autograd function computes them with approx_bwd=True
    (pam/native.py:173-188): dA = pad(delta, B) without the offset, dB = -pad(pam(A, delta), pam(B, B)), each of
    those three with the offset.  The GPU path of the reference, which this repository's kernels follow, uses other
    formulas (pam/cuda_bindings.py:78-97); PAM is not associative, so the two differ in the last bits.
    flavour "chain" models the float emulation of native.py bit for bit, "exact" is the integer definition."""
    mul, div = (pam_chain, pad_chain) if flavour == "chain" else (pam, pad)
    d_a = div(delta, b)
    d_b = -div(mul(a, delta, offset), mul(b, b, offset), offset)
    return d_a, d_b


def pa_log2_raw(x):
    x = _f32(x); y = np.empty_like(x)
    lib().pamo_pa_log2(_p(x), _p(y), x.size)
    return y


def pa_exp2_raw(x):
    x = _f32(x); y = np.empty_like(x)
    lib().pamo_pa_exp2(_p(x), _p(y), x.size)
    return y


def pa_exp(x, base=math.e, offset=None):
    x = _f32(x); y = np.empty_like(x)
    lib().pamo_pa_exp(_p(x), _p(y), x.size, log2_base(base), _off(offset))
    return y


def pa_log(x, base=math.e, offset=None):
    x = _f32(x); y = np.empty_like(x)
    lib().pamo_pa_log(_p(x), _p(y), x.size, log2_base(base), _off(offset))
    return y


def pa_exp_chain(x, base=math.e, offset=None):
    x = _f32(x); y = np.empty_like(x)
    lib().pamo_pa_exp_chain(_p(x), _p(y), x.size, log2_base(base), _off(offset), int(offset is not None))
    return y


def pa_log_chain(x, base=math.e, offset=None):
    x = _f32(x); y = np.empty_like(x)
    lib().pamo_pa_log_chain(_p(x), _p(y), x.size, log2_base(base), _off(offset), int(offset is not None))
    return y


def pa_exp_bwd(x, dy, base=math.e, offset=None):
    x, dy = np.broadcast_arrays(_f32(x), _f32(dy)); x, dy = _f32(x), _f32(dy)
    dx = np.empty_like(x)
    lib().pamo_pa_exp_bwd(_p(x), _p(dy), _p(dx), x.size, log2_base(base), _off(offset))
    return dx


def pa_log_bwd(x, dy, base=math.e, offset=None):
    x, dy = np.broadcast_arrays(_f32(x), _f32(dy)); x, dy = _f32(x), _f32(dy)
    dx = np.empty_like(x)
    lib().pamo_pa_log_bwd(_p(x), _p(dy), _p(dx), x.size, log2_base(base), _off(offset))
    return dx


MODE_PAM, MODE_STD, MODE_BWD_DELTA_L, MODE_BWD_DELTA_R = 0, 1, 2, 3


def _strides3(a):
    s = [st // 4 for st in a.strides]
    return (0, s[0], s[1]) if a.ndim == 2 else tuple(s)


def gemm(L, R, mode=MODE_PAM, D=None, offset=None, kchunk=0, kgroup=1):
    """Y = L (x) R for 2-D or 3-D (batched) float32 arrays of any strides."""
    L = np.asarray(L, dtype=np.float32); R = np.asarray(R, dtype=np.float32)
    batched = L.ndim == 3
    batch = L.shape[0] if batched else 1
    M, K = L.shape[-2:]; K2, N = R.shape[-2:]
    assert K == K2
    Y = np.empty(((batch, M, N) if batched else (M, N)), dtype=np.float32)
    if D is None:
        D = Y
    else:
        D = np.asarray(D, dtype=np.float32)
    lib().pamo_gemm(mode, batch, M, N, K,
                    _p(L), *_strides3(L), _p(R), *_strides3(R), _p(D), *_strides3(D),
                    _p(Y), *_strides3(Y), _off(offset), kchunk, kgroup)
    return Y


def gemm_fast(L, R):
    L = _f32(L); R = _f32(R)
    M, K = L.shape; _, N = R.shape
    Y = np.empty((M, N), dtype=np.float32)
    lib().pamo_gemm_fast(M, N, K, _p(L), _p(R), _p(Y))
    return Y


# ---- row-wise compositions over the last dimension (fixed summation order) ----

def _rows(x):
    x = _f32(x)
    n = x.shape[-1]
    return x.reshape(-1, n), x.shape


def softmax_fwd(x, offset=None):
    """Returns (y, row_sum[rows], shift)."""
    x2, shape = _rows(x)
    y = np.empty_like(x2); rs = np.empty(x2.shape[0], dtype=np.float32); shift = np.empty(1, dtype=np.float32)
    lib().pamo_softmax_fwd(_p(x2), _p(y), _p(rs), _p(shift), x2.shape[0], x2.shape[1], _off(offset))
    return y.reshape(shape), rs, shift[0]


def softmax_bwd(x, dy, row_sum, shift, offset=None, approx=(False, False, False)):
    x2, shape = _rows(x); dy2, _ = _rows(dy)
    rs = _f32(row_sum); dx = np.empty_like(x2)
    lib().pamo_softmax_bwd(_p(x2), _p(dy2), _p(rs), float(shift), _p(dx), x2.shape[0], x2.shape[1], _off(offset),
                           int(approx[0]), int(approx[1]), int(approx[2]))
    return dx.reshape(shape)


def logsumexp_fwd(x, offset=None, with_log_softmax=False):
    x2, shape = _rows(x)
    lse = np.empty(x2.shape[0], dtype=np.float32)
    y = np.empty_like(x2) if with_log_softmax else None
    lib().pamo_logsumexp_fwd(_p(x2), _p(lse), _p(y) if with_log_softmax else None, x2.shape[0], x2.shape[1], _off(offset))
    lse = lse.reshape(shape[:-1])
    return (lse, y.reshape(shape)) if with_log_softmax else lse


def row_mean_fwd(x, offset=None):
    x2, shape = _rows(x)
    y = np.empty(x2.shape[0], dtype=np.float32)
    lib().pamo_row_mean_fwd(_p(x2), _p(y), x2.shape[0], x2.shape[1], _off(offset))
    return y.reshape(shape[:-1])


def layer_norm_fwd(x, weight=None, bias=None, eps=1e-5, offset=None):
    x2, shape = _rows(x)
    w = None if weight is None else _f32(weight).ravel()
    b = None if bias is None else _f32(bias).ravel()
    y = np.empty_like(x2)
    lib().pamo_layer_norm_fwd(_p(x2), None if w is None else _p(w), None if b is None else _p(b), _p(y),
                              x2.shape[0], x2.shape[1], float(np.float32(eps)), _off(offset))
    return y.reshape(shape)


def adam_step(p, g, m, v, beta1, one_minus_beta1, beta2, one_minus_beta2, eps, decay, step_size, offset=None):
    """Returns the updated (p, m, v); decay None or 0 skips the weight-decay term."""
    p, g, m, v = (_f32(t).copy() for t in (p, g, m, v))
    f = lambda x: float(np.float32(x))
    lib().pamo_adam_step(_p(p), _p(g), _p(m), _p(v), p.size, f(beta1), f(one_minus_beta1), f(beta2), f(one_minus_beta2),
                         f(eps), f(decay or 0.0), int(bool(decay)), f(step_size), _off(offset))
    return p, m, v


def logsumexp_bwd(x, grad, shift, offset=None, approx=(False, False, False), log_softmax=False):
    """dx of logsumexp over the last dim (grad per row) or of log_softmax (grad per element)."""
    x2, shape = _rows(x)
    g = _f32(grad).reshape(x2.shape if log_softmax else (x2.shape[0],))
    dx = np.empty_like(x2)
    lib().pamo_logsumexp_bwd(_p(x2), _p(g), float(shift), _p(dx), x2.shape[0], x2.shape[1], int(log_softmax), _off(offset),
                             int(approx[0]), int(approx[1]), int(approx[2]))
    return dx.reshape(shape)


def layer_norm_bwd(x, weight, grad, eps=1e-5, offset=None, approx=(False, False, False)):
    """Returns (dx, dw_terms or None): dw_terms[rows, n] sums over rows to the weight gradient."""
    x2, shape = _rows(x); g, _ = _rows(grad)
    w = None if weight is None else _f32(weight).ravel()
    dx = np.empty_like(x2); dw = np.empty_like(x2) if w is not None else None
    lib().pamo_layer_norm_bwd(_p(x2), None if w is None else _p(w), _p(g), _p(dx), None if dw is None else _p(dw),
                              x2.shape[0], x2.shape[1], float(np.float32(eps)), _off(offset),
                              int(approx[0]), int(approx[1]), int(approx[2]))
    return dx.reshape(shape), dw
