"""ctypes binding of libpam_hip.so and the tensor-level kernel object built on it.

`HipKernels` exposes the fourteen functions of the reference's extension module
(pam/cuda_kernels.cu:932-947) with the same names, argument order and return convention
(a new tensor; inputs untouched).  PyTorch is used for device memory and the current
stream only.  There is no CPU fallback: a missing library or a non-GPU tensor raises.
"""
import ctypes
import pathlib

import torch

_LIB_PATH = pathlib.Path(__file__).resolve().parent / "lib" / "libpam_hip.so"

_f = ctypes.c_float
_p = ctypes.c_void_p
_l = ctypes.c_long
_z = ctypes.c_size_t
_i = ctypes.c_int

_MAT = [_p, _l, _l, _l]          # pointer, batch stride, row stride, col stride
_MAT2 = [_p, _l, _l]             # pointer, row stride, col stride

_SIGNATURES = {
    "pam_hip_abi_version": ([], _i),
    "pam_hip_last_error": ([], ctypes.c_char_p),
    "pam_hip_source_hash": ([], ctypes.c_char_p),
    "pam_hip_device_info": ([ctypes.POINTER(_i), ctypes.POINTER(_i)], _i),
    "pam_hip_pam_fwd": ([_p, _p, _p, _z, _f, _p], _i),
    "pam_hip_pam_bwd": ([_p, _p, _p, _p, _z, _f, _p], _i),
    "pam_hip_pad_fwd": ([_p, _p, _p, _z, _f, _p], _i),
    "pam_hip_pad_bwd": ([_p, _p, _p, _p, _z, _f, _p], _i),
    "pam_hip_pam_fwd_bcast": ([_p, _p, _i, _p, _z, _f, _p], _i),
    "pam_hip_pad_fwd_bcast": ([_p, _p, _i, _p, _z, _f, _p], _i),
    "pam_hip_log2_base": ([_f], _f),
    "pam_hip_pa_exp_fwd": ([_p, _p, _z, _f, _f, _p], _i),
    "pam_hip_pa_exp_bwd": ([_p, _p, _p, _z, _f, _f, _p], _i),
    "pam_hip_issue_probe": ([_p, _p, _i, _i, _p], _i),
    "pam_hip_issue_probe_lds": ([_p, _p, _i, _i, _i, _i, _p], _i),
    "pam_hip_pam_bwd_pair": ([_p, _p, _p, _p, _p, _z, _f, _i, _i, _p], _i),
    "pam_hip_pad_bwd_pair": ([_p, _p, _p, _p, _p, _z, _f, _i, _i, _p], _i),
    "pam_hip_pow_fwd": ([_p, _p, _z, _f, _f, _p], _i),
    "pam_hip_pow_bwd": ([_p, _p, _p, _z, _f, _f, _i, _i, _p], _i),
    "pam_hip_pa_log_fwd": ([_p, _p, _z, _f, _f, _p], _i),
    "pam_hip_pa_log_bwd": ([_p, _p, _p, _z, _f, _f, _p], _i),
    "pam_hip_gemm_workspace_bytes": ([_l, _l, _l, _l], _z),
    "pam_hip_gemm_plan": ([_l, _l, _l, _l, ctypes.POINTER(_i)], _i),
    "pam_hip_pam_matmul_fwd": (_MAT2 * 3 + [_l, _l, _l, _f, _p, _z, _p], _i),
    "pam_hip_pam_matmul_fwd_noalloc": (_MAT2 * 3 + [_l, _l, _l, _f, _p], _i),
    "pam_hip_pam_linear_fwd": (_MAT2 * 2 + [_p] + _MAT2 + [_l, _l, _l, _f, _p, _z, _p], _i),
    "pam_hip_pam_bmm_fwd": (_MAT * 3 + [_l, _l, _l, _l, _f, _p, _z, _p], _i),
    "pam_hip_standard_matmul": (_MAT2 * 3 + [_l, _l, _l, _f, _p, _z, _p], _i),
    "pam_hip_standard_bmm": (_MAT * 3 + [_l, _l, _l, _l, _f, _p, _z, _p], _i),
    "pam_hip_pam_matmul_bwd": (_MAT2 * 4 + [_l, _l, _l, _i, _f, _p, _z, _p], _i),
    "pam_hip_pam_bmm_bwd": (_MAT * 4 + [_l, _l, _l, _l, _i, _f, _p, _z, _p], _i),
    "pam_hip_conv2d_workspace_bytes": ([_l] * 12 + [_i, _f], _z),
    "pam_hip_conv2d_fwd": ([_p, _p, _p] + [_l] * 12 + [_f, _p, _z, _p], _i),
    "pam_hip_conv2d_bwd_weight": ([_p, _p, _p, _p] + [_l] * 12 + [_i, _f, _p, _z, _p], _i),
    "pam_hip_conv2d_bwd_input": ([_p, _p, _p, _p] + [_l] * 12 + [_i, _f, _p, _z, _p], _i),
    "pam_hip_adam_step": ([_p, _p, _p, _p, _z, _f, _f, _f, _f, _f, _f, _i, _f, _f, _p], _i),
    "pam_hip_rowop_workspace_bytes": ([], _z),
    "pam_hip_softmax_fwd": ([_p, _p, _p, _p, _l, _l, _f, _p, _z, _p], _i),
    "pam_hip_softmax_bwd": ([_p, _p, _p, _p, _p, _l, _l, _f, _i, _i, _i, _p], _i),
    "pam_hip_logsumexp_fwd": ([_p, _p, _p, _p, _l, _l, _f, _p, _z, _p], _i),
    "pam_hip_logsumexp_bwd": ([_p, _p, _p, _p, _l, _l, _i, _f, _i, _i, _i, _p], _i),
    "pam_hip_layer_norm_bwd": ([_p, _p, _p, _p, _p, _l, _l, _f, _f, _i, _i, _i, _p], _i),
    "pam_hip_row_mean_fwd": ([_p, _p, _l, _l, _f, _p], _i),
    "pam_hip_layer_norm_fwd": ([_p, _p, _p, _p, _l, _l, _f, _f, _p], _i),
}

_lib = None


def library_path():
    return _LIB_PATH


def load_library():
    """Loads libpam_hip.so; raises if it has not been built (python -m pam_amd.build)."""
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build the HIP extension first (python -m pam_amd.build). "
                "This package has no CPU or PyTorch fallback.")
        lib = ctypes.CDLL(str(_LIB_PATH))
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        if lib.pam_hip_abi_version() != 2:
            raise RuntimeError("libpam_hip.so has an unexpected ABI version")
        _lib = lib
    return _lib


def exported_symbols():
    return sorted(_SIGNATURES)


def _call(name, *args):
    lib = load_library()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.pam_hip_last_error().decode(errors="replace")
        raise (ValueError if rc == -1 else RuntimeError)(f"{name} failed ({rc}): {msg}")


def device_info():
    cu, khz = _i(0), _i(0)
    _call("pam_hip_device_info", ctypes.byref(cu), ctypes.byref(khz))
    return cu.value, khz.value


def gemm_plan(batch, m, n, k):
    """k_chunk: the fixed accumulation order used for this shape (see pam_hip_gemm_plan in include/pam_hip.h)."""
    c = _i(0)
    _call("pam_hip_gemm_plan", batch, m, n, k, ctypes.byref(c))
    return c.value


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)

# The matrix products' scratch (pieces of cut tiles, their arrival words): one buffer per device and stream, kept and
# grown as needed.  Products on one stream run one after the other, and each leaves the arrival words ready for the
# next one; products on different streams may overlap in time and must not share a buffer.
_workspaces = {}


def _gemm_workspace(device, nbytes):
    """Called with `device` current."""
    key = (device.index, _stream())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() * 4 < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20) // 4 + 64, dtype=torch.float32, device=device)
        _workspaces[key] = ws
    return ws


def _stream():
    """The current device's current stream as a hipStream_t value."""
    if _raw_stream is not None:                       # a plain integer, without building a Stream object
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


class _Current:
    """Stands in for torch.cuda.device(d) when d already is the current device."""

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_CURRENT = _Current()


def _on(device):
    """Context that makes `device` current for the launches inside it."""
    return _CURRENT if device.index is None or device.index == torch.cuda.current_device() else torch.cuda.device(device)


def _check(*tensors):
    for t in tensors:
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise RuntimeError("argument must be a CUDA tensor")      # CHECK_CUDA, pam/cuda_kernels.cu:8
        if t.dtype != torch.float32:
            raise TypeError(f"PAM kernels compute in float32, got {t.dtype}")


def _is_single_value(t):
    return t.numel() > 1 and all(s == 0 for s in t.stride())


def _flat(t):
    """Contiguous 1-D view; copies only when the tensor is not already contiguous
    (the reference's flatten(), pam/cuda_kernels.cu:163-165)."""
    return t.contiguous().view(-1)


class HipKernels:
    """The kernel object the autograd layer calls; same surface as the reference's
    `cuda_kernels` extension module."""

    # ---------------------------------------------------------------- elementwise
    @staticmethod
    def _binary(name, A, B, offset):
        _check(A, B)
        if A.shape != B.shape:
            raise ValueError(f"{name}: operands must have the same shape, got {tuple(A.shape)} and {tuple(B.shape)}")
        out = torch.empty(A.shape, dtype=torch.float32, device=A.device)
        n = out.numel()
        if n == 0:
            return out
        with _on(A.device):
            if name in ("pam_fwd", "pad_fwd") and (_is_single_value(A) or _is_single_value(B)):
                scalar_is_a = _is_single_value(A)
                s, x = (A, B) if scalar_is_a else (B, A)
                if _is_single_value(x):
                    x = x.contiguous()
                x = _flat(x)
                _call(f"pam_hip_{name}_bcast", x.data_ptr(), s.data_ptr(), int(scalar_is_a), out.data_ptr(), n,
                      float(offset), _stream())
            else:
                a, b = _flat(A), _flat(B)
                _call(f"pam_hip_{name}", a.data_ptr(), b.data_ptr(), out.data_ptr(), n, float(offset), _stream())
        return out

    @staticmethod
    def _ternary(name, A, B, dC, offset):
        _check(A, B, dC)
        if not (A.shape == B.shape == dC.shape):
            raise ValueError(f"{name}: operands must have the same shape")
        out = torch.empty(A.shape, dtype=torch.float32, device=A.device)
        n = out.numel()
        if n:
            a, b, d = _flat(A), _flat(B), _flat(dC)
            with _on(A.device):
                _call(f"pam_hip_{name}", a.data_ptr(), b.data_ptr(), d.data_ptr(), out.data_ptr(), n, float(offset), _stream())
        return out

    def pam_fwd(self, A, B, offset):
        return self._binary("pam_fwd", A, B, offset)

    def pad_fwd(self, A, B, offset):
        return self._binary("pad_fwd", A, B, offset)

    def pam_bwd(self, A, B, dC, offset):
        return self._ternary("pam_bwd", A, B, dC, offset)

    @staticmethod
    def _pair(name, A, B, dC, offset, approx_a, approx_b):
        _check(A, B, dC)
        if not (A.shape == B.shape == dC.shape):
            raise ValueError(f"{name}: operands must have the same shape")
        dA = torch.empty(A.shape, dtype=torch.float32, device=A.device)
        dB = torch.empty(A.shape, dtype=torch.float32, device=A.device)
        if dA.numel():
            a, b, d = _flat(A), _flat(B), _flat(dC)
            with _on(A.device):
                _call(f"pam_hip_{name}", a.data_ptr(), b.data_ptr(), d.data_ptr(), dA.data_ptr(), dB.data_ptr(), dA.numel(),
                      float(offset), int(bool(approx_a)), int(bool(approx_b)), _stream())
        return dA, dB

    def pam_bwd_pair(self, A, B, dC, offset, approx_a, approx_b):
        """(dA, dB) of C = A (*) B in one pass; not part of the reference's extension surface."""
        return self._pair("pam_bwd_pair", A, B, dC, offset, approx_a, approx_b)

    def pad_bwd_pair(self, A, B, dC, offset, approx_a, approx_b):
        """(dA, dB) of C = A (/) B in one pass; not part of the reference's extension surface."""
        return self._pair("pad_bwd_pair", A, B, dC, offset, approx_a, approx_b)

    def pad_bwd(self, A, B, dC, offset):
        return self._ternary("pad_bwd", A, B, dC, offset)

    # ---------------------------------------------------------------- exp / log
    @staticmethod
    def _unary(name, X, base, offset, dY=None):
        _check(X) if dY is None else _check(X, dY)
        out = torch.empty(X.shape, dtype=torch.float32, device=X.device)
        n = out.numel()
        if n:
            x = _flat(X)
            with _on(X.device):
                if dY is None:
                    _call(f"pam_hip_{name}", x.data_ptr(), out.data_ptr(), n, float(base), float(offset), _stream())
                else:
                    d = _flat(dY)
                    _call(f"pam_hip_{name}", x.data_ptr(), d.data_ptr(), out.data_ptr(), n, float(base), float(offset), _stream())
        return out

    def pa_exp_fwd(self, X, base, offset):
        return self._unary("pa_exp_fwd", X, base, offset)

    def pa_log_fwd(self, X, base, offset):
        return self._unary("pa_log_fwd", X, base, offset)

    def pa_exp_bwd(self, X, dY, base, offset):
        return self._unary("pa_exp_bwd", X, base, offset, dY)

    def pa_log_bwd(self, X, dY, base, offset):
        return self._unary("pa_log_bwd", X, base, offset, dY)

    # ---------------------------------------------------------------- matrix products
    @staticmethod
    def _mat(t, batched):
        s = t.stride()
        return (t.data_ptr(), s[0], s[1], s[2]) if batched else (t.data_ptr(), s[0], s[1])

    @classmethod
    def _product(cls, name, batched, L, R, Mop, extra, offset):
        ops = (L, R) if Mop is None else (L, R, Mop)
        _check(*ops)
        nd = 3 if batched else 2
        if any(t.dim() != nd for t in ops):
            raise ValueError(f"{name}: expected {nd}-D operands")
        if L.shape[-1] != R.shape[-2] or (batched and L.shape[0] != R.shape[0]):
            raise ValueError(f"{name}: shapes {tuple(L.shape)} and {tuple(R.shape)} do not multiply")
        batch = L.shape[0] if batched else 1
        m, k, n = L.shape[-2], L.shape[-1], R.shape[-1]
        if Mop is not None and tuple(Mop.shape[-2:]) != (m, n):
            raise ValueError(f"{name}: third operand must have the shape of the result")
        out = torch.empty((batch, m, n) if batched else (m, n), dtype=torch.float32, device=L.device)
        if out.numel() == 0:
            return out
        with _on(L.device):
            lib = load_library()
            ws_bytes = lib.pam_hip_gemm_workspace_bytes(batch, m, n, k)
            ws = _gemm_workspace(L.device, ws_bytes) if ws_bytes else None
            args = []
            for t in ops:
                args += cls._mat(t, batched)
            args += cls._mat(out, batched)
            args += ([batch] if batched else []) + [m, n, k] + extra + [float(offset)]
            args += [ws.data_ptr() if ws is not None else None, ws_bytes, _stream()]
            _call(f"pam_hip_{name}", *args)
        return out

    def pam_matmul_fwd(self, A, B, A_row_major, B_row_major, offset):
        # the layout flags of the reference select a kernel instance there; here the strides do
        return self._product("pam_matmul_fwd", False, A, B, None, [], offset)

    def pam_bmm_fwd(self, A, B, A_row_major, B_row_major, offset):
        return self._product("pam_bmm_fwd", True, A, B, None, [], offset)

    def standard_matmul(self, A, B, A_row_major, B_row_major, offset):
        return self._product("standard_matmul", False, A, B, None, [], offset)

    def standard_bmm(self, A, B, A_row_major, B_row_major, offset):
        return self._product("standard_bmm", True, A, B, None, [], offset)

    def pam_matmul_bwd(self, L, R, M, L_row_major, R_row_major, delta_L, offset):
        return self._product("pam_matmul_bwd", False, L, R, M, [int(bool(delta_L))], offset)

    def pam_bmm_bwd(self, L, R, M, L_row_major, R_row_major, delta_L, offset):
        return self._product("pam_bmm_bwd", True, L, R, M, [int(bool(delta_L))], offset)


class HipRowKernels:
    """Row-wise compositions over the last dimension of a contiguous [rows, n] tensor, one
    kernel each (softmax forward and backward, logsumexp / log_softmax, row mean,
    layer_norm); the order of their row sums is the one include/pam_hip.h states."""

    @staticmethod
    def _rows(name, X, *others):
        _check(X, *[t for t in others if t is not None])
        if X.dim() != 2 or not X.is_contiguous():
            raise ValueError(f"{name}: expected a contiguous 2-D tensor")
        for t in others:
            if t is not None and not t.is_contiguous():
                raise ValueError(f"{name}: operands must be contiguous")
        return X.shape

    @staticmethod
    def _workspace(device):
        nbytes = load_library().pam_hip_rowop_workspace_bytes()
        return torch.empty(nbytes // 4, dtype=torch.float32, device=device), nbytes

    def softmax_fwd(self, X, offset):
        rows, n = self._rows("softmax_fwd", X)
        Y = torch.empty_like(X)
        row_sum = torch.empty(rows, dtype=torch.float32, device=X.device)
        shift = torch.empty(1, dtype=torch.float32, device=X.device)
        if X.numel():
            with _on(X.device):
                ws, nbytes = self._workspace(X.device)
                _call("pam_hip_softmax_fwd", X.data_ptr(), Y.data_ptr(), row_sum.data_ptr(), shift.data_ptr(), rows, n,
                      float(offset), ws.data_ptr(), nbytes, _stream())
        return Y, row_sum, shift

    def softmax_bwd(self, X, dY, row_sum, shift, offset, approx_a, approx_b, approx_exp):
        rows, n = self._rows("softmax_bwd", X, dY, row_sum, shift)
        if dY.shape != X.shape or row_sum.numel() != rows or shift.numel() != 1:
            raise ValueError("softmax_bwd: operand shapes do not match")
        dX = torch.empty_like(X)
        if X.numel():
            with _on(X.device):
                _call("pam_hip_softmax_bwd", X.data_ptr(), dY.data_ptr(), row_sum.data_ptr(), shift.data_ptr(),
                      dX.data_ptr(), rows, n, float(offset), int(bool(approx_a)), int(bool(approx_b)),
                      int(bool(approx_exp)), _stream())
        return dX

    def logsumexp_fwd(self, X, offset, want_lse=True, want_log_softmax=False):
        """Returns (lse or None, log_softmax or None, shift)."""
        rows, n = self._rows("logsumexp_fwd", X)
        lse = torch.empty(rows, dtype=torch.float32, device=X.device) if want_lse else None
        Y = torch.empty_like(X) if want_log_softmax else None
        shift = torch.empty(1, dtype=torch.float32, device=X.device)
        if X.numel():
            with _on(X.device):
                ws, nbytes = self._workspace(X.device)
                _call("pam_hip_logsumexp_fwd", X.data_ptr(), lse.data_ptr() if want_lse else None,
                      Y.data_ptr() if want_log_softmax else None, shift.data_ptr(), rows, n, float(offset),
                      ws.data_ptr(), nbytes, _stream())
        return lse, Y, shift


    def logsumexp_bwd(self, X, grad, shift, offset, approx_a, approx_b, approx_exp, log_softmax):
        rows, n = self._rows("logsumexp_bwd", X, grad, shift)
        if grad.numel() != (X.numel() if log_softmax else rows):
            raise ValueError("logsumexp_bwd: gradient has the wrong size")
        dX = torch.empty_like(X)
        if X.numel():
            with _on(X.device):
                _call("pam_hip_logsumexp_bwd", X.data_ptr(), grad.data_ptr(), shift.data_ptr(), dX.data_ptr(), rows, n,
                      int(bool(log_softmax)), float(offset), int(bool(approx_a)), int(bool(approx_b)), int(bool(approx_exp)),
                      _stream())
        return dX

    def layer_norm_bwd(self, X, weight, dY, eps, offset, approx_a, approx_b, approx_exp, want_weight_terms):
        """Returns (dX, per-element weight-gradient terms or None)."""
        rows, n = self._rows("layer_norm_bwd", X, weight, dY)
        if dY.shape != X.shape or (weight is not None and weight.numel() != n):
            raise ValueError("layer_norm_bwd: operand shapes do not match")
        dX = torch.empty_like(X)
        terms = torch.empty_like(X) if (want_weight_terms and weight is not None) else None
        if X.numel():
            with _on(X.device):
                _call("pam_hip_layer_norm_bwd", X.data_ptr(), None if weight is None else weight.data_ptr(), dY.data_ptr(),
                      dX.data_ptr(), None if terms is None else terms.data_ptr(), rows, n, float(eps), float(offset),
                      int(bool(approx_a)), int(bool(approx_b)), int(bool(approx_exp)), _stream())
        return dX, terms

    def row_mean_fwd(self, X, offset):
        rows, n = self._rows("row_mean_fwd", X)
        Y = torch.empty(rows, dtype=torch.float32, device=X.device)
        if rows:
            with _on(X.device):
                _call("pam_hip_row_mean_fwd", X.data_ptr(), Y.data_ptr(), rows, n, float(offset), _stream())
        return Y

    def layer_norm_fwd(self, X, weight, bias, eps, offset):
        rows, n = self._rows("layer_norm_fwd", X, weight, bias)
        for t in (weight, bias):
            if t is not None and t.numel() != n:
                raise ValueError("layer_norm_fwd: weight and bias must have one value per column")
        Y = torch.empty_like(X)
        if X.numel():
            with _on(X.device):
                _call("pam_hip_layer_norm_fwd", X.data_ptr(), None if weight is None else weight.data_ptr(),
                      None if bias is None else bias.data_ptr(), Y.data_ptr(), rows, n, float(eps), float(offset), _stream())
        return Y


def issue_probe(work_groups_per_cu, iters=400, lds_tile=None):
    """T lane-operations per second of product-accumulate pairs (v_add_u32 + dependent v_add_f32) with that many
    256-lane work-groups per compute unit (= wavefronts per SIMD): operands in registers, or, with
    lds_tile=(tm, tn), read from LDS per step as the matrix kernel's inner loop reads them."""
    cus, _ = device_info()
    blocks = cus * work_groups_per_cu
    seed = torch.full((1024,), 2.0 ** -20, dtype=torch.float32, device="cuda")
    out = torch.empty(blocks * 256, dtype=torch.float32, device="cuda")

    def launch(n):
        if lds_tile is None:
            _call("pam_hip_issue_probe", seed.data_ptr(), out.data_ptr(), blocks, n, _stream())
        else:
            _call("pam_hip_issue_probe_lds", seed.data_ptr(), out.data_ptr(), blocks, n, lds_tile[0], lds_tile[1], _stream())

    pairs = 128 if lds_tile is None else 32 * lds_tile[0] * lds_tile[1]
    if lds_tile is not None:
        iters = max(1, iters * 128 // pairs)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    launch(2)
    torch.cuda.synchronize()
    start.record()
    launch(iters)
    stop.record(); stop.synchronize()
    return blocks * 256.0 * iters * pairs * 2 / (start.elapsed_time(stop) * 1e-3) / 1e12


def pow_fwd(X, exponent, offset):
    """X ** exponent (scalar) in one pass: exp2(log2(X) (*) exponent), zero where X is zero."""
    return HipKernels._unary("pow_fwd", X, exponent, offset)


def pow_bwd(X, dY, exponent, offset, approx_a, approx_exp):
    """The gradient for X of pow_fwd, the chain through select, exp2, product and log2 in one pass."""
    _check(X, dY)
    out = torch.empty(X.shape, dtype=torch.float32, device=X.device)
    if out.numel():
        x, d = _flat(X), _flat(dY)
        with _on(X.device):
            _call("pam_hip_pow_bwd", x.data_ptr(), d.data_ptr(), out.data_ptr(), out.numel(), float(exponent), float(offset),
                  int(bool(approx_a)), int(bool(approx_exp)), _stream())
    return out


def adam_step(p, g, m, v, beta1, one_minus_beta1, beta2, one_minus_beta2, eps, decay, step_size, offset):
    """In-place Adam update of the contiguous fp32 GPU tensors p, m, v from the gradient g;
    decay None or 0 skips the weight-decay term."""
    _check(p, g, m, v)
    if not (p.is_contiguous() and g.is_contiguous() and m.is_contiguous() and v.is_contiguous()):
        raise ValueError("adam_step: tensors must be contiguous")
    if not (p.shape == g.shape == m.shape == v.shape):
        raise ValueError("adam_step: tensors must have the same shape")
    if p.numel():
        with _on(p.device):
            _call("pam_hip_adam_step", p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), p.numel(), float(beta1),
                  float(one_minus_beta1), float(beta2), float(one_minus_beta2), float(eps), float(decay or 0.0),
                  int(bool(decay)), float(step_size), float(offset), _stream())


def _conv_geometry(X, W, stride, padding, groups=1):
    if X.dim() != 4 or W.dim() != 4 or groups < 1 or X.shape[1] != W.shape[1] * groups or W.shape[0] % groups:
        raise ValueError("conv2d: expected X[batch, c, h, w] and W[co, c / groups, kh, kw]")
    batch, c, h, w = X.shape
    co, _, kh, kw = W.shape
    return [batch, c, h, w, co, kh, kw, stride[0], stride[1], padding[0], padding[1], groups]


def conv2d_fwd(X, W, stride, padding, offset, groups=1):
    """Y[batch, co, ho, wo] for contiguous fp32 GPU tensors, dilation 1; the image patches are read in place."""
    _check(X, W)
    X, W = X.contiguous(), W.contiguous()
    geo = _conv_geometry(X, W, stride, padding, groups)
    batch, c, h, w, co, kh, kw, sh, sw, ph, pw, _ = geo
    ho, wo = (h + 2 * ph - kh) // sh + 1, (w + 2 * pw - kw) // sw + 1
    Y = torch.empty((batch, co, ho, wo), dtype=torch.float32, device=X.device)
    if Y.numel():
        with _on(X.device):
            nbytes = load_library().pam_hip_conv2d_workspace_bytes(*geo, 0, float(offset))
            ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=X.device)
            _call("pam_hip_conv2d_fwd", X.data_ptr(), W.data_ptr(), Y.data_ptr(), *geo, float(offset), ws.data_ptr(), nbytes, _stream())
    return Y


def conv2d_bwd_weight(X, dY, W, stride, padding, exact, offset, groups=1):
    """Per-image weight gradients [batch, co, (c / groups)*kh*kw]; W is only read by the exact variant."""
    _check(X, dY, W)
    X, dY, W = X.contiguous(), dY.contiguous(), W.contiguous()
    geo = _conv_geometry(X, W, stride, padding, groups)
    batch, c, _, _, co, kh, kw = geo[:7]
    dW = torch.empty((batch, co, c // groups * kh * kw), dtype=torch.float32, device=X.device)
    if dW.numel():
        with _on(X.device):
            nbytes = load_library().pam_hip_conv2d_workspace_bytes(*geo, 1, float(offset))
            ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=X.device)
            _call("pam_hip_conv2d_bwd_weight", X.data_ptr(), dY.data_ptr(), W.data_ptr(), dW.data_ptr(), *geo,
                  int(bool(exact)), float(offset), ws.data_ptr(), nbytes, _stream())
    return dW


def conv2d_bwd_input(dY, W, X, padding, exact, offset, groups=1):
    """dX[batch, c, h, w] of a stride-1 convolution with dY's patches read in place; X gives the
    shape and, for the exact variant, the values."""
    _check(dY, W, X)
    dY, W, X = dY.contiguous(), W.contiguous(), X.contiguous()
    geo = _conv_geometry(X, W, (1, 1), padding, groups)
    dX = torch.empty_like(X)
    if dX.numel():
        with _on(X.device):
            nbytes = load_library().pam_hip_conv2d_workspace_bytes(*geo, 2, float(offset))
            if nbytes == 0:
                raise ValueError("conv2d_bwd_input: needs stride 1 and padding <= kernel - 1")
            ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=X.device)
            _call("pam_hip_conv2d_bwd_input", dY.data_ptr(), W.data_ptr(), X.data_ptr(), dX.data_ptr(), *geo,
                  int(bool(exact)), float(offset), ws.data_ptr(), nbytes, _stream())
    return dX


def linear_fwd(X, Wt, bias, offset):
    """X[m, k] (x) Wt[k, n] + bias[n] in one pass (any strides for X and Wt; bias contiguous or None)."""
    _check(X, Wt) if bias is None else _check(X, Wt, bias)
    if X.dim() != 2 or Wt.dim() != 2 or X.shape[1] != Wt.shape[0]:
        raise ValueError(f"linear_fwd: shapes {tuple(X.shape)} and {tuple(Wt.shape)} do not multiply")
    m, k = X.shape
    n = Wt.shape[1]
    if bias is not None and (bias.numel() != n or not bias.is_contiguous()):
        raise ValueError("linear_fwd: bias must be contiguous with one value per output column")
    out = torch.empty((m, n), dtype=torch.float32, device=X.device)
    if out.numel():
        with _on(X.device):
            ws_bytes = load_library().pam_hip_gemm_workspace_bytes(1, m, n, k)
            ws = _gemm_workspace(X.device, ws_bytes) if ws_bytes else None
            _call("pam_hip_pam_linear_fwd", X.data_ptr(), X.stride(0), X.stride(1), Wt.data_ptr(), Wt.stride(0), Wt.stride(1),
                  None if bias is None else bias.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1), m, n, k,
                  float(offset), ws.data_ptr() if ws is not None else None, ws_bytes, _stream())
    return out
