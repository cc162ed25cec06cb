"""Writes the golden vectors under tests/golden/ from the reference's CPU implementation.

Runs only in the build container, where the reference checkout is mounted at
/root/reference; it is the one file in this repository that touches that path.
pam/native.py is imported in script mode (its own `import utils` branch,
pam/native.py:4-6) because importing the package would start the nvcc build of
pam/cuda_bindings.py:19-25.  Only inputs and outputs are stored, as uint32 bit
patterns, so that signed zeros and NaNs survive.

    python tests/golden/make_goldens.py            # writes tests/golden/*.npz
    python tests/golden/make_goldens.py pad_bwd    # only the file(s) of the named section(s)

Functions covered are those that nothing but running the reference can pin: the
output bits of native.pam_fwd / pad_fwd on full-mantissa inputs, the edge-class grid,
get_exp_mantissa just below powers of two, pam_bwd, pa_exp/pa_log, and pam_matmul.
"""
import math
import pathlib
import sys
import time

import numpy as np
import torch

REF = pathlib.Path("/root/reference/pam")
OUT = pathlib.Path(__file__).resolve().parent


def u32(t):
    return t.detach().contiguous().view(torch.int32).numpy().view(np.uint32).copy()


def from_u32(a):
    return torch.from_numpy(np.asarray(a, dtype=np.uint32).view(np.float32).copy())


def edge_values():
    f = np.float32
    vals = [0.0, 1.0, 1.5, 1.9999999, 2.0, 3.0, 0.75, 1e-30, 1e30, 1e-20, 1e20,
            2.0 ** -100, 2.0 ** 100, 1.2345, 3.4e38, 1.7e38, 1.2e-38, 2.4e-38, 2.0 ** -126,
            2.0 ** -63, 2.0 ** 64, 2.0 ** 127, 1.99 * 2.0 ** -64]
    bits = [0x00000001, 0x00000002, 0x00000003, 0x00400000, 0x00555555, 0x007fffff, 0x00000100,
            0x00800000, 0x00800001, 0x7f7fffff, 0x7f000000, 0x7effffff, 0x3f7fffff, 0x3fffffff,
            0x7f800000, 0x7fc00000]
    mags = list(np.array(vals, dtype=f).view(np.uint32)) + bits
    out = []
    for m in mags:
        out += [int(m), int(m) | 0x80000000]
    return np.array(sorted(set(out)), dtype=np.uint32)


def main():
    if not REF.exists():
        sys.exit("reference checkout not present; goldens can only be written in the build container")
    sys.path.insert(0, str(REF))
    import native  # noqa: E402  (the reference's CPU implementation)

    torch.manual_seed(0)
    torch.set_num_threads(8)
    OFF = 1.0552
    only = set(sys.argv[1:])
    if only == {"pad_bwd"}:
        return pad_bwd_section(native, OFF)

    # ---- 1. edge-class grid: all pairs of edge values
    ev = edge_values()
    A = from_u32(np.repeat(ev, len(ev)))
    B = from_u32(np.tile(ev, len(ev)))
    np.savez_compressed(
        OUT / "edge_grid.npz", values=ev,
        pam=u32(native.pam_fwd(A, B)), pad=u32(native.pad_fwd(A, B)),
        pam_off=u32(native.pam_fwd(A, B, offset=OFF)), pad_off=u32(native.pad_fwd(A, B, offset=OFF)),
        offset=np.float32(OFF))

    # ---- 2. short-mantissa operands (native's float chain is exact there)
    g = torch.Generator().manual_seed(1)
    n = 8192
    def short(nbits, emax):
        e = torch.randint(-emax, emax + 1, (n,), generator=g)
        m = torch.randint(0, 1 << nbits, (n,), generator=g).float() / (1 << nbits)
        s = torch.randint(0, 2, (n,), generator=g).float() * 2 - 1
        return s * (2.0 ** e.float()) * (1 + m)
    A = short(12, 50); B = short(12, 50); D = short(8, 10)
    np.savez_compressed(
        OUT / "short_mantissa.npz", a=u32(A), b=u32(B), d=u32(D),
        pam=u32(native.pam_fwd(A, B)), pad=u32(native.pad_fwd(A, B)),
        pam_bwd=u32(native.pam_bwd(A, B, D)),
        pam_off=u32(native.pam_fwd(A, B, offset=OFF)), pad_off=u32(native.pad_fwd(A, B, offset=OFF)),
        offset=np.float32(OFF))

    # ---- 3. full-mantissa N(0,1) and wide-exponent operands
    g = torch.Generator().manual_seed(2)
    n = 32768
    A = torch.randn(n, generator=g); B = torch.randn(n, generator=g); D = torch.randn(n, generator=g)
    A[n // 2:] *= 2.0 ** torch.randint(-40, 40, (n // 2,), generator=g).float()
    B[n // 2:] *= 2.0 ** torch.randint(-40, 40, (n // 2,), generator=g).float()
    np.savez_compressed(
        OUT / "normal_fullmant.npz", a=u32(A), b=u32(B), d=u32(D),
        pam=u32(native.pam_fwd(A, B)), pad=u32(native.pad_fwd(A, B)),
        pam_off=u32(native.pam_fwd(A, B, offset=OFF)), pad_off=u32(native.pad_fwd(A, B, offset=OFF)),
        pam_bwd=u32(native.pam_bwd(A, B, D)), pam_bwd_off=u32(native.pam_bwd(A, B, D, offset=OFF)),
        offset=np.float32(OFF))

    # ---- 4. just below / at / above powers of two (the floor(log2) band)
    ks = np.arange(-126, 128)
    p2 = (np.float32(2.0) ** ks.astype(np.float32)).astype(np.float32)
    band = np.concatenate([np.nextafter(p2, np.float32(0)), p2, np.nextafter(p2, np.float32(np.inf))]).astype(np.float32)
    X = torch.from_numpy(band)
    e, m = native.get_exp_mantissa(X)
    Bc = torch.full_like(X, 1.75); Dc = torch.full_like(X, 3.0)
    np.savez_compressed(
        OUT / "pow2_band.npz", x=u32(X), exp=u32(e), mant=u32(m), pa_log2=u32(native.pa_log2_fwd(X)),
        pam_bwd_a=u32(native.pam_bwd(X, Bc, Dc)), pam_bwd_b=u32(native.pam_bwd(Bc, X, Dc)),
        pam=u32(native.pam_fwd(X, Bc)))

    # ---- 5. pa_log2 / pa_exp2 / pa_exp / pa_log
    g = torch.Generator().manual_seed(3)
    xs = torch.cat([
        torch.linspace(-160, 160, 2049), torch.randn(4096, generator=g) * 8,
        torch.randn(2048, generator=g) * 0.01, from_u32(ev),
        torch.tensor([127.5, 128.0, 127.99999, -149.0, -149.5, -150.0, -150.5, -126.0, -126.5, 2.0 ** 23,
                      2.0 ** 24, 2.0 ** 25, 1e30, -1e30, -2.0 ** 24])])
    xl = torch.cat([
        torch.rand(4096, generator=g) * 10, torch.randn(2048, generator=g).abs() * 1e-3,
        2.0 ** (torch.rand(2048, generator=g) * 250 - 125), from_u32(ev)])
    d = {"x_exp": u32(xs), "x_log": u32(xl),
         "pa_exp2_fwd": u32(native.pa_exp2_fwd(xs)), "pa_log2_fwd": u32(native.pa_log2_fwd(xl))}
    for name, base in (("e", math.e), ("2", 2.0), ("10", 10.0)):
        d[f"exp_{name}"] = u32(native.pa_exp_fwd(xs, base))
        d[f"log_{name}"] = u32(native.pa_log_fwd(xl, base))
        d[f"exp_{name}_off"] = u32(native.pa_exp_fwd(xs, base, offset=OFF))
        d[f"log_{name}_off"] = u32(native.pa_log_fwd(xl, base, offset=OFF))
    d["offset"] = np.float32(OFF)
    np.savez_compressed(OUT / "exp_log.npz", **d)

    # ---- 6. the reference's own small deterministic matmul (pam/test_pam.py:96-97,129-130)
    d = {}
    for tag, shift in (("p21", 2.1), ("p20", 2.0)):
        A1 = (torch.arange(20) ** 3 % 7 - shift).reshape((5, 4)).requires_grad_()
        B1 = (torch.arange(12) ** 2 % 5 - shift).reshape((3, 4)).T.requires_grad_()
        C = native.pam_matmul(A1, B1)                       # exact backward (approx_bwd=False)
        C.sum().backward()
        d[f"{tag}_a"] = u32(A1); d[f"{tag}_b"] = u32(B1.detach().contiguous()); d[f"{tag}_c"] = u32(C)
        d[f"{tag}_da_exact_sum"] = u32(A1.grad); d[f"{tag}_db_exact_sum"] = u32(B1.grad.contiguous())
        A2 = A1.detach().clone().requires_grad_(); B2 = B1.detach().clone().requires_grad_()
        C2 = native.pam_matmul(A2, B2, approx_bwd=True)
        delta = torch.arange(C2.numel()).float().reshape_as(C2)
        C2.backward(delta)
        d[f"{tag}_delta"] = u32(delta)
        d[f"{tag}_da_approx"] = u32(A2.grad); d[f"{tag}_db_approx"] = u32(B2.grad.contiguous())
    np.savez_compressed(OUT / "matmul_small.npz", **d)

    # ---- 7. benchmark configuration 0: A[256,512] @ B[512,256], seeds 0/1/2, fwd + approx bwd
    A = torch.randn(256, 512, generator=torch.Generator().manual_seed(0)).requires_grad_()
    B = torch.randn(512, 256, generator=torch.Generator().manual_seed(1)).requires_grad_()
    dY = torch.randn(256, 256, generator=torch.Generator().manual_seed(2))
    t0 = time.perf_counter()
    Y = native.pam_matmul(A, B, approx_bwd=True)
    t1 = time.perf_counter()
    Y.backward(dY)
    t2 = time.perf_counter()
    # inputs are regenerable from the seeds; a checksum guards against a changed RNG
    np.savez_compressed(
        OUT / "matmul_c0.npz", y=u32(Y), da_rows=u32(A.grad[::8]), db_rows=u32(B.grad[::8]),
        a_head=u32(A.detach()[0, :8]), b_head=u32(B.detach()[0, :8]), dy_head=u32(dY[0, :8]))
    print(f"native.pam_matmul config 0: fwd {t1 - t0:.3f} s, approx bwd {t2 - t1:.3f} s, "
          f"{torch.get_num_threads()} threads")

    pad_bwd_section(native, OFF)

    # ---- timing of the elementwise reference path (for the baseline table)
    for n_log in (24,):
        n = 1 << n_log
        A = torch.randn(n, generator=torch.Generator().manual_seed(10))
        B = torch.randn(n, generator=torch.Generator().manual_seed(11))
        for name, fn in (("pam_fwd", native.pam_fwd), ("pad_fwd", native.pad_fwd)):
            ts = []
            for _ in range(3):
                t0 = time.perf_counter(); fn(A, B); ts.append(time.perf_counter() - t0)
            t = sorted(ts)[1]
            print(f"native.{name} n=2^{n_log}: {t:.3f} s  ({12 * n / t / 1e9:.3f} GB/s at 12 B/elem)")


def pad_bwd_section(native, OFF):
    """native.pad with approx_bwd=True through torch autograd (pam/native.py:173-196): the CPU flavour of the
    quotient's gradients, which differs from the GPU flavour of pam/cuda_bindings.py:78-97."""
    g = torch.Generator().manual_seed(4)
    n = 4096
    A = torch.randn(n, generator=g); B = torch.randn(n, generator=g); D = torch.randn(n, generator=g)
    A[n // 2:] *= 2.0 ** torch.randint(-20, 20, (n // 2,), generator=g).float()
    B[n // 2:] *= 2.0 ** torch.randint(-20, 20, (n // 2,), generator=g).float()
    d = {"a": u32(A), "b": u32(B), "d": u32(D), "offset": np.float32(OFF)}
    for tag, off in (("", None), ("_off", OFF)):
        a = A.clone().requires_grad_(); b = B.clone().requires_grad_()
        c = native.pad(a, b, offset=off, approx_bwd=True)
        c.backward(D)
        d["c" + tag] = u32(c); d["da" + tag] = u32(a.grad); d["db" + tag] = u32(b.grad)
    np.savez_compressed(OUT / "pad_native_bwd.npz", **d)


if __name__ == "__main__":
    main()
