"""Compiles the HIP sources of this package into pam_amd/lib/libpam_hip.so for gfx950.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
Packed-fp32 instruction selection is switched off and floating-point contraction is off:
the kernels' results are defined operation by operation.
"""
import concurrent.futures
import pathlib
import subprocess
import sys
import tempfile

HERE = pathlib.Path(__file__).resolve().parent
SOURCES = [HERE / "csrc" / "pam_elementwise.hip", HERE / "csrc" / "pam_gemm.hip", HERE / "csrc" / "pam_rowops.hip"]
LIB = HERE / "lib" / "libpam_hip.so"

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
_NOISE = "is not a recognized feature for this target"      # the host pass does not know the device feature


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if _NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose=False):
    """Compiles the sources side by side (the matrix kernel's many instances dominate), then links."""
    LIB.parent.mkdir(exist_ok=True)
    with tempfile.TemporaryDirectory() as tmp:
        objects = [str(pathlib.Path(tmp) / (src.stem + ".o")) for src in SOURCES]
        with concurrent.futures.ThreadPoolExecutor(len(SOURCES)) as pool:
            jobs = [pool.submit(_run, ["hipcc", *FLAGS, "-c", str(src), "-o", obj], verbose) for src, obj in zip(SOURCES, objects)]
            for job in jobs:
                job.result()
        _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", str(LIB)], verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
