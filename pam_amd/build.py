"""Compiles the HIP sources of this package into pam_amd/lib/libpam_hip.so for gfx950.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
Packed-fp32 instruction selection is switched off and floating-point contraction is off:
the kernels' results are defined operation by operation.
"""
import pathlib
import subprocess
import sys

HERE = pathlib.Path(__file__).resolve().parent
SOURCES = [HERE / "csrc" / "pam_elementwise.hip", HERE / "csrc" / "pam_gemm.hip", HERE / "csrc" / "pam_rowops.hip"]
LIB = HERE / "lib" / "libpam_hip.so"

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose=False):
    LIB.parent.mkdir(exist_ok=True)
    cmd = ["hipcc", *FLAGS, *map(str, SOURCES), "-o", str(LIB)]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
