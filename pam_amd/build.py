"""Compiles the HIP sources of this package into pam_amd/lib/libpam_hip.so for gfx950.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
Packed-fp32 instruction selection is switched off and floating-point contraction is off:
the kernels' results are defined operation by operation.
"""
import concurrent.futures
import hashlib
import pathlib
import shutil
import subprocess
import sys
import tempfile

HERE = pathlib.Path(__file__).resolve().parent
SOURCES = [HERE / "csrc" / "pam_elementwise.hip", HERE / "csrc" / "pam_gemm.hip", HERE / "csrc" / "pam_rowops.hip", HERE / "csrc" / "pam_probe.hip"]
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


def source_hash():
    """Hash of everything the library is built from: the sources and headers under csrc/, the public headers and
    the compiler flags.  It is compiled into the library (pam_hip_source_hash), so a library can be told from one
    built from other sources."""
    h = hashlib.sha256(" ".join(FLAGS).encode())
    files = sorted((HERE / "csrc").glob("*")) + sorted((HERE.parent / "include").glob("*.h"))
    for f in files:
        h.update(f.name.encode() + b"\0" + f.read_bytes())
    return h.hexdigest()[:16]


def built_hash():
    """The hash the built library carries, or None if there is no library (or one from before the hash)."""
    if not LIB.exists():
        return None
    import ctypes
    try:
        fn = ctypes.CDLL(str(LIB)).pam_hip_source_hash
    except (OSError, AttributeError):
        return None
    fn.restype = ctypes.c_char_p
    return fn().decode()


def ensure_built(verbose=False):
    """What tests, the smoke check and the benchmark call: the library that is built is used as it is when it was
    built from this tree's sources; a missing or stale one is rebuilt where hipcc is at hand, and is an error where
    it is not.  Returns (path, hash)."""
    want = source_hash()
    if built_hash() != want:
        if shutil.which("hipcc") is None:
            raise RuntimeError(f"{LIB} is missing or was built from other sources (want {want}, have {built_hash()}) and there is no hipcc to rebuild it")
        build(verbose)
        if built_hash() != want:
            raise RuntimeError("the library just built does not carry the hash of the sources")
    return LIB, want


def build(verbose=False):
    """Compiles the sources side by side (the matrix kernel's many instances dominate), then links."""
    LIB.parent.mkdir(exist_ok=True)
    stamp = f'-DPAM_HIP_SOURCE_HASH="{source_hash()}"'
    with tempfile.TemporaryDirectory() as tmp:
        objects = [str(pathlib.Path(tmp) / (src.stem + ".o")) for src in SOURCES]
        with concurrent.futures.ThreadPoolExecutor(len(SOURCES)) as pool:
            jobs = [pool.submit(_run, ["hipcc", *FLAGS, stamp, "-c", str(src), "-o", obj], verbose) for src, obj in zip(SOURCES, objects)]
            for job in jobs:
                job.result()
        _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", str(LIB)], verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
