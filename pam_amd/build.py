"""Compiles the HIP sources of this package into pam_amd/lib/libpam_hip.so for gfx950.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
Packed-fp32 instruction selection is switched off and floating-point contraction is off:
the kernels' results are defined operation by operation.
"""
import concurrent.futures
import hashlib
import pathlib
import re
import shutil
import subprocess
import sys
import tempfile

HERE = pathlib.Path(__file__).resolve().parent
CSRC = HERE / "csrc"
SOURCES = [CSRC / "pam_rowops_plain.hip", CSRC / "pam_rowops_offset.hip"] + sorted(CSRC.glob("pam_gemm_inst_*.hip")) + [
    CSRC / "pam_gemm.hip", CSRC / "pam_elementwise.hip", CSRC / "pam_rowops.hip", CSRC / "pam_probe.hip"]   # slowest first
JOBS = 8
STAMP_SOURCE = CSRC / "pam_stamp.cpp"
LIB = HERE / "lib" / "libpam_hip.so"

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
_NOISE = "is not a recognized feature for this target"      # the host pass does not know the device feature
_TAG = b"pam_hip_source_hash="


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if _NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)


def _with_includes(src, seen=None):
    """src and the project headers it includes ("..." includes, followed recursively), in a fixed order."""
    seen = [] if seen is None else seen
    src = src.resolve()
    if src in seen or not src.is_file():
        return seen
    seen.append(src)
    for name in re.findall(r'^\s*#\s*include\s+"([^"]+)"', src.read_text(), flags=re.M):
        _with_includes(src.parent / name, seen)
    return seen


def source_files():
    """What the library is built from: the HIP / C++ sources and headers under csrc/ and the public headers.
    Anything else lying in those folders (editor backups, objects, folders) is not part of it."""
    files = [f for pat in ("*.hip", "*.cpp", "*.h") for f in CSRC.glob(pat)] + list((HERE.parent / "include").glob("*.h"))
    return sorted(f for f in files if f.is_file())


def source_hash():
    """Hash of everything the library is built from (source_files() and the compiler flags).  It is compiled
    into the library (pam_hip_source_hash), so a library can be told from one built from other sources."""
    h = hashlib.sha256(" ".join(FLAGS).encode())
    for f in source_files():
        h.update(f.name.encode() + b"\0" + f.read_bytes())
    return h.hexdigest()[:16]


def built_hash():
    """The hash the built library carries, or None if there is no library (or one without a stamp).  Read from the
    file's bytes: loading a possibly stale library into this process, which may go on to load its replacement,
    would register two copies of the code objects."""
    if not LIB.exists():
        return None
    m = re.search(re.escape(_TAG) + rb"([0-9a-f]{16})\0", LIB.read_bytes())
    return m.group(1).decode() if m else None


def ensure_built(verbose=False):
    """What tests, the smoke check and the benchmark call: the library that is built is used as it is when it was
    built from this tree's sources; a missing or stale one is rebuilt where hipcc is at hand, and is an error where
    it is not.  Returns (path, hash)."""
    want = source_hash()
    have = built_hash()
    if have != want:
        if shutil.which("hipcc") is None:
            raise RuntimeError(f"{LIB} is missing or was built from other sources (want {want}, have {have}) and there is no hipcc to rebuild it")
        build(verbose)
        if built_hash() != want:
            raise RuntimeError("the library just built does not carry the hash of the sources")
    return LIB, want


def build(verbose=False, object_dir=None):
    """Compiles the sources side by side (the matrix kernel's many instances dominate), then links.
    object_dir: keep the objects there and recompile only the sources that changed since (for development;
    the default compiles everything)."""
    LIB.parent.mkdir(exist_ok=True)
    stamp = f'-DPAM_HIP_SOURCE_HASH="{source_hash()}"'
    with tempfile.TemporaryDirectory() as tmp:
        out = pathlib.Path(object_dir) if object_dir else pathlib.Path(tmp)
        out.mkdir(parents=True, exist_ok=True)
        jobs, objects = [], []
        with concurrent.futures.ThreadPoolExecutor(JOBS) as pool:
            for src in SOURCES + [STAMP_SOURCE]:
                obj = out / (src.stem + ".o")
                objects.append(str(obj))
                flags = FLAGS + ([stamp] if src == STAMP_SOURCE else [])
                key = hashlib.sha256(" ".join(flags).encode() + b"".join(f.read_bytes() for f in _with_includes(src))).hexdigest()
                keyfile = out / (src.stem + ".key")
                if object_dir and obj.exists() and keyfile.exists() and keyfile.read_text() == key:
                    continue
                keyfile.unlink(missing_ok=True)
                jobs.append((pool.submit(_run, ["hipcc", *flags, "-c", str(src), "-o", str(obj)], verbose), keyfile, key))
            for job, keyfile, key in jobs:
                job.result()
                if object_dir:
                    keyfile.write_text(key)
        _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", str(LIB)], verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, object_dir=sys.argv[1] if len(sys.argv) > 1 else None))
