"""Helpers shared by the tests: bit-level comparison and seeded operand generators."""
import pathlib

import numpy as np

GOLDEN = pathlib.Path(__file__).resolve().parent / "golden"


def f32(u):
    return np.asarray(u, dtype=np.uint32).view(np.float32)


def bits(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32)).view(np.uint32)


def same_bits(x, y):
    """Elementwise: identical bit pattern, or both NaN (NaN is compared as a class)."""
    x = np.asarray(x, dtype=np.float32); y = np.asarray(y, dtype=np.float32)
    return (bits(x) == bits(y)) | (np.isnan(x) & np.isnan(y))


def assert_same_bits(got, want, what=""):
    ok = same_bits(got, want)
    if not ok.all():
        i = np.flatnonzero(~ok.ravel())[:5]
        g = np.asarray(got, dtype=np.float32).ravel(); w = np.asarray(want, dtype=np.float32).ravel()
        lines = [f"  [{k}] got {g[k]!r} ({bits(g[k:k+1])[0]:08x})  want {w[k]!r} ({bits(w[k:k+1])[0]:08x})" for k in i]
        raise AssertionError(f"{what}: {(~ok).sum()} of {ok.size} elements differ\n" + "\n".join(lines))


def below_pow2(x):
    """True where x is the fp32 value just below a power of two (all mantissa bits set):
    the band where torch's floor(log2(x)) reports the exponent one too high."""
    u = bits(x)
    return ((u & 0x007FFFFF) == 0x007FFFFF) & ((u & 0x7F800000) != 0x7F800000)


def fclass(v):
    v = np.asarray(v, dtype=np.float32)
    return np.where(np.isnan(v), 3, np.where(np.isinf(v), 2, np.where(v == 0, 0, 1)))


EDGE_BITS = np.array(
    [0x00000000, 0x00000001, 0x00000003, 0x00400000, 0x00555555, 0x007fffff, 0x00800000, 0x00800001,
     0x7f7fffff, 0x7f000000, 0x7effffff, 0x7e900000, 0x7f800000, 0x7fc00000, 0x3f800000, 0x3fc00000,
     0x1f800000, 0x5f800000, 0x00ffffff, 0x3f7fffff], dtype=np.uint32)


def edge_values():
    return f32(np.concatenate([EDGE_BITS, EDGE_BITS | np.uint32(0x80000000)]))


def mixed_operands(n, seed, edge_frac=0.02):
    """98 % N(0,1), 2 % edge values (zeros, subnormals, inf, NaN, near FLT_MAX) at seeded places."""
    rng = np.random.RandomState(seed)
    x = rng.standard_normal(n).astype(np.float32)
    k = int(n * edge_frac)
    idx = rng.choice(n, size=k, replace=False)
    kind = rng.randint(0, 6, size=k)
    sign = rng.randint(0, 2, size=k).astype(np.uint32) << np.uint32(31)
    sub = rng.randint(1, 1 << 23, size=k).astype(np.uint32)
    big = (np.uint32(0x7f7fffff) - rng.randint(0, 3 << 23, size=k).astype(np.uint32))
    u = np.select([kind == 0, kind == 1, kind == 2, kind == 3, kind == 4, kind == 5],
                  [np.uint32(0), sub, np.uint32(0x7f800000), np.uint32(0x7fc00000), big, sub >> np.uint32(9)])
    x[idx] = f32((u.astype(np.uint32) | sign).astype(np.uint32))
    return x


def ulp_histogram(got, want):
    """{distance in units of the last place: count} between two fp32 arrays of finite values, as a JSON-ready dict."""
    g = np.ascontiguousarray(np.asarray(got, dtype=np.float32)).view(np.int32).astype(np.int64)
    w = np.ascontiguousarray(np.asarray(want, dtype=np.float32)).view(np.int32).astype(np.int64)
    dist, count = np.unique(np.abs(g - w), return_counts=True)
    return {str(int(d)): int(c) for d, c in zip(dist, count)}


def full_mantissa_histograms(fns):
    """The histograms kept in tests/golden/ulp_histogram.json: for each of pam, pad with and without the offset, the
    distance between `fns[op](a, b, offset)` and what pam/native.py gave on the same operands (normal_fullmant.npz),
    separately for its N(0,1) half and its wide-exponent half (|e| up to 40)."""
    g = np.load(GOLDEN / "normal_fullmant.npz")
    a, b = f32(g["a"]), f32(g["b"]); off = float(g["offset"]); n = a.size
    out = {}
    for name in ("pam", "pad", "pam_off", "pad_off"):
        got = fns[name.split("_")[0]](a, b, off if name.endswith("_off") else None)
        want = f32(g[name])
        out[name] = {"unit_normal": ulp_histogram(got[:n // 2], want[:n // 2]),
                     "wide_exponent": ulp_histogram(got[n // 2:], want[n // 2:])}
    return out
