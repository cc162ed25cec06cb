"""Writes tests/golden/ulp_histogram.json: how far the integer definition of the PAM product and quotient (this
repository's oracle, `exact` flavour, which the GPU kernels equal bit for bit) lies from the reference's float
emulation pam/native.py on full-mantissa operands, as counts per distance in units of the last place.  It reads
the golden vectors of normal_fullmant.npz and the oracle only; the reference itself is not needed.

    python tests/golden/make_ulp_histogram.py
"""
import json
import pathlib
import sys

ROOT = pathlib.Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from _util import full_mantissa_histograms  # noqa: E402
from oracle import pam_oracle  # noqa: E402

if __name__ == "__main__":
    pam_oracle.build()
    o = pam_oracle
    hist = full_mantissa_histograms({"pam": o.pam, "pad": o.pad})
    (pathlib.Path(__file__).resolve().parent / "ulp_histogram.json").write_text(json.dumps(hist, indent=1, sort_keys=True) + "\n")
    for name, h in hist.items():
        for half, counts in h.items():
            total = sum(counts.values())
            print(f"{name:8s} {half:14s} identical {counts.get('0', 0) / total:.3f}  max {max(map(int, counts))} ulp")
