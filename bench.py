"""Benchmark of the PAM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = the six PAM matrix products of a DeiT-tiny MLP block on 64 x 197 tokens
(fp32, synthetic data): for each of the layers 192->768 and 768->192 the forward product,
dX and dW (the approximate backward of the reference's training recipe,
pam/cuda_bindings.py:154-161).  `value` is G PAM-MAC/s over whole steps with all operands
resident in HBM.  Each product is also timed on its own with HIP events, which gives the
roofline figure of the matrix kernel (VALU issue rate: 2 lane-ops per MAC against
CUs x 128 lanes x clock), and the elementwise multiply / divide are timed on 2^26
elements against HBM bandwidth.  The CPU baseline is this repository's own C restatement
of the same arithmetic (oracle/, OpenMP) on the host cores, on the 192->768 layer.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--settle-ms", type=float, default=30.0,
                    help="each timed row first runs its launches for this long (0 for counter-collecting profiler passes)")
    ap.add_argument("--no-elementwise", action="store_true")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one device-to-device copy of 2^26 floats (calibrates FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--write-traffic", metavar="DIR",
                    help="no GPU work: read the FETCH_SIZE and WRITE_SIZE counter passes of this program under DIR "
                         "(DIR/pmc_<COUNTER>/p_counter_collection.csv, DIR/pmc_<COUNTER>.json = that pass's bench line) "
                         "and rewrite profiles/traffic.json, stamped with the source hash of the library they measured")
    return ap.parse_args()


SETTLE_S = 0.03
HERE = os.path.dirname(os.path.abspath(__file__))
TRAFFIC_FILE = os.path.join(HERE, "profiles", "traffic.json")
HEADLINE_KERNEL = "gemm_kernel<64, 64, 4, 4, 32, 0, 0, 0, false>"      # whole tiles, both operands contiguous along k
ELEMENTWISE_KERNEL = "ew_vec_kernel<OpPam, 2>"


def write_traffic(prof_dir):
    """HBM bytes per launch of the headline product (12608x768, k = 192) and of the elementwise multiply on 2^26 elements
    from two counter passes over `bench.py --steps 5 --warmup 2 --no-cpu-baseline --copy-probe --settle-ms 0`.  The
    counters' unit is calibrated on the elementwise multiply, which reads exactly 2 x 256 MiB and writes 256 MiB."""
    import csv
    import re
    per_counter, stamps = {}, set()
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        with open(os.path.join(prof_dir, f"pmc_{counter}.json")) as f:
            stamps.add(json.loads(f.read().strip().splitlines()[-1])["library_source_hash"])
        dispatches = {}
        with open(os.path.join(prof_dir, f"pmc_{counter}", "p_counter_collection.csv")) as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] != counter:
                    continue
                name = re.sub(r"\(anonymous namespace\)::|pamgemm::|^void ", "", r["Kernel_Name"])
                name = re.sub(r"\(.*", "", name)
                dispatches[int(r["Dispatch_Id"])] = (name, int(r["Grid_Size"]), float(r["Counter_Value"]))
        ids = sorted(dispatches)
        first_ew = min(i for i in ids if dispatches[i][0] == ELEMENTWISE_KERNEL)
        # the headline product's launches are those of its kernel instance before the first elementwise launch with the
        # launch size that occurs most often there (the six-product step and the per-product rows)
        head = [dispatches[i] for i in ids if i < first_ew and dispatches[i][0] == HEADLINE_KERNEL]
        grids = [g for _, g, _ in head]
        grid = max(set(grids), key=grids.count)
        ew = [v for n, g, v in dispatches.values() if n == ELEMENTWISE_KERNEL]
        per_counter[counter] = (sum(v for _, g, v in head if g == grid) / grids.count(grid), sum(ew) / len(ew))
    if len(stamps) != 1:
        sys.exit(f"bench.py: the two counter passes ran different libraries: {sorted(stamps)}")
    n = 1 << 26
    known = {"FETCH_SIZE": 8 * n, "WRITE_SIZE": 4 * n}
    head_bytes = sum(per_counter[c][0] * known[c] / per_counter[c][1] for c in known)
    out = {"library_source_hash": stamps.pop(), "gemm_fwd_12608x768x192_bytes": round(head_bytes), "ew_mul_2p26_bytes": 12 * n,
           "counter_units": {c: round(known[c] / per_counter[c][1], 2) for c in known},
           "source": "FETCH_SIZE and WRITE_SIZE per dispatch (rocprofv3 --pmc over bench.py), in units of what the same counter "
                     "reads for the elementwise multiply on 2^26 elements (8 and 4 bytes per element); "
                     "written by bench.py --write-traffic"}
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(json.dumps(out))


def event_time_ms(fn, iters, torch, settle_s=None):
    """Average duration of fn() over `iters` back-to-back launches, HIP events on the launch stream.  The same launches
    run for `settle_s` first: the operands of a row are made on the host while the GPU idles, and the first
    milliseconds after an idle period run at lower clocks (a 130 us product measured 146 us with seven warm-up launches
    and 122 us after 30 ms of them)."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn(); torch.cuda.synchronize()
    t_end = time.perf_counter() + (SETTLE_S if settle_s is None else settle_s)
    while time.perf_counter() < t_end:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    for _ in range(max(3, iters // 4)):        # untimed launches ahead of the start event: the queue is full when timing begins
        fn()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def config1_operand(n, seed, torch, dev):
    """An operand of benchmark configuration 1: 98 % N(0,1); 2 % edge values at seeded random places, drawn uniformly
    from +0, -0, subnormals of either sign with a random 23-bit mantissa, +-inf, NaN, and +-[FLT_MAX / 8, FLT_MAX]."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(n, generator=g)
    k = n // 50
    idx = torch.randperm(n, generator=g)[:k]
    kind = torch.randint(0, 6, (k,), generator=g)
    sign = torch.randint(0, 2, (k,), generator=g).to(torch.int64) << 31
    mant = torch.randint(1, 1 << 23, (k,), generator=g).to(torch.int64)
    big = 0x7f7fffff - torch.randint(0, 3 << 23, (k,), generator=g).to(torch.int64)
    bits = torch.zeros(k, dtype=torch.int64)                                     # kind 0: +0, kind 1: -0 (sign forced below)
    bits = torch.where(kind == 2, mant, bits)                                    # subnormal
    bits = torch.where(kind == 3, torch.full_like(bits, 0x7f800000), bits)       # inf
    bits = torch.where(kind == 4, torch.full_like(bits, 0x7fc00000), bits)       # NaN
    bits = torch.where(kind == 5, big, bits)                                     # near FLT_MAX
    sign = torch.where(kind == 0, torch.zeros_like(sign), torch.where(kind == 1, torch.full_like(sign, 1 << 31), sign))
    u = (bits | sign)
    u = torch.where(u >= (1 << 31), u - (1 << 32), u).to(torch.int32)
    x[idx] = u.view(torch.float32)
    return x.to(dev)


def main():
    global SETTLE_S
    args = parse()
    SETTLE_S = args.settle_ms / 1e3
    if args.write_traffic:
        return write_traffic(args.write_traffic)
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only; --gpus must be 1 "
                 "(the path has no collective: it shards by rows, with one all-reduce of dW per layer)")
    import torch
    from pam_amd import _abi
    from pam_amd._abi import HipKernels
    from pam_amd import build as hip_build
    # the built library travels with the tree; it is rebuilt only if it is missing or was built from other sources
    _, source_stamp = hip_build.ensure_built()
    _abi.load_library()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    K = HipKernels()
    dev = torch.device("cuda:0")
    cus, khz = _abi.device_info()
    # VALU issue peak.  Measured on MI355X, a SIMD retires a wave64 32-bit VALU instruction every
    # two cycles (128 lanes per CU per clock): 256 CUs x 128 x 2.4 GHz = 78.6 T lane-ops/s, which
    # is the published 157.3 TFLOP/s fp32 vector peak counted as FMAs.  `single_issue` is the
    # 64-lanes-per-clock figure the baseline plan assumed.
    lane_peak = cus * 128 * khz * 1e3
    single_issue_peak = cus * 64 * khz * 1e3

    g = torch.Generator(device="cpu").manual_seed(0)
    T, D1, D2 = 64 * 197, 192, 768
    X1 = torch.randn(T, D1, generator=g).to(dev)
    X2 = torch.randn(T, D2, generator=g).to(dev)
    W1 = torch.nn.init.trunc_normal_(torch.empty(D2, D1), std=0.02, a=-0.04, b=0.04, generator=g).to(dev)
    W2 = torch.nn.init.trunc_normal_(torch.empty(D1, D2), std=0.02, a=-0.04, b=0.04, generator=g).to(dev)
    dY1 = (torch.randn(T, D2, generator=g) * 1e-2).to(dev)
    dY2 = (torch.randn(T, D1, generator=g) * 1e-2).to(dev)

    products = {
        "fwd_12608x768x192": lambda: K.pam_matmul_fwd(X1, W1.T, True, False, 1.0),
        "dX_12608x192x768": lambda: K.pam_matmul_fwd(dY1, W1, True, True, 1.0),
        "dW_192x768x12608": lambda: K.pam_matmul_fwd(X1.T, dY1, False, True, 1.0),
        "fwd_12608x192x768": lambda: K.pam_matmul_fwd(X2, W2.T, True, False, 1.0),
        "dX_12608x768x192": lambda: K.pam_matmul_fwd(dY2, W2, True, True, 1.0),
        "dW_768x192x12608": lambda: K.pam_matmul_fwd(X2.T, dY2, False, True, 1.0),
    }
    macs_each = T * D1 * D2

    def step():
        for fn in products.values():
            fn()

    # Clocks and the launch queue need some tens of milliseconds of work to settle; the same products run for a
    # moment before the W warm-up steps so that a short timed run (small K) measures the settled rate too.
    ramp_end = time.perf_counter() + 0.25
    while time.perf_counter() < ramp_end:
        step()
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    gmacs = len(products) * macs_each / (dt / args.steps) / 1e9

    per = {}
    for name, fn in products.items():
        ms = event_time_ms(fn, min(max(10, args.steps), 200), torch)
        per[name] = {"ms": round(ms, 4), "gmacs": round(macs_each / ms / 1e6, 1),
                     "valu_frac": round(2 * macs_each / (ms * 1e-3) / lane_peak, 4)}
    head = per["fwd_12608x768x192"]
    roofline = {
        "kernel": "gemm_kernel (PAM forward, 12608x768x192)", "bound": "valu",
        "achieved": round(2 * macs_each / (head["ms"] * 1e-3) / 1e12, 3),
        "peak": round(lane_peak / 1e12, 3), "unit": "Tlaneop/s",
        "frac": head["valu_frac"], "traffic": None,
        "note": "2 VALU lane-ops (v_add_u32 + v_add_f32) per PAM-MAC; peak = CUs x 128 lanes x clock "
                "(= published 157.3 TFLOP/s fp32 vector / 2); MFMA does not apply to an integer-add product",
        "compute_units": cus, "clock_mhz": khz / 1e3,
        "worst_of_six_frac": min(p["valu_frac"] for p in per.values()),
        "frac_of_single_issue_peak": round(2 * macs_each / (head["ms"] * 1e-3) / single_issue_peak, 4),
        "target_in_baseline_plan": ">= 0.60 of the single-issue figure (11.8 T PAM-MAC/s)",
    }
    # the issue rate of the same instruction mix with register operands only, at 1, 2 and 4 wavefronts per SIMD
    roofline["register_only_probe_Tlaneop_s"] = {str(w): round(_abi.issue_probe(w), 2) for w in (1, 2, 4, 8)}
    # and with every step's operands read from LDS the way the kernel's inner loop reads them (4 x 4 per lane)
    roofline["lds_fed_4x4_probe_Tlaneop_s"] = {str(w): round(_abi.issue_probe(w, lds_tile=(4, 4)), 2) for w in (1, 2, 4, 8)}
    # counter-measured HBM bytes per launch, valid only for the library they were measured with
    traffic = json.load(open(TRAFFIC_FILE)) if os.path.exists(TRAFFIC_FILE) else {}
    if traffic.get("library_source_hash") != source_stamp:
        traffic = {}
    roofline["traffic"] = traffic.get("gemm_fwd_12608x768x192_bytes")

    # the headline metric as BASELINE.json words it (value = its G-MAC/s part, at the 12608x192x768 configuration;
    # the %VALU-peak part is roofline.frac, the elementwise GB/s part roofline_elementwise.achieved)
    metric_name = "PAM-GEMM G-MAC/s + %VALU peak at 12608x192x768 fp32; PAM elementwise GB/s"
    baseline_file = os.path.join(HERE, "BASELINE.json")
    if os.path.exists(baseline_file):
        metric_name = json.load(open(baseline_file)).get("metric") or metric_name
    out = {
        "metric": metric_name, "value": round(gmacs, 1), "unit": "GMAC/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "DeiT-tiny PAM linear fwd+dX+dW, tokens 64x197=12608, 192->768 and 768->192 "
                               "(benchmark configuration 2); 6 products of 1 859 125 248 PAM-MAC per step"},
        "roofline": roofline, "products": per, "library_source_hash": source_stamp,
    }

    if not args.no_elementwise:
        n = 1 << 26
        a = config1_operand(n, 10, torch, dev); b = config1_operand(n, 11, torch, dev)
        ew = {}
        for name, fn in (("mul", lambda: K.pam_fwd(a, b, 1.0)), ("div", lambda: K.pad_fwd(a, b, 1.0))):
            ms = event_time_ms(fn, 20, torch)
            ew[name] = {"ms": round(ms, 4), "GBps": round(12 * n / ms / 1e6, 1)}
        out["roofline_elementwise"] = {
            "kernel": "ew_vec_kernel (PAM multiply, 2^26 elements, benchmark configuration 1)", "bound": "hbm",
            "achieved": ew["mul"]["GBps"], "peak": 8000.0, "unit": "GB/s", "frac": round(ew["mul"]["GBps"] / 8000.0, 4),
            "traffic": traffic.get("ew_mul_2p26_bytes"), "bytes_per_element": 12, "div_GBps": ew["div"]["GBps"],
        }
        if args.copy_probe:
            c = torch.empty_like(a)
            c.copy_(b); torch.cuda.synchronize()
            del c
        # the other kernels of the path, each against its own bound (not part of `value`)
        d = torch.randn(n, generator=g).to(dev)
        other = {}
        stream_ops = (
            ("pam_bwd", 16, lambda: K.pam_bwd(a, b, d, 1.0)), ("pad_bwd", 16, lambda: K.pad_bwd(a, b, d, 1.0)),
            ("pam_fwd_offset", 12, lambda: K.pam_fwd(a, b, 1.0552)),
            ("pam_fwd_scalar_operand", 8, lambda: K.pam_fwd(a, d[:1].expand(n), 1.0)),
            ("pa_exp_fwd", 8, lambda: K.pa_exp_fwd(d, math.e, 1.0)), ("pa_log_fwd", 8, lambda: K.pa_log_fwd(a, math.e, 1.0)),
            ("pa_exp_bwd", 12, lambda: K.pa_exp_bwd(d, b, math.e, 1.0)), ("pa_log_bwd", 12, lambda: K.pa_log_bwd(a, b, math.e, 1.0)),
        )
        from pam_amd import _abi as abi_ew
        a_pos = torch.randn(n, generator=g).to(dev).abs_().add_(1e-3)     # a square root's operand: positive normal numbers
        stream_ops += (("pow_0.5_fwd_positive_operand", 8, lambda: abi_ew.pow_fwd(a_pos, 0.5, 1.0)),
                       ("pow_0.5_bwd_approx_positive_operand", 12, lambda: abi_ew.pow_bwd(a_pos, d, 0.5, 1.0, True, True)))
        stream_ops += (("pam_bwd_pair_approx", 20, lambda: K.pam_bwd_pair(a, b, d, 1.0, True, True)),
                       ("pam_bwd_pair_exact", 20, lambda: K.pam_bwd_pair(a, b, d, 1.0, False, False)),
                       ("pad_bwd_pair_approx", 20, lambda: K.pad_bwd_pair(a, b, d, 1.0, True, True)))
        for name, bpe, fn in stream_ops:
            ms = event_time_ms(fn, 30, torch)
            other[name] = {"ms": round(ms, 4), "GBps": round(bpe * n / ms / 1e6, 1), "hbm_frac": round(bpe * n / ms / 1e6 / 8000.0, 3)}
        del a, b, d, a_pos
        # exact backward products (3 lane-ops per MAC) and the attention products of configuration 3
        Xd = X1.contiguous()
        exact = {
            "exact_dX_12608x192x768": (3, macs_each, lambda: K.pam_matmul_bwd(dY1, W1, Xd, True, True, True, 1.0)),
            "exact_dW_192x768x12608": (3, macs_each, lambda: K.pam_matmul_bwd(X1.T, dY1, W1.T, False, True, False, 1.0)),
        }
        Bh, Tk, Dh = 192, 197, 64
        q, kk, v = (torch.randn(Bh, Tk, Dh, generator=g).to(dev) for _ in range(3))
        pr = torch.softmax(torch.randn(Bh, Tk, Tk, generator=g), -1).to(dev)
        exact["bmm_QKt_192x197x197x64"] = (2, Bh * Tk * Tk * Dh, lambda: K.pam_bmm_fwd(q, kk.transpose(1, 2), True, False, 1.0))
        exact["bmm_PV_192x197x64x197"] = (2, Bh * Tk * Tk * Dh, lambda: K.pam_bmm_fwd(pr, v, True, True, 1.0))
        # operands with zeros: ReLU output as the left operand (the second layer of a ReLU feed-forward block)
        X2r = torch.relu(X2)
        exact["fwd_12608x192x768_relu_input"] = (2, macs_each, lambda: K.pam_matmul_fwd(X2r, W2.T, True, False, 1.0))
        exact["dW_768x192x12608_relu_input"] = (2, macs_each, lambda: K.pam_matmul_fwd(X2r.T, dY2, False, True, 1.0))
        # zeros in both operands: the same input against a weight matrix with 30 % of its entries pruned
        W2s = W2 * (torch.rand(W2.shape, generator=g) >= 0.3).to(dev)
        exact["fwd_12608x192x768_relu_input_pruned_weight"] = (2, macs_each, lambda: K.pam_matmul_fwd(X2r, W2s.T, True, False, 1.0))
        # one value in a thousand of the left operand a subnormal number: its k-step takes the full definition, the rest of its k-tile not
        X2n = torch.where((torch.rand(X2.shape, generator=g) < 1e-3).to(dev), torch.full_like(X2, 1e-40), X2)
        exact["fwd_12608x192x768_0.1pct_subnormal_input"] = (2, macs_each, lambda: K.pam_matmul_fwd(X2n, W2.T, True, False, 1.0))
        # the other linear layers of the same model (qkv 192->576, proj 192->192) and the MLP block at the DeiT-small
        # and DeiT-base widths, same 12608 tokens: forward, dX, dW
        for d_in, d_out in ((192, 576), (192, 192), (384, 1536), (768, 3072)):
            Xw = torch.randn(T, d_in, generator=g).to(dev)
            Ww = torch.nn.init.trunc_normal_(torch.empty(d_out, d_in), std=0.02, a=-0.04, b=0.04, generator=g).to(dev)
            dYw = (torch.randn(T, d_out, generator=g) * 1e-2).to(dev)
            mm = T * d_in * d_out
            exact[f"fwd_12608x{d_out}x{d_in}"] = (2, mm, lambda Xw=Xw, Ww=Ww: K.pam_matmul_fwd(Xw, Ww.T, True, False, 1.0))
            exact[f"dX_12608x{d_in}x{d_out}"] = (2, mm, lambda dYw=dYw, Ww=Ww: K.pam_matmul_fwd(dYw, Ww, True, True, 1.0))
            exact[f"dW_{d_in}x{d_out}x12608"] = (2, mm, lambda Xw=Xw, dYw=dYw: K.pam_matmul_fwd(Xw.T, dYw, False, True, 1.0))
        for name, (ops, macs, fn) in exact.items():
            ms = event_time_ms(fn, 30, torch)
            other[name] = {"ms": round(ms, 4), "gmacs": round(macs / ms / 1e6, 1), "valu_frac": round(ops * macs / (ms * 1e-3) / lane_peak, 4)}
        # row-wise compositions as single kernels and the Adam step (HBM-bound; algorithmic bytes per element)
        from pam_amd import _abi as abi
        R = abi.HipRowKernels()
        rows_cases = {"attention_37824x197": (192 * 197, 197), "rows_65536x1024": (65536, 1024), "vocabulary_4096x10000": (4096, 10000),
                      "deit_tiny_tokens_50432x192": (256 * 197, 192)}     # the layer_norm shape of the headline model (256 images)
        for tag, (r, c) in rows_cases.items():
            xs = torch.randn(r, c, generator=g).to(dev); gs = torch.randn(r, c, generator=g).to(dev)
            wv = torch.randn(c, generator=g).to(dev); bv = torch.randn(c, generator=g).to(dev)
            ys, rs, sh = R.softmax_fwd(xs, 1.0)
            row_ops = (
                ("softmax_fwd", 12, lambda: R.softmax_fwd(xs, 1.0)),
                ("softmax_bwd_approx", 12, lambda: R.softmax_bwd(xs, gs, rs, sh, 1.0, True, True, True)),
                ("softmax_bwd_exact", 12, lambda: R.softmax_bwd(xs, gs, rs, sh, 1.0, False, False, False)),
                ("log_softmax_fwd", 12, lambda: R.logsumexp_fwd(xs, 1.0, False, True)),
                ("layer_norm_fwd", 8, lambda: R.layer_norm_fwd(xs, wv, bv, 1e-5, 1.0)),
                ("row_mean_fwd", 4, lambda: R.row_mean_fwd(xs, 1.0)),
            )
            row_ops += (("log_softmax_bwd_approx", 12, lambda: R.logsumexp_bwd(xs, gs, sh, 1.0, True, True, True, True)),)
            row_ops += (("layer_norm_bwd_approx", 16, lambda: R.layer_norm_bwd(xs, wv, gs, 1e-5, 1.0, True, True, True, True)),)
            row_ops += (("log_softmax_bwd_exact", 12, lambda: R.logsumexp_bwd(xs, gs, sh, 1.0, False, False, False, True)),)
            row_ops += (("layer_norm_bwd_exact", 16, lambda: R.layer_norm_bwd(xs, wv, gs, 1e-5, 1.0, False, False, False, True)),)
            for name, bpe, fn in row_ops:
                ms = event_time_ms(fn, 30, torch)
                other[f"{name}_{tag}"] = {"ms": round(ms, 4), "GBps": round(bpe * r * c / ms / 1e6, 1),
                                          "hbm_frac": round(bpe * r * c / ms / 1e6 / 8000.0, 3)}
            del xs, gs, ys
        # convolution with the image patches read in place (forward; PAM-MAC/s against the vector peak)
        for tag, (cb, cc, chh, co_, ck, cs, cp) in {"conv3x3_128x64x32x32_to128": (128, 64, 32, 128, 3, 1, 1),
                                                     "patch_embed_64x3x224x224_16x16_to192": (64, 3, 224, 192, 16, 16, 0)}.items():
            xc = torch.randn(cb, cc, chh, chh, generator=g).to(dev); wc = (torch.randn(co_, cc, ck, ck, generator=g) * 0.05).to(dev)
            ho = (chh + 2 * cp - ck) // cs + 1
            cm = cb * co_ * ho * ho * cc * ck * ck
            ms = event_time_ms(lambda: abi.conv2d_fwd(xc, wc, (cs, cs), (cp, cp), 1.0), 30, torch)
            other[tag] = {"ms": round(ms, 4), "gmacs": round(cm / ms / 1e6, 1), "valu_frac": round(2 * cm / (ms * 1e-3) / lane_peak, 4)}
            # the per-image weight gradients (the same patches, transposed), approximate and exact
            gy = (torch.randn(cb, co_, ho, ho, generator=g) * 1e-2).to(dev)
            for kind, exact_, ops in (("approx", False, 2), ("exact", True, 3)):
                ms = event_time_ms(lambda: abi.conv2d_bwd_weight(xc, gy, wc, (cs, cs), (cp, cp), exact_, 1.0), 30, torch)
                other[f"{tag}_weight_gradient_{kind}"] = {"ms": round(ms, 4), "gmacs": round(cm / ms / 1e6, 1),
                                                         "valu_frac": round(ops * cm / (ms * 1e-3) / lane_peak, 4)}
            if cs == 1:                 # the gradient of the input, also in place (a convolution of the upstream gradient)
                for kind, exact_, ops in (("approx", False, 2), ("exact", True, 3)):
                    ms = event_time_ms(lambda: abi.conv2d_bwd_input(gy, wc, xc, (cp, cp), exact_, 1.0), 30, torch)
                    other[f"{tag}_input_gradient_{kind}"] = {"ms": round(ms, 4), "gmacs": round(cm / ms / 1e6, 1),
                                                            "valu_frac": round(ops * cm / (ms * 1e-3) / lane_peak, 4)}
            del gy, xc, wc
        # grouped convolutions (one launch over (image, group) pairs) and a depthwise one (kernels of its own)
        for tag, (cb, cc, chh, gr) in {"conv3x3_32x128x28x28_to128_groups32": (32, 128, 28, 32),
                                       "conv3x3_32x192x28x28_depthwise": (32, 192, 28, 192)}.items():
            xc = torch.randn(cb, cc, chh, chh, generator=g).to(dev); wc = (torch.randn(cc, cc // gr, 3, 3, generator=g) * 0.05).to(dev)
            gy = (torch.randn(cb, cc, chh, chh, generator=g) * 1e-2).to(dev)
            cm = cb * cc * chh * chh * (cc // gr) * 9
            for name, fn in (("", lambda: abi.conv2d_fwd(xc, wc, (1, 1), (1, 1), 1.0, gr)),
                             ("_weight_gradient_approx", lambda: abi.conv2d_bwd_weight(xc, gy, wc, (1, 1), (1, 1), False, 1.0, gr)),
                             ("_input_gradient_approx", lambda: abi.conv2d_bwd_input(gy, wc, xc, (1, 1), False, 1.0, gr))):
                ms = event_time_ms(fn, 30, torch)
                other[tag + name] = {"ms": round(ms, 4), "gmacs": round(cm / ms / 1e6, 1), "valu_frac": round(2 * cm / (ms * 1e-3) / lane_peak, 4)}
                if gr == cc:            # nine products per output: bound by the two tensors' bytes, if by anything
                    other[tag + name]["hbm_frac"] = round(8 * xc.numel() / ms / 1e6 / 8000.0, 3)
            del gy, xc, wc
        na = 1 << 26
        pa, ga, ma, va = (torch.randn(na, generator=g).to(dev) * s_ for s_ in (1.0, 1e-2, 1e-2, 1e-4))
        va.abs_()
        ms = event_time_ms(lambda: abi.adam_step(pa, ga, ma, va, 0.9, 0.1, 0.98, 0.02, 1e-8, 5e-8, 4e-4, 1.0), 30, torch)
        other["adam_step_2p26"] = {"ms": round(ms, 4), "GBps": round(28 * na / ms / 1e6, 1), "hbm_frac": round(28 * na / ms / 1e6 / 8000.0, 3)}
        del pa, ga, ma, va
        out["other_kernels"] = other

    if not args.no_cpu_baseline:
        from oracle import pam_oracle as oracle
        oracle.build()
        cores = len(os.sched_getaffinity(0))
        os.environ.setdefault("OMP_NUM_THREADS", str(cores))
        Xh, Wh, dYh = X1.cpu().numpy(), W1.cpu().numpy(), dY1.cpu().numpy()
        WT = np.ascontiguousarray(Wh.T); XT = np.ascontiguousarray(Xh.T)
        oracle.gemm_fast(Xh, WT)                                   # first touch: library load, thread pool, page faults
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 10.0 and reps < 200):
            oracle.gemm_fast(Xh, WT); oracle.gemm_fast(dYh, Wh); oracle.gemm_fast(XT, dYh)
            reps += 1
        cdt = (time.perf_counter() - t0) / reps
        out["cpu_baseline"] = {
            "value": round(3 * macs_each / cdt / 1e9, 2), "unit": "GMAC/s", "cores": int(os.environ.get("OMP_NUM_THREADS", cores)),
            "kind": "port",
            "sample": f"fwd + dX + dW of the 192->768 layer (5.58 G PAM-MAC), {reps} times in about 10 s, this repository's C "
                      "restatement (integer add + fp32 accumulate, OpenMP over rows), contiguous operands",
        }
        # A second figure beside it: the reference's class of CPU algorithm (float log2 / add / exp2 on tensors, every
        # product of the matrix product materialised and then summed) on its own CPU-runnable case, 256 x 512 x 256
        # (benchmark configuration 0): forward and the two products of the approximate backward, median of 5.
        from oracle import float_chain
        gc = torch.Generator(device="cpu").manual_seed(0)
        A0, B0, dY0 = torch.randn(256, 512, generator=gc), torch.randn(512, 256, generator=gc), torch.randn(256, 256, generator=gc)
        float_chain.pam_matmul(A0, B0)
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            float_chain.pam_matmul(A0, B0); float_chain.pam_matmul(dY0, B0.T); float_chain.pam_matmul(A0.T, dY0)
            times.append(time.perf_counter() - t0)
        out["cpu_baseline"]["float_chain"] = {
            "value": round(3 * 256 * 512 * 256 / sorted(times)[2] / 1e9, 3), "unit": "GMAC/s", "cores": torch.get_num_threads(),
            "sample": "fwd + dX + dW at 256 x 512 x 256 (0.1 G PAM-MAC), median of 5, torch CPU float chain with the n x k x m "
                      "products materialised (oracle/float_chain.py)",
        }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
