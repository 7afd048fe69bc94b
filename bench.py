#!/usr/bin/env python3
"""Benchmark of the epsilon self-join hot path on one MI355X.

One "step" is one pass of the hot path over the resident dataset: squared-norm pre-pass,
queue/counter reset and the fused MFMA join kernel (the reference's TFLOPS window,
source/findPairs.cuh:625-697,729,745-747).  Inputs are generated on the device and are
resident in HBM before the timed region starts.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c3]

prints ONE JSON line: metric = self-join TFLOPS (2*N^2*D / time), plus `roofline`
(the join kernel against the dense FP16 MFMA peak) and `cpu_baseline` (a blocked FP64 / FP32 brute-force
join timed on this box's host cores: in full for the small workloads, else on 1024 seeded query rows
against all points).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2516.6  # MI355X dense FP16 MFMA: 256 CU x 4 SIMD x 1024 FLOP/clk x 2.4 GHz

CONFIGS = {
    # name: (N, D, generator, mean neighbours, label)
    "c1": (4096, 128, "exponential", 32, "plumbing 4096x128 Exp(40)"),
    "c2": (100_000, 128, "uniform_bytes", 64, "low-dim 100000x128 U{0..255}/255"),
    "c3": (1_000_000, 4096, "exponential", 16, "headline 1000000x4096 Exp(40)"),
    "c4": (500_000, 960, "gaussian_mixture", 100, "clustered 500000x960 GMM(1000, sigma=0.05)"),
    "c5": (2_000_000, 384, "unit_normal", 1000, "output-heavy 2000000x384 unit-normalised N(0,1)"),
}


def generate_points(torch, kind, n, d, seed):
    """FP16 dataset generated on the device in row chunks (seeded)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    out = torch.empty((n, d), dtype=torch.float16, device="cuda")
    rows = max(1, min(n, (1 << 28) // d))
    centers = None
    if kind == "gaussian_mixture":
        centers = torch.rand((1000, d), generator=g, device="cuda", dtype=torch.float32)
    for r0 in range(0, n, rows):
        r1 = min(n, r0 + rows)
        m = r1 - r0
        if kind == "exponential":
            x = torch.empty((m, d), device="cuda", dtype=torch.float32).exponential_(40.0, generator=g).clamp_(0.0, 1.0)
        elif kind == "uniform_bytes":
            x = torch.randint(0, 256, (m, d), generator=g, device="cuda").to(torch.float32) / 255.0
        elif kind == "gaussian_mixture":
            which = torch.randint(0, 1000, (m,), generator=g, device="cuda")
            x = centers[which] + 0.05 * torch.randn((m, d), generator=g, device="cuda", dtype=torch.float32)
        elif kind == "unit_normal":
            x = torch.randn((m, d), generator=g, device="cuda", dtype=torch.float32)
            x = x / x.norm(dim=1, keepdim=True)
        else:
            raise ValueError(kind)
        out[r0:r1] = x.to(torch.float16)
        del x
    return out


def calibrate_epsilon(torch, pts, neighbours, sample=4096, seed=4242):
    """epsilon from a seeded sample of query rows: the distance quantile that yields the wanted
    mean number of neighbours per point (self pairs excluded).  Harness code (torch FP32)."""
    n, d = pts.shape
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    m = min(sample, n)
    rows = torch.randperm(n, generator=g, device="cuda")[:m]
    q = pts[rows].to(torch.float32)
    qs = (q * q).sum(1)
    k = int(round(neighbours * m)) + m + 1  # + the m self pairs
    best = torch.full((0,), float("inf"), device="cuda")
    chunk = max(1, min(n, (1 << 27) // d, (1 << 30) // m))  # torch.topk sorts at most INT_MAX elements
    for c0 in range(0, n, chunk):
        c = pts[c0:c0 + chunk].to(torch.float32)
        d2 = qs[:, None] + (c * c).sum(1)[None, :] - 2.0 * (q @ c.T)
        flat = d2.reshape(-1)
        kk = min(k, flat.numel())
        best = torch.cat([best, torch.topk(flat, kk, largest=False).values])
        if best.numel() > k:
            best = torch.topk(best, k, largest=False).values
        del c, d2, flat
    best = torch.sort(best).values.clamp_min(0.0)
    want = int(round(neighbours * m)) + m  # self pairs sit at (about) zero
    want = min(want, best.numel() - 1)
    eps2 = 0.5 * (best[want - 1] + best[want]).item()
    return math.sqrt(eps2)


def parity_sample(torch, pts, eps, pairs, stored, rows=1024, seed=7, band=1e-3):
    """Pair-set check of `rows` seeded query rows against FP64 distances to all points (torch FP64 on
    the device, outside the timed region): pairs that disagree with FP64, how many of them lie outside
    the relative `band` around epsilon (must be 0), and the largest relative distance error."""
    n, d = pts.shape
    got = pairs[:stored]
    order = torch.argsort(got[:, 0].to(torch.int64) * n + got[:, 1].to(torch.int64))
    q = got[order, 0].to(torch.int64).contiguous()
    c = got[order, 1].to(torch.int64)
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    sel = torch.sort(torch.randperm(n, generator=g, device="cuda")[:rows]).values
    start, stop = torch.searchsorted(q, sel), torch.searchsorted(q, sel + 1)
    mask = torch.zeros((len(sel), n), dtype=torch.bool, device="cuda")
    for i in range(len(sel)):
        mask[i, c[start[i]:stop[i]]] = True
    xs = pts[sel].to(torch.float64)
    xs2 = (xs * xs).sum(1)
    disagree, outside, worst = 0, 0, 0.0
    chunk = max(1, (1 << 26) // d)
    for c0 in range(0, n, chunk):
        y = pts[c0:c0 + chunk].to(torch.float64)
        d2 = (xs2[:, None] + (y * y).sum(1)[None, :] - 2.0 * (xs @ y.T)).clamp_min(0.0)
        diff = (d2 <= eps * eps) != mask[:, c0:c0 + chunk]
        if bool(diff.any()):
            rel = (d2[diff].sqrt() - eps).abs() / eps
            disagree += int(diff.sum())
            outside += int((rel > band).sum())
            worst = max(worst, float(rel.max()))
    return {"rows": int(len(sel)), "pairs_checked": int((stop - start).sum()), "disagree_with_fp64": disagree,
            "outside_band": outside, "max_rel_distance_error": worst, "band": band}


def cpu_baseline(torch, pts, eps, full_limit=2.0e5, sample_rows=1024, budget_s=100.0, seed=99):
    """Blocked brute-force join on this box's host cores (oracle/blocked_join.c: GEMM form, cache blocked,
    OpenMP), FP64 and FP32, same pair definition as the GPU join.  Small workloads (N <= full_limit) run in
    full; the others join `sample_rows` seeded query rows with ALL N candidates and the time is extrapolated
    linearly (x N / rows), labelled as such.  Candidates are streamed from the device in chunks, every chunk
    is joined three times per precision, the per-pass totals give the median of three.  Only time spent inside
    the join routine counts (the dataset is "already in memory")."""
    import numpy as np

    import oracle

    n, d = pts.shape
    threads = oracle.num_threads()
    full = n <= full_limit
    if full:
        rows = torch.arange(n, device="cuda")
    else:
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        rows = torch.sort(torch.randperm(n, generator=g, device="cuda")[:sample_rows]).values
    q = pts[rows].cpu().numpy().view(np.uint16)
    nq = q.shape[0]
    chunk = int(max(1024, min(n, (1 << 27) // d)))
    chunks = [(c0, min(n, c0 + chunk)) for c0 in range(0, n, chunk)]
    passes = {64: [0.0, 0.0, 0.0], 32: [0.0, 0.0, 0.0]}
    found = {64: [0, 0, 0], 32: [0, 0, 0]}
    repeats = 3
    for i, (c0, c1) in enumerate(chunks):
        c = pts[c0:c1].cpu().numpy().view(np.uint16)
        for precision in (64, 32):
            for r in range(repeats):
                _, f, secs = oracle.blocked_join(q, c, eps, precision, want_pairs=False)
                passes[precision][r] += secs
                found[precision][r] += f
        if i == 0 and repeats == 3:
            # one pass only when three would not fit the budget (said in `median_of`)
            projected = (passes[64][0] + passes[32][0]) * len(chunks) * 3
            if projected > budget_s:
                repeats = 1
        del c

    def rate(precision):
        t = sorted(passes[precision][:repeats])[repeats // 2]
        return {"tflops": 2.0 * nq * n * d / t / 1e12, "seconds": t, "pairs_found": int(found[precision][0]),
                "pairs_per_s": found[precision][0] / t, "extrapolated_full_seconds": t * n / nq}

    fp64, fp32 = rate(64), rate(32)
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    what = "all" if full else f"{nq} seeded"
    return {
        "value": fp32["tflops"], "unit": "TFLOPS", "cores": threads, "kind": "port", "precision_of_value": "fp32",
        "sample": f"{what} query rows x all {n} candidates x D={d} ({'full join' if full else 'time x N/rows is an extrapolation'}), "
                  f"blocked GEMM-form join, {oracle.blocked_join_vector_bits()}-bit vectors",
        "fp64": fp64, "fp32": fp32, "threads": threads, "nproc": os.cpu_count(),
        "affinity": len(os.sched_getaffinity(0)), "cpu_model": model, "median_of": repeats,
        "query_rows": nq, "full": bool(full),
    }


class ClockSampler:
    """Shader clock and board power of GPU 0 while the timed steps run, read from the driver's sysfs files
    (pp_dpm_sclk marks the current clock with '*', hwmon power1_input is microwatts, mem_busy_percent is
    the driver's memory-controller activity) by a thread that makes
    no GPU call.  The MFMA rate of a long join is set by the clock the power limit allows, not by 2.4 GHz."""

    def __init__(self, interval=0.05):
        import glob
        import threading
        self.interval = interval
        dev = "/sys/class/drm/card0/device"
        self.sclk = dev + "/pp_dpm_sclk"
        power = glob.glob(dev + "/hwmon/hwmon*/power1_input") + glob.glob(dev + "/hwmon/hwmon*/power1_average")
        cap = glob.glob(dev + "/hwmon/hwmon*/power1_cap")
        self.power = power[0] if power else None
        self.cap = cap[0] if cap else None
        self.busy = dev + "/mem_busy_percent"
        self.mhz, self.watts, self.mem = [], [], []
        self._stop = threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _read_once(self):
        try:
            with open(self.sclk) as f:
                for line in f:
                    if "*" in line:
                        self.mhz.append(float(line.split(":")[1].lower().split("mhz")[0]))
            if self.power:
                with open(self.power) as f:
                    self.watts.append(float(f.read()) / 1e6)
            with open(self.busy) as f:
                self.mem.append(float(f.read()))
        except (OSError, ValueError, IndexError):
            pass

    def _run(self):
        while not self._stop.wait(self.interval):
            self._read_once()

    def __enter__(self):
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join()

    def summary(self):
        def stat(v):
            return {"mean": sum(v) / len(v), "min": min(v), "max": max(v)} if v else None
        cap = None
        try:
            if self.cap:
                with open(self.cap) as f:
                    cap = float(f.read()) / 1e6
        except (OSError, ValueError):
            pass
        return {"sclk_mhz": stat(self.mhz), "power_w": stat(self.watts), "power_cap_w": cap,
                "mem_busy_percent": stat(self.mem),
                "samples": len(self.mhz), "interval_s": self.interval}


def load_traffic(name):
    """Bytes below the L2 per join-kernel launch, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    and scaled by a plain copy kernel (committed under profiles/); None when not measured."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            entry = json.load(f).get(name)
    except OSError:
        return None, None
    return (entry["total"], entry) if entry else (None, None)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", default="c3", choices=sorted(CONFIGS))
    ap.add_argument("--n", type=int, default=0, help="override the number of points")
    ap.add_argument("--d", type=int, default=0, help="override the dimensionality")
    ap.add_argument("--eps", type=float, default=0.0, help="skip calibration and use this epsilon")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-epilogue", action="store_true", help="measurement: contraction only")
    ap.add_argument("--no-symmetric-option", action="store_true",
                    help="skip the extra launch that measures the opt-in FASTED_SYMMETRIC mode")
    ap.add_argument("--allow-ablation", action="store_true",
                    help="measurement: accept a library built with parts of the join kernel compiled out (FASTED_LIBRARY)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a plain 1 GiB read + 1 GiB write elementwise kernel (to scale FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the single-GPU hot path only: run with --gpus 1 (no multi-GPU path exists)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import fasted_amd
    from fasted_amd import find_pairs as fp

    if not torch.cuda.is_available():
        print("no GPU visible: the join has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    lib = fasted_amd.load_findpairs()
    version = lib.fasted_version().decode()
    ablation = "ABLATION" in version
    if ablation and not (args.no_epilogue or args.allow_ablation):
        print(f"refusing to benchmark a measurement build as the product: {version} (pass --allow-ablation to time "
              "it; its line then says what it is and carries no parity claim)", file=sys.stderr)
        sys.exit(4)

    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(4):
            torch.mul(src, 1.0, out=dst)  # one kernel: reads 2^30 bytes, writes 2^30 bytes
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy": {"read_bytes": 1 << 30, "write_bytes": 1 << 30, "launches": 4}}))
        return

    n, d, kind, neighbours, label = CONFIGS[args.config]
    n = args.n or n
    d = args.d or d
    if args.n or args.d:
        label = f"{kind} {n}x{d} (override of {args.config})"
    pts = generate_points(torch, kind, n, d, seed=20260 + n % 997)
    eps = args.eps or calibrate_epsilon(torch, pts, neighbours, sample=16384 if n >= 500_000 and neighbours <= 100 else 4096)
    # pair buffer: the reference's N*256 records, or 1.25x the expected count when that is larger
    cap = int(max(n * 256, 1.25 * n * (neighbours + 1)))
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    sums = torch.empty(n, dtype=torch.float32, device="cuda")
    flags = fp.FASTED_NO_EPILOGUE if args.no_epilogue else 0

    def step():
        return fp.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=sums.data_ptr(),
                                   flags=flags)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    with ClockSampler() as clocks:
        t0 = time.perf_counter()
        stats = [step() for _ in range(args.steps)]
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0

    ms_per_step = wall * 1000.0 / args.steps
    flops = 2.0 * n * n * d
    tflops = flops / (ms_per_step / 1000.0) / 1e12
    st = stats[-1]
    join_ms = sum(s.joinMs for s in stats) / len(stats)
    sums_ms = sum(s.sumSquaredMs for s in stats) / len(stats)
    timing = "hip events on the launch stream"
    device_clock = None
    if st.tiles <= 512 and not args.no_epilogue:
        # A join this small returns on the join kernel's own report and times its kernels with the device's clock
        # (first instruction of the first workgroup to the last workgroup's sign-off): shorter than the dispatch
        # that events and a profiler's kernel trace see.  The roofline's duration is the events' one, from as
        # many steps again with event timing switched on; these steps are not part of `value`.
        device_clock = {"sum_squared_ms": sums_ms, "join_kernel_ms": join_ms}
        timed = [fp.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=sums.data_ptr(),
                                     flags=flags | fp.FASTED_EVENT_TIMING) for _ in range(args.steps)]
        join_ms = sum(s.joinMs for s in timed) / len(timed)
        sums_ms = sum(s.sumSquaredMs for s in timed) / len(timed)
        timing += " (a second pass of %d steps; the timed steps return on the kernel's report)" % args.steps
    achieved = flops / (join_ms / 1000.0) / 1e12
    traffic, traffic_detail = load_traffic(args.config if not (args.n or args.d) else "")
    out = {
        "metric": "self-join TFLOPS (2*N^2*D/s)", "value": tflops, "unit": "TFLOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": label, "N": n, "D": d, "epsilon": eps, "mean_neighbours_target": neighbours,
                   "pairs_found": int(st.pairsFound), "pairs_stored": int(st.pairsStored),
                   "mean_neighbours": (st.pairsFound - n) / n, "pairs_per_s": st.pairsFound / (ms_per_step / 1000.0),
                   "pct_of_fp16_peak": 100.0 * tflops / PEAK_FP16_TFLOPS, "tiles": int(st.tiles),
                   "sum_squared_ms": sums_ms, "join_kernel_ms": join_ms, "kernel_timing": timing,
                   "kernel_ms_by_device_clock": device_clock, "epilogue": not args.no_epilogue,
                   "accumulate": "f32", "library": version,
                   "library_path": fp.library_path(), "peak_used_tflops": PEAK_FP16_TFLOPS, "clocks": clocks.summary()},
        "roofline": {"bound": "mfma", "kernel": "join_kernel", "achieved": achieved, "peak": PEAK_FP16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_FP16_TFLOPS,
                     "traffic": traffic, "traffic_detail": traffic_detail,
                     "traffic_source": (traffic_detail or {}).get("source")},
    }
    # Parity is part of the measurement: a line whose pair set fails the check (a sampled pair outside the
    # relative 1e-3 band around epsilon, a pair buffer that overflowed so that nothing could be checked, a
    # symmetric-mode count that differs) says so and the process exits non-zero.
    problems = []
    if ablation:
        args.no_symmetric_option = True
        out["config"]["parity_ok"] = None
        out["config"]["note"] = "measurement build: results are wrong by construction, no parity claim"
    if not args.no_epilogue and not ablation:
        if st.pairsStored == st.pairsFound:
            out["config"]["parity_vs_fp64"] = parity_sample(torch, pts, eps, pairs, int(st.pairsStored))
            if out["config"]["parity_vs_fp64"]["outside_band"] > 0:
                problems.append("sampled pairs outside the epsilon band")
        else:
            problems.append("pair buffer overflowed: parity not checked")
    if not args.no_epilogue and not args.no_symmetric_option:
        # Not part of `value`: the opt-in FASTED_SYMMETRIC mode computes only the tiles on and above the
        # diagonal (same pair set).  Its rate is 2*N^2*D over its time, i.e. an *effective* figure: the
        # matrix cores execute about half of those FLOPs.
        sym = fp.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=sums.data_ptr(),
                                  flags=fp.FASTED_SYMMETRIC)
        sym_ms = sym.joinMs + sym.sumSquaredMs
        out["config"]["symmetric_option"] = {
            "ms_per_step": sym_ms, "effective_tflops": flops / (sym_ms / 1000.0) / 1e12,
            "pairs_found": int(sym.pairsFound), "same_pair_count": bool(sym.pairsFound == st.pairsFound),
            "note": "opt-in, not the headline: about half of 2*N^2*D is actually executed"}
        if sym.pairsFound != st.pairsFound:
            problems.append("symmetric mode found a different number of pairs")
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, pts, eps)
        out["cpu_baseline"]["gpu_over_cpu"] = tflops / out["cpu_baseline"]["value"]
    if not args.no_epilogue and not ablation:
        out["config"]["parity_ok"] = not problems
        if problems:
            out["config"]["parity_problems"] = problems
    print(json.dumps(out))
    if problems:
        print("parity check failed: " + "; ".join(problems), file=sys.stderr)
        sys.exit(3)


if __name__ == "__main__":
    main()
