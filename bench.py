#!/usr/bin/env python3
"""Headline benchmark: fp16 segmented reduction + segmented inclusive prefix sum over
N = 2^28 elements, segment sizes 16..16384, on one MI355X.

A step is one pass over the whole sweep: 5 segmented reductions (seg 16, 256, 1024, 4096,
16384) and 4 segmented scans (seg 16, 256, 2048, 16384), each over 2^28 synthetic
elements already resident in HBM.  Order of the run:

1. every launch of the sweep (and of `all_sizes`: both operations at every power of two from
   16 to 16384) runs once and a window of 2^24 elements of its output is compared with the
   fp64 sums of the same seeded inputs (CPU oracle, |err| <= 2 ulp_fp16 + 1e-3 * sqrt(segment
   size)); a mismatch ends the run with a non-zero status.  Outside every timed region.
2. warm-up steps, then the timed region: exactly `steps` steps, nothing on the stream but the
   launches, wall clock, synchronised on both sides -> `value`.
3. the same steps once more with a pair of HIP events per launch on the launch stream, stamped
   by the kernel's own dispatch with its begin and end (tcu_time_next_launch): per-kernel
   bandwidths and the `roofline` object (algorithmic bytes / average kernel time / 8 TB/s).
4. `all_sizes`, timed like 3.
5. the CPU baseline: the reference's CPU path (restated in oracle/) on the same sweep.

Two input buffers alternate between launches so that no launch finds its input in the 256 MB
Infinity Cache, and the launches write their outputs to `--output-buffers` buffers in turn (default 3:
1.5 GiB of scan output between two launches that write the same lines), so that no launch
overwrites lines an earlier one left dirty in that cache: what a kernel writes has to reach HBM.
"""
import argparse
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
N_LOG2 = 28
REDUCE_SEGS = [16, 256, 1024, 4096, 16384]
SCAN_SEGS = [16, 256, 2048, 16384]
ALL_SIZES = [16 << i for i in range(11)]  # 16 ... 16384
CHECK_WINDOW_LOG2 = 24
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "seg_reduce_scan_2p28_hbm_traffic.md")
KERNEL_SOURCES = ["wave_ops.hpp", "seg_reduce.hpp", "seg_scan.hpp", "dispatch.hpp"]


def kernel_sources_digest():
    """sha256 over the sources that decide what the segmented launches do (kernels and launch shapes)."""
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "tcu_scope_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic():
    """HBM bytes per launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE summary in profiles/, but only if that
    summary was made from the kernel sources of this tree (it records their digest); otherwise nothing."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return {}
    m = re.search(r"kernel sources digest: `([0-9a-f]+)`", text)
    if not m or m.group(1) != kernel_sources_digest():
        return {}
    out = {}
    for op, seg, by in re.findall(r"\|\s*(reduce|scan) seg=(\d+)\s*\|.*?\|\s*(\d+)\s*\|\s*\d+\s*\|\s*[0-9.]+\s*\|\s*$", text, re.M):
        out[(op, int(seg))] = int(by)
    return out


def algorithmic_bytes(kind, n, seg):
    # reduce: read N halves, write N/seg halves; scan: read N, write N
    return 2 * n + (2 * n // seg if kind == "reduce" else 2 * n)


def cpu_baseline(n_log2, threads):
    """The reference's CPU path (fp32 sequential sum per segment, fp16 result) restated in
    C (oracle/), timed on the same sweep at N = 2^n_log2."""
    from oracle import binding as oracle

    n = 1 << n_log2
    x = oracle.generate_f16(n, 1, oracle.DIST_UNIFORM)
    elems = 0
    t0 = time.perf_counter()
    for seg in REDUCE_SEGS:
        oracle.seg_reduce_ref(x, n // seg, seg, nthreads=threads)
        elems += n
    for seg in SCAN_SEGS:
        oracle.seg_scan_ref(x, n // seg, seg, nthreads=threads)
        elems += n
    dt = time.perf_counter() - t0
    return elems / dt / 1e9, dt


def cpu_baseline_config1(threads, seconds=2.0):
    """The same CPU path on the configuration it is quoted on upstream: N = 2^20 halves from seed 0 in 65536
    segments of 16, repeated until about `seconds` of CPU work are done."""
    from oracle import binding as oracle

    n, seg = 1 << 20, 16
    x = oracle.generate_f16(n, 0, oracle.DIST_UNIFORM)
    oracle.seg_reduce_ref(x, n // seg, seg, nthreads=threads)
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        oracle.seg_reduce_ref(x, n // seg, seg, nthreads=threads)
        reps += 1
    dt = time.perf_counter() - t0
    return reps * n / dt / 1e9, reps, dt


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--n-log2", type=int, default=N_LOG2, help="log2 of the element count (28 = the benchmark configuration)")
    ap.add_argument("--variant", default="AUTO", help="kernel family for every launch (AUTO, WAVE_SHUFFLE, MFMA_16N, ...); sizes the family does not cover are reported as skipped, never substituted")
    ap.add_argument("--tiles-per-wave", type=int, default=0)
    ap.add_argument("--waves-per-block", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true", help="skip the comparison with the CPU oracle before timing (for profiler runs)")
    ap.add_argument("--no-all-sizes", action="store_true", help="skip the second list (every power of two 16 ... 16384)")
    ap.add_argument("--with-copy-probe", action="store_true", help="also launch the plain copy kernel over 2^n_log2 halves before timing (calibrates hardware counters)")
    ap.add_argument("--output-buffers", type=int, default=3, help="output buffers the launches take in turn (1 = every launch rewrites the same buffer)")
    ap.add_argument("--scan-store-policy", type=int, default=0, choices=(0, 1, 2), help="stores of the scan kernels: 0 = the library's default, 1 = every other tile of a wave through the cache, 2 = all non-temporal")
    ap.add_argument("--large-n-log2", type=int, default=30, help="element count of the second, larger run of the sweep's segment sizes (0 = leave it out)")
    ap.add_argument("--cpu-n-log2", type=int, default=28, help="element count of the CPU-baseline sample")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (--gpus 1); segments are independent, so a multi-GPU run would be N copies of this one", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import tcu_scope_amd as tcu

    tcu.init(0)
    info = tcu.device_info()
    n = 1 << args.n_log2
    variant = tcu.Variant[args.variant]
    stream = torch.cuda.current_stream()

    seeds = (1, 2)
    inputs = [tcu.generate(n, s, tcu.Dist.UNIFORM) for s in seeds]
    if args.scan_store_policy:
        tcu.set_option("scan_store_policy", args.scan_store_policy)
    n_out = max(1, args.output_buffers)
    red_outs = [torch.empty(n // 16, dtype=torch.float16, device="cuda") for _ in range(n_out)]
    scan_outs = [torch.empty(n, dtype=torch.float16, device="cuda") for _ in range(n_out)]
    red_out, scan_out = red_outs[0], scan_outs[0]  # what launch 0 writes (the checks read these)
    configs = [("reduce", s) for s in REDUCE_SEGS] + [("scan", s) for s in SCAN_SEGS]
    all_sizes = [] if args.no_all_sizes else [("reduce", s) for s in ALL_SIZES] + [("scan", s) for s in ALL_SIZES]

    class Buffers:
        """the arrays one element count works on: alternating inputs, outputs taken in turn"""

        def __init__(self, n, inputs, red_outs, scan_outs):
            self.n, self.inputs, self.red_outs, self.scan_outs = n, inputs, red_outs, scan_outs

    main_buffers = Buffers(n, inputs, red_outs, scan_outs)
    current = [main_buffers]

    turns = {"reduce": 0, "scan": 0}  # launches of each kind so far: a kind's output buffers are taken in turn by its own launches

    def launch(i, kind, seg):
        b = current[0]
        x = b.inputs[i % len(b.inputs)]
        turn = turns[kind] if i else 0  # launch 0 (the checks read its output) writes the first buffer
        turns[kind] += 1
        if kind == "reduce":
            tcu.seg_reduce(x, seg, variant=variant, tiles_per_wave=args.tiles_per_wave, waves_per_block=args.waves_per_block, out=b.red_outs[turn % len(b.red_outs)], stream=stream)
        else:
            tcu.seg_scan(x, seg, variant=variant, tiles_per_wave=args.tiles_per_wave, waves_per_block=args.waves_per_block, out=b.scan_outs[turn % len(b.scan_outs)], stream=stream)

    # families do not cover every size (MFMA_16 is 16 only, ...): such launches are left out and said so
    skipped = []
    for kind, seg in list(dict.fromkeys(configs + all_sizes)):
        try:
            launch(0, kind, seg)
        except tcu.TcuError as e:
            if e.status != 2:
                raise
            skipped.append({"op": kind, "segment_size": seg, "reason": str(e)})
    torch.cuda.synchronize()
    unsupported = {(s["op"], s["segment_size"]) for s in skipped}
    configs = [c for c in configs if c not in unsupported]
    all_sizes = [c for c in all_sizes if c not in unsupported]
    if not configs:
        print("bench.py: the chosen variant covers no launch of the sweep", file=sys.stderr)
        sys.exit(2)

    # 1. every launch once, a window of its output against the fp64 sums of the same inputs
    checked = None
    if not args.no_check:
        from oracle import binding as oracle

        w = min(n, 1 << CHECK_WINDOW_LOG2)
        first = (n - w) // 2  # a window in the middle of the array (a multiple of every segment size)
        x_host = oracle.generate_f16(w, seeds[0], oracle.DIST_UNIFORM, first=first)
        worst_excess = 0.0
        for kind, seg in list(dict.fromkeys(configs + all_sizes)):
            launch(0, kind, seg)
            torch.cuda.synchronize()
            nseg = w // seg
            if kind == "reduce":
                got = red_out[first // seg:first // seg + nseg].cpu().numpy().view(np.uint16)
                ref = oracle.seg_reduce_f64(x_host, nseg, seg)
            else:
                got = scan_out[first:first + w].cpu().numpy().view(np.uint16)
                ref = oracle.seg_scan_f64(x_host, nseg, seg)
            bad, worst, first_bad = oracle.check_f16(got, ref, seg, 2.0, 1e-3)
            if bad:
                print(f"bench.py: seg_{kind} segment_size={seg} disagrees with the CPU oracle: {bad} of {got.size} outside 2 ulp + 1e-3*sqrt(S), first at {first_bad}", file=sys.stderr)
                sys.exit(1)
            worst_excess = max(worst_excess, worst)
        checked = {"launches": len(dict.fromkeys(configs + all_sizes)), "window_elements": w, "window_first": first,
                   "tolerance": "2 ulp_fp16 + 1e-3*sqrt(segment_size) against the fp64 sum", "passed": True}

    if args.with_copy_probe:
        for i in range(4):  # 2*n bytes read + 2*n bytes written per launch, same launch shape as the scan kernels
            tcu.stream_probe(scan_out, inputs[i & 1], 2 * n, 0, 1, 1, stream=stream)
        torch.cuda.synchronize()

    counter = 0
    for _ in range(args.warmup):
        for kind, seg in configs:
            launch(counter, kind, seg)
            counter += 1
    torch.cuda.synchronize()

    # 2. the timed region: exactly `steps` steps, nothing but the launches on the stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        for kind, seg in configs:
            launch(counter, kind, seg)
            counter += 1
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    # 3. the same steps once more with a pair of events per launch, carried by the kernel's own
    # dispatch (tcu_time_next_launch): the pair brackets the kernel and nothing else.  Kept out of
    # the region above because a dispatch that reports its times costs the step about 4 %.
    def timed_with_events(launches, repeats):
        nonlocal counter
        events = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in launches] for _ in range(repeats)]
        for step_events in events:
            for a, b in step_events:  # a torch event gets its handle with its first record
                a.record(stream)
                b.record(stream)
        torch.cuda.synchronize()
        ta = time.perf_counter()
        for k in range(repeats):
            for c, (kind, seg) in enumerate(launches):
                tcu.time_next_launch(*events[k][c])
                launch(counter, kind, seg)
                counter += 1
        torch.cuda.synchronize()
        tb = time.perf_counter()
        rows = []
        for c, (kind, seg) in enumerate(launches):
            ms = sorted(events[k][c][0].elapsed_time(events[k][c][1]) for k in range(repeats))
            avg = sum(ms) / len(ms)
            n = current[0].n
            by = algorithmic_bytes(kind, n, seg)
            rows.append({
                "op": kind, "segment_size": seg, "avg_ms": round(avg, 5), "min_ms": round(ms[0], 5), "median_ms": round(ms[len(ms) // 2], 5),
                "gelem_per_s": round(n / avg / 1e6, 1), "algorithmic_bytes": by, "gb_per_s": round(by / avg / 1e6, 1),
                "frac_hbm_peak": round(by / avg / 1e6 / HBM_PEAK_GBS, 4),
            })
        return rows, (tb - ta) / repeats

    per_config, step_with_events_s = timed_with_events(configs, args.steps)
    default_shapes = args.n_log2 == 28 and variant == tcu.Variant.AUTO and args.tiles_per_wave == 0 and args.waves_per_block == 0
    traffic = measured_traffic() if default_shapes else {}
    for r in per_config:
        r["traffic"] = traffic.get((r["op"], r["segment_size"]))

    # 4. every power of two from 16 to 16384, both operations (not part of `value`)
    all_rows = None
    if all_sizes:
        for kind, seg in all_sizes:  # warm
            launch(counter, kind, seg)
            counter += 1
        all_rows, _ = timed_with_events(all_sizes, max(5, args.steps // 2))

    # 4b. the sweep's segment sizes once more at a larger element count (not part of `value`): an output of
    # 2^(large_n_log2 + 1) bytes is several times the 256 MiB memory-side cache by itself
    large_rows = None
    if args.large_n_log2 and variant == tcu.Variant.AUTO:
        ln = 1 << args.large_n_log2
        large = Buffers(ln, [tcu.generate(ln, s, tcu.Dist.UNIFORM) for s in seeds],
                        [torch.empty(ln // 16, dtype=torch.float16, device="cuda") for _ in range(n_out)],
                        [torch.empty(ln, dtype=torch.float16, device="cuda") for _ in range(min(n_out, 2))])
        current[0] = large
        if not args.no_check:
            from oracle import binding as oracle

            w = 1 << CHECK_WINDOW_LOG2
            first = ln - w  # the last window of the array
            x_host = oracle.generate_f16(w, seeds[0], oracle.DIST_UNIFORM, first=first)
            for kind, seg in configs:
                launch(0, kind, seg)
                torch.cuda.synchronize()
                if kind == "reduce":
                    got = large.red_outs[0][first // seg:first // seg + w // seg].cpu().numpy().view(np.uint16)
                    ref = oracle.seg_reduce_f64(x_host, w // seg, seg)
                else:
                    got = large.scan_outs[0][first:first + w].cpu().numpy().view(np.uint16)
                    ref = oracle.seg_scan_f64(x_host, w // seg, seg)
                bad, worst, first_bad = oracle.check_f16(got, ref, seg, 2.0, 1e-3)
                if bad:
                    print(f"bench.py: seg_{kind} segment_size={seg} at N=2^{args.large_n_log2} disagrees with the CPU oracle: {bad} of {got.size}, first at {first_bad}", file=sys.stderr)
                    sys.exit(1)
        for kind, seg in configs:  # warm
            launch(counter, kind, seg)
            counter += 1
        large_rows, _ = timed_with_events(configs, max(5, args.steps // 2))
        current[0] = main_buffers
        del large

    total_s = t1 - t0
    elems_per_step = len(configs) * n
    value = args.steps * elems_per_step / total_s / 1e9

    # the dominant kernel: the launch that takes the largest share of a step
    dom = max(per_config, key=lambda r: r["avg_ms"])
    roofline = {
        "bound": "hbm", "kernel": f"seg_{dom['op']} segment_size={dom['segment_size']}", "achieved": dom["gb_per_s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": dom["frac_hbm_peak"], "traffic": dom["traffic"], "algorithmic_bytes_per_launch": dom["algorithmic_bytes"], "avg_launch_ms": dom["avg_ms"],
        "min_frac_over_sweep": min(r["frac_hbm_peak"] for r in per_config),
    }
    if all_rows:
        roofline["min_frac_all_sizes_16_to_16384"] = min(r["frac_hbm_peak"] for r in all_rows)

    result = {
        "metric": "fp16 segmented reduce+scan throughput, 2^%d elems, seg 16..16384" % args.n_log2,
        "value": round(value, 2), "unit": "Gelem/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(total_s / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 in/out, f32 accumulate", "data": "synthetic (uniform [-1,1) fp16 from a seeded counter-based generator)",
        "config": {"workload": "segmented sum reduction (seg %s) + segmented inclusive scan (seg %s), N=2^%d fp16 each" % (
                       ",".join(str(s) for k, s in configs if k == "reduce"), ",".join(str(s) for k, s in configs if k == "scan"), args.n_log2),
                   "variant": variant.name, "tiles_per_wave": args.tiles_per_wave, "waves_per_block": args.waves_per_block, "compute_units": info["compute_units"],
                   "input_buffers": len(inputs), "output_buffers": n_out, "scan_store_policy": args.scan_store_policy,
                   "kernel_sources_digest": kernel_sources_digest()},
        "roofline": roofline,
        "checked_against_cpu_oracle": checked,
        "ms_per_step_with_kernel_events": round(step_with_events_s * 1e3, 4),
        "per_config": per_config,
    }
    if skipped:
        result["skipped"] = skipped
    if all_rows:
        result["all_sizes"] = all_rows
    if large_rows:
        result["larger_n"] = {"n_log2": args.large_n_log2, "scan_output_buffers": min(n_out, 2), "rows": large_rows}
        roofline["min_frac_larger_n"] = min(r["frac_hbm_peak"] for r in large_rows)
    if not args.no_cpu_baseline:
        cpu1, dt1 = cpu_baseline(args.cpu_n_log2, 1)
        threads = min(16, os.cpu_count() or 1)
        cpun, dtn = cpu_baseline(args.cpu_n_log2, threads)
        sample = "same 9-launch sweep at N=2^%d per launch (%.1f s of CPU work)" % (args.cpu_n_log2, dt1)
        result["cpu_baseline"] = {"value": round(cpu1, 4), "unit": "Gelem/s", "cores": 1, "kind": "port", "sample": sample}
        result["cpu_baseline_threaded"] = {"value": round(cpun, 4), "unit": "Gelem/s", "cores": threads, "kind": "port", "sample": sample.replace("%.1f s" % dt1, "%.1f s" % dtn)}
        c1, reps1, dtc = cpu_baseline_config1(1)
        result["cpu_baseline_config1"] = {"value": round(c1, 4), "unit": "Gelem/s", "cores": 1, "kind": "port",
                                          "sample": "segmented sum reduction, N=2^20 fp16 from seed 0, 65536 segments of 16: %d passes in %.1f s" % (reps1, dtc)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
