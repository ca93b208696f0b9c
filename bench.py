#!/usr/bin/env python3
"""Headline benchmark: fp16 segmented reduction + segmented inclusive prefix sum over
N = 2^28 elements, segment sizes 16..16384, on one MI355X.

A step is one pass over the whole sweep: 5 segmented reductions (seg 16, 256, 1024, 4096,
16384) and 4 segmented scans (seg 16, 256, 2048, 16384), each over 2^28 synthetic
elements already resident in HBM.  `value` = elements processed per second over the
timed steps (wall clock, synchronised on both sides).  The same steps then run once more
with a pair of HIP events per launch on the launch stream, stamped by the kernel's own
dispatch with its begin and end (tcu_time_next_launch); from those come the per-kernel
bandwidths and the `roofline` object (algorithmic bytes / average kernel time / 8 TB/s).
Two input buffers alternate between launches so that no launch finds its input in the
256 MB Infinity Cache.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
N_LOG2 = 28
REDUCE_SEGS = [16, 256, 1024, 4096, 16384]
SCAN_SEGS = [16, 256, 2048, 16384]


# HBM bytes per launch at N = 2^28 with the AUTO launch shapes, from rocprofv3 FETCH_SIZE /
# WRITE_SIZE runs of this script, each counter scaled by what it reads for the plain copy
# kernel of known size (profiles/seg_reduce_scan_2p28_hbm_traffic.md).
MEASURED_TRAFFIC_2P28_AUTO = {
    ("reduce", 16): 570417963, ("reduce", 256): 538966187, ("reduce", 1024): 537931269, ("reduce", 4096): 537925093, ("reduce", 16384): 537136897,
    ("scan", 16): 1073728548, ("scan", 256): 1073787570, ("scan", 2048): 1073609230, ("scan", 16384): 1073637069,
}


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--n-log2", type=int, default=N_LOG2, help="log2 of the element count (28 = the benchmark configuration)")
    ap.add_argument("--variant", default="AUTO", help="kernel family for every launch (AUTO, WAVE_SHUFFLE, MFMA_16N, ...)")
    ap.add_argument("--tiles-per-wave", type=int, default=0)
    ap.add_argument("--waves-per-block", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--with-copy-probe", action="store_true", help="also launch the plain copy kernel over 2^n_log2 halves before timing (calibrates hardware counters)")
    ap.add_argument("--cpu-n-log2", type=int, default=28, help="element count of the CPU-baseline sample")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (--gpus 1); segments are independent, so a multi-GPU run would be N copies of this one", file=sys.stderr)
        sys.exit(2)

    import torch

    import tcu_scope_amd as tcu

    tcu.init(0)
    info = tcu.device_info()
    n = 1 << args.n_log2
    variant = tcu.Variant[args.variant]
    stream = torch.cuda.current_stream()

    inputs = [tcu.generate(n, 1, tcu.Dist.UNIFORM), tcu.generate(n, 2, tcu.Dist.UNIFORM)]
    red_out = torch.empty(n // 16, dtype=torch.float16, device="cuda")
    scan_out = torch.empty(n, dtype=torch.float16, device="cuda")
    configs = [("reduce", s) for s in REDUCE_SEGS] + [("scan", s) for s in SCAN_SEGS]

    def supported(kind, seg):
        V = tcu.Variant
        if variant in (V.BLOCK_LDS, V.MFMA_256N_BLOCK, V.MFMA_16N_BLOCK):
            return seg >= 512
        if variant == V.MFMA_16:
            return seg == 16
        if variant == V.MFMA_256:
            return seg == 256
        if variant == V.MFMA_256N:
            return seg >= 256
        return True

    def launch(i, kind, seg):
        x = inputs[i & 1]
        v = variant if supported(kind, seg) else tcu.Variant.AUTO
        if kind == "reduce":
            tcu.seg_reduce(x, seg, variant=v, tiles_per_wave=args.tiles_per_wave, waves_per_block=args.waves_per_block, out=red_out, stream=stream)
        else:
            tcu.seg_scan(x, seg, variant=v, tiles_per_wave=args.tiles_per_wave, waves_per_block=args.waves_per_block, out=scan_out, stream=stream)

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

    # the timed region: exactly `steps` steps, nothing but the launches on the stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        for kind, seg in configs:
            launch(counter, kind, seg)
            counter += 1
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    # the same steps once more with a pair of events per launch, carried by the kernel's own
    # dispatch (tcu_time_next_launch): the pair brackets the kernel and nothing else.  Kept out of
    # the region above because a dispatch that reports its times costs the step about 4 %
    # (1.09 against 1.05 ms; an event recorded before and after every launch 1.12).
    events = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in configs] for _ in range(args.steps)]
    for step_events in events:
        for a, b in step_events:  # a torch event gets its handle with its first record
            a.record(stream)
            b.record(stream)
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for k in range(args.steps):
        for c, (kind, seg) in enumerate(configs):
            tcu.time_next_launch(*events[k][c])
            launch(counter, kind, seg)
            counter += 1
    torch.cuda.synchronize()
    t3 = time.perf_counter()

    total_s = t1 - t0
    elems_per_step = len(configs) * n
    value = args.steps * elems_per_step / total_s / 1e9

    measured_shapes = args.n_log2 == 28 and variant == tcu.Variant.AUTO and args.tiles_per_wave == 0 and args.waves_per_block == 0
    per_config = []
    for c, (kind, seg) in enumerate(configs):
        ms = sorted(events[k][c][0].elapsed_time(events[k][c][1]) for k in range(args.steps))
        avg = sum(ms) / len(ms)
        by = algorithmic_bytes(kind, n, seg)
        per_config.append({
            "op": kind, "segment_size": seg, "avg_ms": round(avg, 5), "min_ms": round(ms[0], 5), "median_ms": round(ms[len(ms) // 2], 5),
            "gelem_per_s": round(n / avg / 1e6, 1), "algorithmic_bytes": by, "gb_per_s": round(by / avg / 1e6, 1),
            "frac_hbm_peak": round(by / avg / 1e6 / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_2P28_AUTO.get((kind, seg)) if measured_shapes else None,
        })
    # the dominant kernel: the launch that takes the largest share of a step
    dom = max(per_config, key=lambda r: r["avg_ms"])
    roofline = {
        "bound": "hbm", "kernel": f"seg_{dom['op']} segment_size={dom['segment_size']}", "achieved": dom["gb_per_s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": dom["frac_hbm_peak"], "traffic": dom["traffic"], "algorithmic_bytes_per_launch": dom["algorithmic_bytes"], "avg_launch_ms": dom["avg_ms"],
        "min_frac_over_sweep": min(r["frac_hbm_peak"] for r in per_config),
    }

    result = {
        "metric": "fp16 segmented reduce+scan throughput, 2^%d elems, seg 16..16384" % args.n_log2,
        "value": round(value, 2), "unit": "Gelem/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(total_s / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 in/out, f32 accumulate", "data": "synthetic (uniform [-1,1) fp16 from a seeded counter-based generator)",
        "config": {"workload": "segmented sum reduction (seg 16,256,1024,4096,16384) + segmented inclusive scan (seg 16,256,2048,16384), N=2^%d fp16 each" % args.n_log2,
                   "variant": variant.name, "tiles_per_wave": args.tiles_per_wave, "waves_per_block": args.waves_per_block, "compute_units": info["compute_units"]},
        "roofline": roofline,
        "ms_per_step_with_kernel_events": round((t3 - t2) / args.steps * 1e3, 4),
        "per_config": per_config,
    }
    if not args.no_cpu_baseline:
        cpu1, dt1 = cpu_baseline(args.cpu_n_log2, 1)
        threads = min(16, os.cpu_count() or 1)
        cpun, dtn = cpu_baseline(args.cpu_n_log2, threads)
        sample = "same 9-launch sweep at N=2^%d per launch (%.1f s of CPU work)" % (args.cpu_n_log2, dt1)
        result["cpu_baseline"] = {"value": round(cpu1, 4), "unit": "Gelem/s", "cores": 1, "kind": "port", "sample": sample}
        result["cpu_baseline_threaded"] = {"value": round(cpun, 4), "unit": "Gelem/s", "cores": threads, "kind": "port", "sample": sample.replace("%.1f s" % dt1, "%.1f s" % dtn)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
