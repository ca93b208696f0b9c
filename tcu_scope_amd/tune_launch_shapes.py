"""Launch-shape sweep of the segmented reduction / inclusive scan: the measurement behind the AUTO tables
(`auto_plan_reduce`, `auto_plan_scan` in csrc/dispatch.hpp), to be repeated when the kernels, the driver or the
machine change.

For one operation and element count, every segment size of the list is run with every combination of kernel family
(wave kernels: WAVE_SHUFFLE, block kernels: BLOCK_LDS), 1 KiB tiles in flight per wave (1, 2, 4, 8), waves per block
(1 ... 16) and XCD run length (blocks of one XCD on consecutive pieces of the array: 0, 8, 32, 128, 512), and once
with AUTO.  With --pads the block kernels of the scan are also run with that many KiB of LDS requested and left
unused per block (option scan_lds_pad), which caps the blocks a compute unit holds (160 KiB per unit: 39 = four
blocks, 52 = three, 79 = two).  The cases are shuffled anew for every repetition; a launch is timed by a pair of HIP events that the
kernel's own dispatch stamps (tcu_time_next_launch); two inputs alternate and the outputs are taken in turn
(three buffers up to 2^28 elements, two beyond), so that nothing is served from or absorbed by the 256 MiB
memory-side cache.  The median over the repetitions is reported as time and as a fraction of 8 TB/s (algorithmic
bytes: reduce 2N + 2N/S, scan 4N).

    python -m tcu_scope_amd.tune_launch_shapes --op scan --n-log2 28 [--sizes 16,256,...] [--pads 0,39,52] [--markdown out.md]
"""
import argparse
import random
import sys


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--op", choices=("reduce", "scan"), default="scan")
    ap.add_argument("--n-log2", type=int, default=28)
    ap.add_argument("--sizes", default=",".join(str(16 << i) for i in range(11)), help="segment sizes, comma separated")
    ap.add_argument("--pads", default="0", help="KiB of unused LDS per block of the scan's block kernels, comma separated (0 = none)")
    ap.add_argument("--repetitions", type=int, default=5)
    ap.add_argument("--top", type=int, default=6, help="how many shapes to list per segment size")
    ap.add_argument("--markdown", default=None, help="append the table to this file")
    args = ap.parse_args()

    import torch

    import tcu_scope_amd as t

    t.init(0)
    stream = torch.cuda.current_stream()
    kind, n = args.op, 1 << args.n_log2
    sizes = [int(s) for s in args.sizes.split(",")]
    pads = [int(p) for p in args.pads.split(",")] if kind == "scan" else [0]
    inputs = [t.generate(n, s, t.Dist.UNIFORM) for s in (1, 2)]
    n_out = 3 if args.n_log2 <= 28 else 2
    outs = [torch.empty(n if kind == "scan" else n // min(sizes), dtype=torch.float16, device="cuda") for _ in range(n_out)]
    run = t.seg_scan if kind == "scan" else t.seg_reduce
    launches = [0]

    def once(S, variant, u, w, c, pad, events=None):
        t.set_option("xcd_run", c)
        t.set_option("scan_lds_pad", pad)
        if events is not None:
            t.time_next_launch(*events)
        i = launches[0]
        launches[0] += 1
        run(inputs[i & 1], S, variant=variant, tiles_per_wave=u, waves_per_block=w, out=outs[i % n_out], stream=stream)

    cases = []
    for S in sizes:
        cases.append((S, t.Variant.AUTO, 0, 0, -1, -1))
        for u in (1, 2, 4, 8):
            for w in (1, 2, 4, 8, 16):
                for c in (0, 8, 32, 128, 512):
                    if S <= 512 or u * 512 <= S * 16:  # a wave takes at most 16 segments of a tile or more
                        cases.append((S, t.Variant.WAVE_SHUFFLE, u, w, c, 0))
                    if S >= 512 and u * w * 512 <= max(S, 512) * 4:  # a block takes at most 4 segments at a time
                        for pad in pads:
                            cases.append((S, t.Variant.BLOCK_LDS, u, w, c, pad))
    times = {}
    try:
        for _ in range(args.repetitions):
            random.shuffle(cases)
            timed = []
            for case in cases:
                try:
                    once(*case)  # warms the case and tells whether the family takes the shape
                except t.TcuError:
                    continue
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(stream)
                b.record(stream)
                timed.append((case, a, b))
            torch.cuda.synchronize()
            for case, a, b in timed:
                once(*case, (a, b))
            torch.cuda.synchronize()
            for case, a, b in timed:
                times.setdefault(case, []).append(a.elapsed_time(b) * 1e3)
    finally:
        t.set_option("xcd_run", -1)
        t.set_option("scan_lds_pad", -1)

    def name(k):
        if k[1] == t.Variant.AUTO:
            return "AUTO"
        return f"{'wave' if k[1] == t.Variant.WAVE_SHUFFLE else 'block'} {k[2]} x {k[3]}, run {k[4]}" + (f", pad {k[5]}" if k[5] else "")

    lines = [f"### {kind}, N = 2^{args.n_log2} ({args.repetitions} shuffled repetitions, median kernel time in us, fraction of 8 TB/s)", "",
             "| segment size | AUTO | " + " | ".join(f"#{i + 1}" for i in range(args.top)) + " |", "|---|---|" + "---|" * args.top]
    for S in sizes:
        by = 4 * n if kind == "scan" else 2 * n + 2 * n // S
        rows = sorted((sorted(v)[len(v) // 2], k) for k, v in times.items() if k[0] == S)
        auto = next(us for us, k in rows if k[1] == t.Variant.AUTO)
        best = [(us, k) for us, k in rows if k[1] != t.Variant.AUTO][:args.top]
        lines.append(f"| {S} | {auto:.1f} ({by / auto / 8e6:.3f}) | " + " | ".join(f"{name(k)}: {us:.1f} ({by / us / 8e6:.3f})" for us, k in best) + " |")
    text = "\n".join(lines) + "\n"
    print(text)
    if args.markdown:
        with open(args.markdown, "a") as f:
            f.write(text + "\n")


if __name__ == "__main__":
    sys.exit(main())
