"""The C++ benchmark harness: names and argument grammar on the CPU, real runs on the GPU."""
import json
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "tcu_scope_amd", "host", "bench")


def _bench():
    if not os.path.exists(BENCH):
        subprocess.check_call(["make", "-C", os.path.dirname(BENCH)], stdout=subprocess.DEVNULL)
    return BENCH


def test_benchmark_names_follow_the_reference_grammar():
    names = subprocess.check_output([_bench(), "--benchmark_list_tests"], text=True).split("\n")
    names = [n for n in names if n]
    have = set(names)
    # spot checks taken from the reference's registrations and plot specs
    for n in [
        "CUDA_WMMA_SEGMENTED_REDUCTION_16<1, 8>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_WMMA_SEGMENTED_REDUCTION_16N<8>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_WMMA_SEGMENTED_REDUCTION_256<4, 2>/num_segments:1048576/segment_size:256/num_elements:268435456/manual_time",
        "CUDA_WMMA_SEGMENTED_REDUCTION_256N_BLOCK<16>/num_segments:16384/segment_size:16384/num_elements:268435456/manual_time",
        "CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_256N<4>/num_segments:4194304/segment_size:256/base_segment_size:256/max_elements_log2:30/manual_time",
        "CUB_WARP_SEGMENTED_REDUCTION<256, 16>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUB_BLOCK_SEGMENTED_PREFIXSUM<512, 32, BLOCK_SCAN_RAKING>/num_segments:16384/segment_size:16384/num_elements:268435456/manual_time",
        "CUDA_WMMA_SEGMENTED_PREFIXSUM_16<4, 2>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_WMMA_SEGMENTED_PREFIXSUM_256N<2>/num_segments:131072/segment_size:2048/num_elements:268435456/manual_time",
        "CUDA_WMMA_FULL_REDUCTION_2KERS_BASE_16<2 * 256, 1>/num_elements:4096/manual_time",
        "CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_ATOMIC_BALLOT<4 * 256, 4>/num_elements:1073741824/manual_time",
        "CUDA_WMMA_FULL_PREFIXSUM_3KERS<8 * 256, 8>/num_elements:1073741824/manual_time",
        "CUDA_WMMA_GEMM/M:8192/N:8192/K:8192/manual_time",
        "CUDA_WMMA_GEMM_NAIVE/M:8192/N:8192/K:8192/manual_time",
        "CUDA_WMMA_GEMM/M:9728/N:9728/K:9728/manual_time",
        "CUDA_WMMA_HGEMM/M:28160/N:28160/K:28160/manual_time",
        "CUDA_WMMA_GEMV_NAIVE/M:25600/N:25600/manual_time",
        "CUDA_WMMA_GEMV_NAIVE/M:16384/N:16384/manual_time",
        "CPU_SEQUENTIAL_SEGMENTED_REDUCTION/num_segments:65536/segment_size:16/num_elements:1048576/manual_time",
        # the "unsafe" twins and the library baselines that the reference's plot specs select
        "CUDA_UNSAFE_WMMA_SEGMENTED_REDUCTION_16N<8>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_UNSAFE_WMMA_SEGMENTED_REDUCTION_16N_OPT<2>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_UNSAFE_WMMA_SEGMENTED_PREFIXSUM_256N_BLOCK<4>/num_segments:16384/segment_size:16384/num_elements:268435456/manual_time",
        "CUDA_UNSAFE_WMMA_TUNE_SEGMENTED_REDUCTION_256N<4>/num_segments:4194304/segment_size:256/base_segment_size:256/max_elements_log2:30/manual_time",
        "CUDA_UNSAFE_WMMAFULL_REDUCTION_ATOMIC_W_ATOMIC_BALLOT<2 * 256, 4>/num_elements:1073741824/manual_time",
        "CUDA_WMMA_FULL_REDUCTION_2KERS_BLOCK_BASE_256<8 * 256, 16>/num_elements:1073741824/manual_time",
        "CUB_DEVICE_SEGMENTED_REDUCTION/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUB_FULL_REDUCTION/num_elements:1073741824/manual_time",
        "CUB_FULL_PREFIXSUM/num_elements:1073741824/manual_time",
        "CUBLAS_WMMA_GEMM/M:8192/N:8192/K:8192/manual_time",
        # fp16-output twins (reference src/gemm/wmma.cu:777, wmma_naive.cu:340, src/gemv/wmma_naive.cu:358, src/gemm/cublas.cu:623)
        "CUDA_WMMA_HGEMM/M:8192/N:8192/K:8192/manual_time",
        "CUDA_WMMA_HGEMM_NAIVE/M:8192/N:8192/K:8192/manual_time",
        "CUDA_WMMA_HGEMV_NAIVE/M:16384/N:16384/manual_time",
        "CUBLAS_WMMA_HGEMM/M:8192/N:8192/K:8192/manual_time",
        "CUDA_WMMA_GEMM_ACCURACY/M:1024/N:1024/K:1024/manual_time",
        "CUDA_WMMA_GEMV_ACCURACY/M:4096/N:4096/manual_time",
    ]:
        assert n in have, n
    # the filter is a regular expression over those names
    out = subprocess.check_output([_bench(), "--benchmark_list_tests", "--benchmark_filter=CUDA_WMMA_SEGMENTED_REDUCTION_16N<(4|8)>.*segment_size:256/"], text=True).split()
    assert len(out) == 2 * 19 and all(re.search(r"_16N<(4|8)>", n) for n in out)


@pytest.mark.gpu
def test_harness_runs_verifies_and_reports(tmp_path):
    out = tmp_path / "out.json"
    filt = ("(CUDA_WMMA_SEGMENTED_(REDUCTION|PREFIXSUM)_(16<1, 4>|256<1, 4>|16N<4>|256N<4>|256N_BLOCK<4>)|CUB_(WARP|BLOCK)_SEGMENTED_(REDUCTION|PREFIXSUM)<(256, 16|512, 32, BLOCK_(SCAN|REDUCE)_RAKING)>"
            "|TCU_AUTO_SEGMENTED_(REDUCTION|PREFIXSUM))/.*num_elements:4194304/"
            "|CUDA_WMMA_FULL_(REDUCTION_(2KERS_BASE_16|ATOMIC_W_BLOCK_SYNC)|PREFIXSUM_(3KERS|CG))<8 \\* 256, 4>/num_elements:4194304/"
            "|CUDA_WMMA_H?GEM[MV](_NAIVE)?/M:512/|TCU_(WAVE|COL_MAJOR)_H?GEMV/M:512/|CPU_SEQUENTIAL_SEGMENTED_REDUCTION/num_segments:65536/"
            "|CUDA_UNSAFE_WMMA_SEGMENTED_(REDUCTION|PREFIXSUM)_(16N<4>|256N_BLOCK<4>)/.*num_elements:4194304/"
            "|CUB_FULL_(REDUCTION|PREFIXSUM)/num_elements:4194304/|CUB_DEVICE_SEGMENTED_REDUCTION/.*segment_size:256/num_elements:4194304/|CUBLAS_(WMMA_H?GEMM|GEMV)/M:512/|HIPBLASLT_H?GEMM/M:512/"
            "|(THRUST|TCU_BY_KEY)_SEGMENTED_(REDUCTION|PREFIXSUM)/.*segment_size:(16|2048)/num_elements:4194304/|THRUST_FULL_(REDUCTION|PREFIXSUM)/num_elements:4194304/")
    p = subprocess.run([BENCH, f"--benchmark_filter={filt}", "--benchmark_min_time=0.02", f"--benchmark_out={out}", "--benchmark_out_format=json", "--tcu_verify=all", "--v=1"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "ERROR OCCURRED" not in p.stdout, p.stdout
    data = json.loads(out.read_text())
    rows = data["benchmarks"]
    assert len(rows) >= 54
    for r in rows:
        assert r["iterations"] >= 1 and r["real_time"] > 0 and r["flops"] > 0, r
        assert r["name"].endswith("/manual_time")
    # the accuracy comparisons report agreement counters instead of rates
    out2 = tmp_path / "acc.json"
    p = subprocess.run([BENCH, "--benchmark_filter=CUDA_WMMA_GEM[MV]_ACCURACY/M:(512|96)/", "--benchmark_min_time=0.01", f"--benchmark_out={out2}", "--benchmark_out_format=json"],
                       capture_output=True, text=True, timeout=120)
    assert p.returncode == 0 and "ERROR OCCURRED" not in p.stdout, p.stdout + p.stderr
    acc = {r["name"]: r for r in json.loads(out2.read_text())["benchmarks"]}
    assert len(acc) == 4
    for name, r in acc.items():
        # GEMM: two kernels that add the same fp32 products in different groupings; GEMV: fp16-rounded operands
        # against the fp32 originals (relative error of a sum of positive terms stays near 2^-11)
        assert r["max_rel_diff"] < (1e-5 if "GEMM" in name else 1e-3), r
        assert r["errors"] >= 0 and r["max_abs_diff"] >= 0
    # precondition failures surface as skipped benchmarks, as in the reference
    p = subprocess.run([BENCH, "--benchmark_filter=CUDA_WMMA_FULL_REDUCTION_2KERS_BASE_16<16 \\* 256, 1>/num_elements:4096/", "--benchmark_min_time=0.01"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0 and "ERROR OCCURRED" not in p.stdout  # 4096 is a multiple of 4096: runs
    p = subprocess.run([BENCH, "--benchmark_filter=CUDA_WMMA_SEGMENTED_REDUCTION_16N_BLOCK<4>/.*segment_size:512/num_elements:4096/", "--tcu_input=constant", "--benchmark_min_time=0.01"],
                       capture_output=True, text=True, timeout=120)
    assert p.returncode == 0 and "ERROR OCCURRED" not in p.stdout, p.stdout


def _series_points(rows, regex, xfield, yfield):
    """What the reference's plotting tool does with one `series:` entry (tools/plot.py:105-163, restated): anchor the
    regex, keep the benchmarks it finds that did not fail, take the key:value parts of the name as fields where the
    row has none of that name, drop rows whose x or y is missing or zero, sort by x."""
    rx = re.compile(regex if regex.startswith("^") else "^" + regex)
    pts = []
    for b in rows:
        if not rx.search(b["name"]) or b.get("error_occurred", False):
            continue
        fields = dict(b)
        for part in b["name"].split("/")[1:]:
            if part != "manual_time" and ":" in part:
                k, v = part.split(":", 1)
                fields.setdefault(k, float(v))
        if xfield in fields and yfield in fields and float(fields[xfield]) != 0 and float(fields[yfield]) != 0:
            pts.append((float(fields[xfield]), float(fields[yfield])))
    return sorted(pts)


@pytest.mark.gpu
def test_json_output_feeds_the_reference_figure_specs(tmp_path):
    """The JSON the harness writes goes through the selection steps of the reference's plotting tool for three of
    its figure specifications (one per x axis: num_elements, num_segments, M) and yields a curve for every series
    this build has benchmarks for."""
    spec = json.loads(open(os.path.join(os.path.dirname(__file__), "golden", "plot_spec_series.json")).read())
    out = tmp_path / "figs.json"
    filt = ("^(CUB_FULL_PREFIXSUM|CUDA_WMMA_FULL_PREFIXSUM_3KERS<(256|8 \\* 256), (1|2|4|8)>)/num_elements:(4096|65536|1048576|16777216)/"
            "|^(THRUST_SEGMENTED_PREFIXSUM|CUB_WARP_SEGMENTED_PREFIXSUM<256, 16>|CUDA_WMMA_SEGMENTED_PREFIXSUM_16<(1|2), 2>)/num_segments:(1024|16384|262144)/segment_size:16/"
            "|^(CUDA_WMMA_HGEMM|CUDA_WMMA_GEMM_NAIVE|CUBLAS_HGEMM|CUBLAS_WMMA_HGEMM)/M:(256|512|1024)/N:(256|512|1024)/K:(256|512|1024)/")
    p = subprocess.run([BENCH, f"--benchmark_filter={filt}", "--benchmark_min_time=0.01", f"--benchmark_out={out}", "--benchmark_out_format=json"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout + p.stderr
    doc = json.loads(out.read_text())
    assert {"context", "benchmarks"} <= set(doc) and "date" in doc["context"]
    rows = doc["benchmarks"]
    curves = 0
    for fig, min_points in (("full_prefixsum.yml", 3), ("segmented_prefixsum_16.yml", 3), ("gemm_16_16.yml", 3)):
        s = spec[fig]
        xfield, yfield = s["xaxis"]["field"], s["yaxis"]["field"]
        assert yfield == "flops"
        for series in s["series"]:
            pts = _series_points(rows, series["regex"], series.get("xfield", xfield), series.get("yfield", yfield))
            if not pts:
                continue  # a series whose benchmarks the filter above leaves out (other template arguments, CUTLASS)
            xs = [x for x, _ in pts]
            assert len(pts) >= min_points and len(set(xs)) == len(xs), (fig, series["regex"], pts)
            assert all(y > 0 and y == y for _, y in pts)
            curves += 1
    assert curves >= 12, curves
