"""The reference's figure specifications (figures/spec/*.yml) select benchmark results by regular
expressions over benchmark names; a drop-in harness must emit names those expressions find.
tests/golden/plot_spec_series.json holds the 673 `regex:` strings (written by
tests/golden/make_plot_spec_fixture.py from the reference's YAML values).  Every one of them must match
at least one name of `bench --benchmark_list_tests`, except the ones listed below with the reason."""
import json
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "tcu_scope_amd", "host", "bench")

# (pattern over the regex string itself, why no benchmark of this build answers to it)
EXCLUDED = [
    # libraries and micro-benchmarks outside the hot path
    (r"^CUTLASS_", "CUTLASS GEMM baselines: a vendored third-party library, not part of the path"),
    (r"^CUDA_Memory_Device_", "memory micro-benchmarks of a scope plugin that is not in the reference's tree"),
    # names that no source file of the reference registers, so they match nothing upstream either
    (r"^CUDA_WMMA_UNSAFE_", "the specs transpose two words: the reference registers CUDA_UNSAFE_WMMA_* (src/unsafe_prefixsum/*.cu)"),
    (r"^CUDA_WMMA_SEGMENTED_REDUCTION_256N_SHORT_CIRCUITED", "no such benchmark in the reference's sources"),
    (r"^CUDA_(UNSAFE_)?WMMA_FULL_REDUCTION_2KERS<", "registered upstream only as ..._2KERS_BASE_16 / _BASE_256 (src/reduction/wmma_2kers.cu:173-177)"),
    (r"^CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_(ATOMIC_BALLOT|BLOCK_SYNC)<256 \\\* 256,",
     "the reference registers the atomic forms up to SEGMENT_SIZE 16 * 256 (src/reduction/wmma_atomic.cu:181-191)"),
]


def _names():
    if not os.path.exists(BENCH):
        subprocess.check_call(["make", "-C", os.path.dirname(BENCH)], stdout=subprocess.DEVNULL)
    out = subprocess.check_output([BENCH, "--benchmark_list_tests"], text=True)
    return [n for n in out.split("\n") if n]


def test_every_series_of_the_reference_figures_finds_a_benchmark():
    names = _names()
    spec = json.load(open(os.path.join(ROOT, "tests", "golden", "plot_spec_series.json")))
    assert len(spec) == 107 and sum(len(v["series"]) for v in spec.values()) == 673
    blob = "\n".join(names)
    used = [0] * len(EXCLUDED)
    matched, unexplained = 0, []
    for fname, v in sorted(spec.items()):
        for s in v["series"]:
            rx = re.compile(s["regex"], re.M)
            hit = rx.search(blob) is not None
            rule = next((i for i, (pat, _) in enumerate(EXCLUDED) if re.search(pat, s["regex"])), None)
            if rule is not None:
                used[rule] += 1
                assert not hit, f"{fname}: {s['regex']!r} is listed as excluded but matches a benchmark: remove the exclusion"
            elif hit:
                matched += 1
            else:
                unexplained.append((fname, s["regex"]))
    assert not unexplained, f"{len(unexplained)} series of the reference's figures match no benchmark name, e.g. {unexplained[:5]}"
    assert all(used), [EXCLUDED[i][0] for i, u in enumerate(used) if not u]
    assert matched == 673 - sum(used) and matched >= 553, (matched, used)


def test_names_of_the_reference_registrations_exist():
    """Spot checks of the registrations the exclusions must not hide (reference file:line in comments)."""
    have = set(_names())
    for n in [
        # src/reduction/seg_wmma_16n_block.cu:229, seg_wmma_256n_block.cu:242, seg_wmma_16n_opt.cu:216
        "CUDA_WMMA_SEGMENTED_REDUCTION_16N_BLOCK<1>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_WMMA_SEGMENTED_REDUCTION_256N_BLOCK<16>/num_segments:1048576/segment_size:256/num_elements:268435456/manual_time",
        "CUDA_WMMA_SEGMENTED_REDUCTION_16N_OPT<2>/num_segments:8388608/segment_size:32/num_elements:268435456/manual_time",
        # src/prefixsum/seg_wmma_16n_block.cu:232, seg_wmma_16n.cu:208
        "CUDA_WMMA_SEGMENTED_PREFIXSUM_16N_BLOCK<1>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_16N<4>/num_segments:67108864/segment_size:16/base_segment_size:16/max_elements_log2:30/manual_time",
        # src/reduction/seg_cub_block.cu:145, :175; src/prefixsum/seg_cub_block.cu:159; src/prefixsum/seg_cub_warp.cu:140, :154
        "CUB_BLOCK_SEGMENTED_REDUCTION<32, 1, BLOCK_REDUCE_RAKING>/num_segments:8388608/segment_size:32/num_elements:268435456/manual_time",
        "CUB_BLOCK_SEGMENTED_REDUCTION<256, 1, BLOCK_REDUCE_RAKING>/num_segments:1048576/segment_size:256/num_elements:268435456/manual_time",
        "CUB_BLOCK_SEGMENTED_PREFIXSUM<32, 1, BLOCK_SCAN_RAKING>/num_segments:8388608/segment_size:32/num_elements:268435456/manual_time",
        "CUB_WARP_SEGMENTED_PREFIXSUM<32, 16>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUB_WARP_SEGMENTED_PREFIXSUM<1024, 32>/num_segments:8388608/segment_size:32/num_elements:268435456/manual_time",
        # src/reduction/wmma_atomic.cu:181, src/prefixsum/wmma_3kers.cu:173, src/reduction/wmma_2kers_block.cu:196
        "CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_BLOCK_SYNC<256, 8>/num_elements:268435456/manual_time",
        "CUDA_WMMA_FULL_PREFIXSUM_3KERS<256, 1>/num_elements:268435456/manual_time",
        "CUDA_WMMA_FULL_REDUCTION_2KERS_BLOCK_BASE_256<64 * 256, 8>/num_elements:268435456/manual_time",
        # src/unsafe_reduction/seg_wmma_16.cu:138-152, seg_wmma_16n_block.cu:230, wmma_atomic.cu:166-172
        "CUDA_UNSAFE_WMMA_SEGMENTED_REDUCTION_16<4, 2>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_UNSAFE_WMMA_SEGMENTED_REDUCTION_16N_BLOCK<1>/num_segments:16777216/segment_size:16/num_elements:268435456/manual_time",
        "CUDA_UNSAFE_WMMAFULL_REDUCTION_ATOMIC_W_BLOCK_SYNC<4 * 256, 8>/num_elements:268435456/manual_time",
        # src/reduction/seg_cub_device.cu:153-155
        "CUB_DEVICE_TUNE_SEGMENTED_REDUCTION/num_segments:262144/segment_size:16/base_segment_size:16/max_elements_log2:22/manual_time",
        # src/gemm/cublas.cu:618-627, src/gemv/wmma_cublas.cu:245-246
        "CUBLAS_GEMM/M:8192/N:8192/K:8192/manual_time",
        "CUDA_WMMA_HGEMV_CUBLAS/M:16384/N:16384/manual_time",
    ]:
        assert n in have, n
