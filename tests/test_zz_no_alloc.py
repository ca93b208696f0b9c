"""tcu_seg_scan_f16_noalloc (the entry point for callers that cannot allocate device memory) against
tcu_seg_scan_f16, through the C ABI: two calls in a row on the look-back path (segments of 2^21 halves and
more, whose partition descriptors live in the library's built-in scratch array), the second with a smaller
input, so that what the first call left in the array must not matter; then the paths that need no scratch,
and the size limit.  Bar: inputs on the k/2048 grid (exact fp32 partial sums) bit for bit equal to the
existing entry point and to the rounded fp64 prefix; uniform inputs within 2 ulp_fp16 + 1e-3*sqrt(segment
size) of the fp64 prefix for both entry points (the look-back's fp32 carry depends on timing in its last bit,
so two calls of either entry point need not agree bit for bit on such inputs)."""
import numpy as np
import pytest

from gpu_common import expect_ok, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tcu():
    import tcu_scope_amd as t

    t.init(0)
    return t


def _both(tcu, oracle, x16, seg, what, exact):
    import torch

    n = x16.size
    nseg = n // seg
    xd = to_dev(x16)
    ref = oracle.seg_scan_f64(x16, nseg, seg)
    tot_a = torch.zeros(nseg, dtype=torch.float16, device="cuda")
    tot_b = torch.zeros(nseg, dtype=torch.float16, device="cuda")
    out_b = torch.full((n,), float("nan"), dtype=torch.float16, device="cuda")
    got_a = to_host(tcu.seg_scan(xd, seg, totals=tot_a))
    got_b = to_host(tcu.seg_scan_noalloc(xd, seg, out_b, totals=tot_b))
    ref_tot = ref.reshape(nseg, seg)[:, -1]
    if exact:
        want = ref.astype(np.float16).view(np.uint16)
        assert np.array_equal(got_a, want), what + ": tcu_seg_scan_f16 vs rounded fp64 prefix"
        assert np.array_equal(got_b, got_a), what + ": tcu_seg_scan_f16_noalloc differs from tcu_seg_scan_f16"
        assert np.array_equal(to_host(tot_b), to_host(tot_a)), what + ": totals differ"
        assert np.array_equal(to_host(tot_b), want.reshape(nseg, seg)[:, -1]), what + ": totals vs rounded fp64 sums"
    else:
        expect_ok(oracle, got_a, ref, seg, what + ": tcu_seg_scan_f16")
        expect_ok(oracle, got_b, ref, seg, what + ": tcu_seg_scan_f16_noalloc")
        expect_ok(oracle, to_host(tot_b), ref_tot, seg, what + ": tcu_seg_scan_f16_noalloc totals")
        # the two entry points against each other: both are within the bound of the same fp64 prefix, so
        # they are within twice the bound of each other
        a = got_a.view(np.float16).astype(np.float64)
        b = got_b.view(np.float16).astype(np.float64)
        bound = 2 * (2 * np.maximum(np.spacing(np.abs(a).astype(np.float16)).astype(np.float64), 2.0 ** -24) + 1e-3 * np.sqrt(seg))
        assert (np.abs(a - b) <= bound).all(), what + ": the two entry points disagree beyond the tolerance"


def test_noalloc_allocates_nothing(tcu, oracle):
    """The property the entry point is named for, on its look-back path (the only path of tcu_seg_scan_f16 that takes
    temporary memory): the library's count of temporary allocations and the device's free memory do not move across
    the call -- made before any other call of this test has warmed the library's memory pool -- while the same
    call through tcu_seg_scan_f16 does take temporary memory.  On a side stream as well, whose device the scratch
    array is looked up for."""
    import torch

    n, seg = 1 << 22, 1 << 21
    g = oracle.generate_f16(n, 39, oracle.DIST_GRID)
    xd = to_dev(g)
    out = torch.empty(n, dtype=torch.float16, device="cuda")
    want = oracle.seg_scan_f64(g, n // seg, seg).astype(np.float16).view(np.uint16)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):  # the stream's first launch sets up its queue: not part of what is measured
        out.zero_()
    torch.cuda.synchronize()
    for stream in (None, side):
        allocations, free = tcu.temporary_allocations(), torch.cuda.mem_get_info()[0]
        tcu.seg_scan_noalloc(xd, seg, out, stream=stream)
        torch.cuda.synchronize()
        assert tcu.temporary_allocations() == allocations, "tcu_seg_scan_f16_noalloc took temporary device memory"
        assert torch.cuda.mem_get_info()[0] == free, "free device memory changed across tcu_seg_scan_f16_noalloc"
        assert np.array_equal(to_host(out), want)
        out.zero_()
    allocations = tcu.temporary_allocations()
    tcu.seg_scan(xd, seg, out=out)
    assert tcu.temporary_allocations() == allocations + 1  # the counter does see the allocating entry point
    assert np.array_equal(to_host(out), want)


def test_noalloc_matches_seg_scan_on_two_calls_in_a_row(tcu, oracle):
    # first call: 2^24 halves in 4 segments of 2^22 (256 partitions); second call: 2^22 halves in 2 segments of
    # 2^21 (64 partitions) - fewer descriptors than the first call left behind
    for call, (n_log2, seg_log2) in enumerate([(24, 22), (22, 21)]):
        n, seg = 1 << n_log2, 1 << seg_log2
        g = oracle.generate_f16(n, 40 + call, oracle.DIST_GRID)
        assert np.abs(oracle.seg_scan_f64(g, n // seg, seg)).max() < 8192  # every fp32 partial sum is exact
        _both(tcu, oracle, g, seg, f"call {call} grid inputs n=2^{n_log2} seg=2^{seg_log2}", exact=True)
    for call, (n_log2, seg_log2) in enumerate([(24, 23), (21, 21)]):
        n, seg = 1 << n_log2, 1 << seg_log2
        x = oracle.generate_f16(n, 50 + call, oracle.DIST_UNIFORM)
        _both(tcu, oracle, x, seg, f"call {call} uniform inputs n=2^{n_log2} seg=2^{seg_log2}", exact=False)


def test_noalloc_other_paths_and_limit(tcu, oracle):
    import torch

    # sizes and variants that need no scratch run the same kernels: bit for bit on any input
    x = oracle.generate_f16(1 << 20, 60, oracle.DIST_UNIFORM)
    xd = to_dev(x)
    for seg, variant in [(16, tcu.Variant.AUTO), (256, tcu.Variant.MFMA_256), (2048, tcu.Variant.AUTO), (16384, tcu.Variant.BLOCK_LDS), (24, tcu.Variant.AUTO)]:
        nseg = x.size // seg
        xs = xd[:nseg * seg]
        out = torch.zeros(nseg * seg, dtype=torch.float16, device="cuda")
        tcu.seg_scan_noalloc(xs, seg, out, variant=variant)
        assert torch.equal(out, tcu.seg_scan(xs, seg, variant=variant)), (seg, variant.name)
    # empty input
    tcu.seg_scan_noalloc(xd[:0], 1 << 21, xd[:0])
    # beyond the built-in array: 131073 partitions of 65536 halves.  Rejected on the host before anything is
    # launched, so the (far too small) buffers are never touched
    small = torch.zeros(1 << 21, dtype=torch.float16, device="cuda")
    with pytest.raises(tcu.TcuError) as e:
        tcu.seg_scan_noalloc(small, 1 << 21, small, num_segments=(1 << 12) + 1)
    assert e.value.status == 2 and "scratch" in str(e.value)
    # exactly at the limit the host side accepts the size; not launched here (that would need 16 GiB)


def test_noalloc_in_a_captured_graph(tcu, oracle):
    """What the entry point is for: its launches recorded into a HIP graph (no allocation, no memset node) and replayed.
    Three segment sizes: the wave kernel, the block scan with its LDS request (whose kernel may meet its first launch,
    and with it the host-side attribute calls, inside the capture) and the look-back path with its clearing kernel.
    Three replays with the program's own eager work and synchronisations between them, each checked bit for bit
    against the rounded fp64 prefix (inputs on the k/2048 grid)."""
    import torch

    n = 1 << 23
    x16 = oracle.generate_f16(n, 77, oracle.DIST_GRID)
    xd = to_dev(x16)
    sizes = (256, 8192, 1 << 22)
    want = {s: oracle.seg_scan_f64(x16, n // s, s).astype(np.float16).view(np.uint16) for s in sizes}
    outs = {s: torch.empty(n, dtype=torch.float16, device="cuda") for s in sizes}
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for s in sizes:
                tcu.seg_scan_noalloc(xd, s, outs[s], stream=side)
    for replay in range(3):
        for s in sizes:
            outs[s].fill_(float("nan"))
        eager = to_host(tcu.seg_scan(xd, 2048))  # eager work of the program between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for s in sizes:
            assert np.array_equal(to_host(outs[s]), want[s]), (replay, s)
        assert np.array_equal(eager, oracle.seg_scan_f64(x16, n // 2048, 2048).astype(np.float16).view(np.uint16))
