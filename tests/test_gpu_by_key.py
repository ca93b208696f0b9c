"""GPU parity of tcu_seg_scan_by_key_f16 / tcu_seg_reduce_by_key_f16 (segments = runs of equal consecutive keys,
the semantics of the reference's thrust::inclusive_scan_by_key / thrust::reduce_by_key baselines,
src/prefixsum/seg_thrust.cu:46-47, src/reduction/seg_thrust.cu:50-51) against the CPU oracle, through the C ABI.
Tolerance: |out - fp64 sum| <= 2 ulp_fp16(result) + 1e-3*sqrt(run length); inputs on the k/2048 grid bit for bit."""
import numpy as np
import pytest

from gpu_common import to_dev, to_host

pytestmark = pytest.mark.gpu

PART = 4 * 16 * 512  # elements per block of the kernel


@pytest.fixture(scope="module")
def tcu():
    import tcu_scope_amd as t

    t.init(0)
    return t


def keys_with_runs(rng, n, mean_run, wide):
    heads = rng.random(n) < 1.0 / mean_run
    ids = np.cumsum(heads)
    k = (ids * 7919) % 1013 - 500  # neighbouring runs always differ, equal keys come back in later runs
    if wide:
        k = k + (ids % 2) * (1 << 40)
    return k


def run_lengths(keys):
    starts = np.flatnonzero(np.r_[True, keys[1:] != keys[:-1]])
    lens = np.diff(np.r_[starts, keys.size])
    return starts, lens


def allow_for(ref, length):
    return 2 * np.maximum(np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64), 2.0 ** -24) + 1e-3 * np.sqrt(length)


@pytest.mark.parametrize("bits", [32, 64])
def test_by_key_against_the_oracle(tcu, oracle, bits):
    import torch

    rng = np.random.default_rng(100 + bits)
    dt, kt = (torch.int32, np.int32) if bits == 32 else (torch.int64, np.int64)
    for n, mean_run in ((1, 1), (9, 2), (PART - 5, 30), (PART + 1, 1), (5 * PART + 123, 3), (1 << 22, 17), (1 << 22, 900), ((1 << 22) + 8, 70000), (1 << 21, 10 ** 9)):
        keys = keys_with_runs(rng, n, mean_run, bits == 64).astype(kt)
        x = oracle.generate_f16(n, 3 + mean_run % 1000, oracle.DIST_UNIFORM)
        g = oracle.generate_f16(n, 4 + mean_run % 1000, oracle.DIST_GRID)
        kd, xd, gd = torch.from_numpy(keys).cuda(), to_dev(x), to_dev(g)
        starts, lens = run_lengths(keys)
        what = (n, mean_run, bits)
        # scan
        ref = oracle.seg_scan_by_key_f64(keys, x)
        got = to_host(tcu.seg_scan_by_key(kd, xd)).view(np.float16).astype(np.float64)
        bad = np.abs(got - ref) > allow_for(ref, np.repeat(lens, lens))
        assert not bad.any(), (what, int(bad.sum()), int(np.flatnonzero(bad)[0]))
        wg = oracle.seg_scan_by_key_f64(keys, g)
        exact = np.abs(wg).max() < 2048  # every partial sum is a multiple of 2^-11 below 2^11: exact in fp32 and fp16-representable? only compare when so
        buf = gd.clone()
        tcu.seg_scan_by_key(kd, buf, out=buf)  # in place
        if exact and np.array_equal(wg.astype(np.float16).astype(np.float64), wg):
            assert np.array_equal(to_host(buf), wg.astype(np.float16).view(np.uint16)), what
        # reduction: the four launches that wait for nothing (one and four waves per block), then the one-pass look-back kernel
        want_keys, ref_sums = oracle.seg_reduce_by_key_f64(keys, x)
        _, wsum = oracle.seg_reduce_by_key_f64(keys, g)
        try:
            for chain, waves in ((0, 0), (0, 4), (1, 0)):
                tcu.set_option("by_key_reduce_chain", chain)
                tcu.set_option("by_key_waves", waves)
                what = (n, mean_run, bits, chain, waves)
                keys_out, sums, num = tcu.seg_reduce_by_key(kd, xd)
                r = int(num.item())
                assert r == want_keys.size == starts.size, what
                assert np.array_equal(keys_out[:r].cpu().numpy(), want_keys.astype(kt)), what
                gs = to_host(sums)[:r].view(np.float16).astype(np.float64)
                bad = np.abs(gs - ref_sums) > allow_for(ref_sums, lens)
                assert not bad.any(), (what, int(bad.sum()))
                if not chain:  # sums added in index order at every level: the same bits every time
                    _, again, _ = tcu.seg_reduce_by_key(kd, xd)
                    assert np.array_equal(to_host(again)[:r], to_host(sums)[:r]), what
                if np.abs(wg).max() < 2048:  # exact fp32 partial sums in any order: one rounding, fixed bit for bit
                    _, gsum, _ = tcu.seg_reduce_by_key(kd, gd)
                    assert np.array_equal(to_host(gsum)[:r], wsum.astype(np.float16).view(np.uint16)), what
        finally:
            tcu.set_option("by_key_reduce_chain", 0)
            tcu.set_option("by_key_waves", 0)


def test_by_key_equals_the_fixed_size_kernels_at_full_size(tcu, oracle):
    """2^28 elements, keys = index // S: on exact-grid inputs the by-key results must equal tcu_seg_scan_f16 /
    tcu_seg_reduce_f16 bit for bit (both are then the one correctly rounded value); checked for 32-bit keys at
    S = 16, 1000 (not a power of two: the fixed-size side runs on the first multiple) and 2^20."""
    import torch

    n = 1 << 28
    g = tcu.generate(n, 77, tcu.Dist.GRID)
    idx = torch.arange(n, dtype=torch.int64, device="cuda")
    for seg in (16, 1000, 1 << 20):
        keys = (idx // seg).to(torch.int32)
        nseg = n // seg
        m = nseg * seg
        got = tcu.seg_scan_by_key(keys, g)
        want = tcu.seg_scan(g[:m], seg)
        assert torch.equal(got[:m].view(torch.int16), want.view(torch.int16)), seg
        keys_out, sums, num = tcu.seg_reduce_by_key(keys, g)
        r = int(num.item())
        assert r == (n + seg - 1) // seg
        assert torch.equal(sums[:nseg].view(torch.int16), tcu.seg_reduce(g[:m], seg).view(torch.int16)), seg
        assert torch.equal(keys_out[:r], torch.arange(r, dtype=torch.int32, device="cuda"))
        del keys, got, want, keys_out, sums
    # the whole array as one run: the full-array results within the tolerance at n = 2^28 of a +-1/2048 grid stay exact
    keys = torch.zeros(n, dtype=torch.int32, device="cuda")
    _, sums, num = tcu.seg_reduce_by_key(keys, g)
    assert int(num.item()) == 1
    assert torch.equal(sums[:1].view(torch.int16), tcu.full_reduce(g).view(torch.int16))


def test_by_key_at_the_largest_size(tcu, oracle):
    """n = 2^32 - 24, the most the by-key entry points take (runs are counted in 32 bits): 32-bit keys = index / 4099
    (runs that start anywhere in a partition), exact-grid values; the scan against the fixed-size kernel wherever runs
    and segments coincide is not available at this run length, so both results are checked through properties that do
    not depend on the size: the reduction's sums equal the scan's value at every run's last element, the number of runs
    and their keys are what the keys say, and a sample of runs is summed again with torch in fp64."""
    import torch

    free = torch.cuda.mem_get_info()[0]
    if free < 80 << 30:
        pytest.skip("needs 80 GiB of free device memory")
    n, seg = (1 << 32) - 24, 4099
    g = tcu.generate(n, 78, tcu.Dist.GRID)
    keys = torch.empty(n, dtype=torch.int32, device="cuda")
    step = 1 << 28
    for lo in range(0, n, step):  # keys = index / seg without a 32 GiB index array
        hi = min(n, lo + step)
        keys[lo:hi] = (torch.arange(lo, hi, dtype=torch.int64, device="cuda") // seg).to(torch.int32)
    runs = (n + seg - 1) // seg
    keys_out, sums, num = tcu.seg_reduce_by_key(keys, g)
    assert int(num.item()) == runs
    assert torch.equal(keys_out[:runs], torch.arange(runs, dtype=torch.int32, device="cuda"))
    scan = tcu.seg_scan_by_key(keys, g)
    last = torch.arange(1, runs + 1, dtype=torch.int64, device="cuda") * seg - 1
    last[-1] = n - 1
    assert torch.equal(sums[:runs].view(torch.int16), scan[last].view(torch.int16))
    for r in (0, 1, 65535, 65536, runs // 2, runs - 2, runs - 1):  # around partition and group boundaries, and both ends
        lo, hi = r * seg, min(n, (r + 1) * seg)
        want = g[lo:hi].double().sum().half()  # |sum| < 4099 / 2048: exact in fp64, one rounding
        assert sums[r].view(torch.int16) == want.view(torch.int16), r
        inside = g[lo:hi].double().cumsum(0).half()
        assert torch.equal(scan[lo:hi].view(torch.int16), inside.view(torch.int16)), r


def test_by_key_arguments_and_expired_waits(tcu, oracle):
    import ctypes

    import torch

    from tcu_scope_amd import binding

    x = to_dev(oracle.generate_f16(4096, 1, oracle.DIST_UNIFORM))
    k32 = torch.zeros(4096, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        tcu.seg_scan_by_key(k32[:100], x)
    with pytest.raises(ValueError):
        tcu.seg_scan_by_key(k32.to(torch.int16), x)
    L = binding.lib()
    ws = torch.empty(4096, dtype=torch.uint8, device="cuda")
    have = ctypes.c_size_t(4096)
    assert L.tcu_seg_scan_by_key_f16(k32.data_ptr(), x.data_ptr(), x.data_ptr(), 4096, 16, ws.data_ptr(), ctypes.byref(have), None) == 1
    have = ctypes.c_size_t(8)
    assert L.tcu_seg_scan_by_key_f16(k32.data_ptr(), x.data_ptr(), x.data_ptr(), 4096, 32, ws.data_ptr(), ctypes.byref(have), None) == 4
    have = ctypes.c_size_t(4096)
    assert L.tcu_seg_scan_by_key_f16(k32.data_ptr() + 4, x.data_ptr(), x.data_ptr(), 4000, 32, ws.data_ptr(), ctypes.byref(have), None) == 1  # alignment
    # empty input
    ko, s, num = tcu.seg_reduce_by_key(k32[:0], x[:0])
    assert int(num.item()) == 0
    assert tcu.seg_scan_by_key(k32[:0], x[:0]).numel() == 0

    # a silent partition (forced from the host) with a tiny poll limit: only what depends on it may be NaN, and the
    # reduction must say that it does not know the number of runs rather than return a wrong one
    n = 8 * PART
    rng = np.random.default_rng(8)
    keys = keys_with_runs(rng, n, 5000, False).astype(np.int32)
    xh = oracle.generate_f16(n, 2, oracle.DIST_UNIFORM)
    kd, xd = torch.from_numpy(keys).cuda(), to_dev(xh)
    ref = oracle.seg_scan_by_key_f64(keys, xh)
    starts, lens = run_lengths(keys)
    mute = 3  # partition index 2
    try:
        tcu.set_option("lookback_poll_limit", 16)
        tcu.set_option("test_mute_partition", mute)
        got = to_host(tcu.seg_scan_by_key(kd, xd)).view(np.float16).astype(np.float64)
        first_head_after = starts[starts >= mute * PART][0]
        affected = np.zeros(n, bool)
        affected[mute * PART:first_head_after] = True  # the run that crosses out of the silent partition
        assert np.isnan(got[affected]).all()
        ok = ~affected
        bad = np.abs(got[ok] - ref[ok]) > allow_for(ref[ok], np.repeat(lens, lens)[ok])
        assert not bad.any()
        # the reduction's default form waits for nothing, so a silent partition means nothing to it
        keys_out, sums, num = tcu.seg_reduce_by_key(kd, xd)
        want_keys, ref_sums = oracle.seg_reduce_by_key_f64(keys, xh)
        assert int(num.item()) == want_keys.size
        assert not (np.abs(to_host(sums)[:want_keys.size].view(np.float16).astype(np.float64) - ref_sums) > allow_for(ref_sums, lens)).any()
        tcu.set_option("by_key_reduce_chain", 1)  # its one-pass look-back form
        keys_out, sums, num = tcu.seg_reduce_by_key(kd, xd)
        assert int(num.item()) == -1  # all ones: unknown
        done = int((starts < mute * PART).sum()) - 1  # runs closed by the partitions that could still count
        want_keys, ref_sums = oracle.seg_reduce_by_key_f64(keys, xh)
        gs = to_host(sums)[:done].view(np.float16).astype(np.float64)
        assert not (np.abs(gs - ref_sums[:done]) > allow_for(ref_sums[:done], lens[:done])).any()
        assert np.array_equal(keys_out[:done].cpu().numpy(), want_keys[:done].astype(np.int32))
    finally:
        tcu.set_option("test_mute_partition", 0)
        tcu.set_option("lookback_poll_limit", -1)
        tcu.set_option("by_key_reduce_chain", 0)
    got = to_host(tcu.seg_scan_by_key(kd, xd)).view(np.float16).astype(np.float64)
    assert not (np.abs(got - ref) > allow_for(ref, np.repeat(lens, lens))).any()
