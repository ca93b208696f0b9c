"""Pins the oracle's reduction / prefix-sum functions.

Sources of truth used here, none of which restates the oracle's own loops:
  * numpy's float32 cumsum (strictly sequential accumulation) for the reference CPU path,
  * math.fsum (exactly rounded) and numpy float64 cumsum for the fp64 definition,
  * the reference's constant-0.001 input fixture in closed form, within the tolerances
    the reference's own (disabled) checks use: 0.1 reduce, 0.01 scan, 0.001 CUB/Thrust
    (reference src/reduction/seg_wmma_16.cu:89, src/prefixsum/seg_wmma_16.cu:91,
    src/reduction/seg_cub_block.cu:97-127),
  * inputs on the k/2048 grid, whose partial sums are exact in fp32 and fp64,
  * structural identities (one-hot -> step, zeros -> zeros, scan's last == reduce).
"""
import math

import numpy as np
import pytest

SEGS = [16, 32, 256, 1024, 2048, 16384]
C = 0.00100040435791015625  # fp16(0.001f), the reference's fill value


def as_f(x16, dt):
    return x16.view(np.float16).astype(dt)


@pytest.mark.parametrize("seg", SEGS)
def test_ref_path_matches_numpy_float32_sequential(oracle, seg):
    n = 1 << 17
    nseg = n // seg
    x = oracle.generate_f16(n, 3, oracle.DIST_UNIFORM)
    cs = np.cumsum(as_f(x, np.float32).reshape(nseg, seg), axis=1, dtype=np.float32)
    assert np.array_equal(oracle.seg_scan_ref(x, nseg, seg), cs.astype(np.float16).view(np.uint16).ravel())
    assert np.array_equal(oracle.seg_reduce_ref(x, nseg, seg), cs[:, -1].astype(np.float16).view(np.uint16))
    # threaded split gives the same bits
    assert np.array_equal(oracle.seg_reduce_ref(x, nseg, seg, nthreads=5), oracle.seg_reduce_ref(x, nseg, seg))
    assert np.array_equal(oracle.seg_scan_ref(x, nseg, seg, nthreads=3), oracle.seg_scan_ref(x, nseg, seg))


def test_config1_cpu_reference_case(oracle):
    # N = 2^20, seed 0, segments of 16: the CPU-runnable configuration
    n, seg = 1 << 20, 16
    x = oracle.generate_f16(n, 0, oracle.DIST_UNIFORM)
    out = oracle.seg_reduce_ref(x, n // seg, seg)
    cs = np.cumsum(as_f(x, np.float32).reshape(-1, seg), axis=1, dtype=np.float32)[:, -1]
    assert np.array_equal(out, cs.astype(np.float16).view(np.uint16))
    # and it satisfies the tolerance rule against the fp64 definition
    bad, worst, _ = oracle.check_f16(out, oracle.seg_reduce_f64(x, n // seg, seg), seg)
    assert bad == 0 and worst < 0


def test_full_ref_matches_numpy(oracle):
    n = 50000
    x = oracle.generate_f16(n, 5, oracle.DIST_UNIFORM)
    cs = np.cumsum(as_f(x, np.float32), dtype=np.float32)
    assert np.array_equal(oracle.full_scan_ref(x), cs.astype(np.float16).view(np.uint16))
    assert oracle.full_reduce_ref(x)[0] == cs[-1:].astype(np.float16).view(np.uint16)[0]


@pytest.mark.parametrize("seg", SEGS)
def test_f64_definition_matches_fsum_and_numpy(oracle, seg):
    n = 1 << 16
    nseg = n // seg
    x = oracle.generate_f16(n, 9, oracle.DIST_UNIFORM)
    xd = as_f(x, np.float64).reshape(nseg, seg)
    red = oracle.seg_reduce_f64(x, nseg, seg)
    exact = np.array([math.fsum(row) for row in xd])
    # fp16 values are multiples of 2^-24 below 1 in magnitude: fp64 sums of <= 2^14 of
    # them are exact, so the sequential fp64 sum must equal the exactly rounded sum
    assert np.array_equal(red, exact)
    sc = oracle.seg_scan_f64(x, nseg, seg)
    assert np.array_equal(sc.reshape(nseg, seg), np.cumsum(xd, axis=1))
    assert np.array_equal(sc.reshape(nseg, seg)[:, -1], red)


@pytest.mark.parametrize("seg", SEGS)
def test_reference_fixture_closed_form(oracle, seg):
    nseg = 8
    x = oracle.fill_f16(nseg * seg, 0.001)
    red64 = oracle.seg_reduce_f64(x, nseg, seg)
    assert np.array_equal(red64, np.full(nseg, seg * C))  # exact in fp64
    sc64 = oracle.seg_scan_f64(x, nseg, seg).reshape(nseg, seg)
    assert np.array_equal(sc64, np.tile((np.arange(seg) + 1) * C, (nseg, 1)))
    red = as_f(oracle.seg_reduce_ref(x, nseg, seg), np.float64)
    sc = as_f(oracle.seg_scan_ref(x, nseg, seg), np.float64).reshape(nseg, seg)
    assert np.all(np.abs(red - seg * C) <= 0.001 * max(1.0, seg * C))  # CUB/Thrust tolerance (relative above 1)
    assert np.all(np.abs(red - seg * C) <= 0.1)                       # WMMA reduce tolerance
    assert np.all(np.abs(sc - (np.arange(seg) + 1) * C) <= 0.01)       # WMMA scan tolerance


@pytest.mark.parametrize("seg", [16, 256, 4096, 8192])
def test_exact_grid_inputs_are_bitwise_determined(oracle, seg):
    # k/2048 inputs: every partial sum is a multiple of 2^-11 below 2^13, exact in fp32,
    # so the fp32 path and the fp64 definition must agree bit for bit after one rounding
    n = 1 << 16
    nseg = n // seg
    x = oracle.generate_f16(n, 21, oracle.DIST_GRID)
    sc64 = oracle.seg_scan_f64(x, nseg, seg)
    want = sc64.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.seg_scan_ref(x, nseg, seg), want)
    assert np.array_equal(oracle.seg_reduce_ref(x, nseg, seg), want.reshape(nseg, seg)[:, -1])
    assert all(oracle.f64_to_f16(v) == w for v, w in zip(sc64[:2000].tolist(), want[:2000].tolist()))


def test_structural_identities(oracle):
    seg, nseg = 64, 32
    z = np.zeros(seg * nseg, dtype=np.uint16)
    assert not oracle.seg_reduce_ref(z, nseg, seg).any() and not oracle.seg_scan_ref(z, nseg, seg).any()
    one_hot = z.copy()
    one_hot[5 * seg + 17] = 0x3C00  # 1.0 in segment 5, position 17
    sc = as_f(oracle.seg_scan_ref(one_hot, nseg, seg), np.float32).reshape(nseg, seg)
    want = np.zeros((nseg, seg), np.float32)
    want[5, 17:] = 1.0
    assert np.array_equal(sc, want)
    red = as_f(oracle.seg_reduce_ref(one_hot, nseg, seg), np.float32)
    assert red[5] == 1.0 and red.sum() == 1.0
    # a change in one segment leaves all others bit-identical
    x = oracle.generate_f16(seg * nseg, 2, oracle.DIST_UNIFORM)
    y = x.copy()
    y[7 * seg + 3] ^= 0x0100
    a, b = oracle.seg_scan_ref(x, nseg, seg).reshape(nseg, seg), oracle.seg_scan_ref(y, nseg, seg).reshape(nseg, seg)
    assert np.array_equal(np.delete(a, 7, 0), np.delete(b, 7, 0)) and not np.array_equal(a[7], b[7])
    # zero segments / zero-length is a no-op
    assert oracle.seg_reduce_ref(x, 0, seg).size == 0 and oracle.seg_scan_ref(x, 0, seg).size == 0


def test_add_partial_sums(oracle):
    seg, nseg = 32, 9
    out = oracle.generate_f16(seg * nseg, 4, oracle.DIST_UNIFORM)
    ps = oracle.generate_f16(nseg, 6, oracle.DIST_UNIFORM)
    got = oracle.add_partial_sums_ref(out, ps, nseg, seg)
    want = (as_f(out, np.float32).reshape(nseg, seg) + as_f(ps, np.float32)[:, None]).astype(np.float16)
    assert np.array_equal(got, want.view(np.uint16).ravel())


def test_tolerance_rule(oracle):
    ref = np.array([1.0, 1.0, 1.0, 100.0, 70000.0, 70000.0, -70000.0, 65400.0, 0.0])
    f = lambda v: np.array([v], np.float16).view(np.uint16)[0]
    got = np.array([f(1.0), f(1.0 + 2 * 2 ** -10), f(1.0 + 4 * 2 ** -10), f(100.0), 0x7C00, f(65504.0), 0xFC00, 0x7C00, 0x7E00], np.uint16)
    bad, worst, first = oracle.check_f16(got, ref, 1, ulps=2.0, abs_per_sqrt=0.0)
    # violations: +4ulp, finite where inf is due, inf where 65400 is due, NaN
    assert bad == 4 and first == 2 and worst == float("inf")
    # the sqrt(segment) slack admits the 4-ulp error
    bad, _, _ = oracle.check_f16(got[:4], ref[:4], 16, ulps=2.0, abs_per_sqrt=1e-3)
    assert bad == 0
    bad, _, fb = oracle.check_f32_rel(np.float32([1.0, 2.0, 0.0]), np.array([1.005, 2.5, 1e-9]), 1e-2, 1.0)
    assert bad == 1 and fb == 1


def test_gemv_gemm_f64_against_numpy(oracle):
    M, N, K = 48, 40, 96
    A = oracle.generate_f16(M * K, 1, oracle.DIST_NORMAL)
    B = oracle.generate_f16(N * K, 2, oracle.DIST_NORMAL)  # N rows of K: column-major K x N
    x = oracle.generate_f16(K, 3, oracle.DIST_NORMAL)
    Ad, Bd, xd = as_f(A, np.float64).reshape(M, K), as_f(B, np.float64).reshape(N, K), as_f(x, np.float64)
    y0 = np.linspace(-1, 1, M).astype(np.float32)
    np.testing.assert_allclose(oracle.gemv_f64(A, x, M, K), Ad @ xd, rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(oracle.gemv_f64(A, x, M, K, 1.5, -0.5, y0), 1.5 * (Ad @ xd) - 0.5 * y0.astype(np.float64), rtol=1e-13, atol=1e-13)
    Cm = np.arange(M * N, dtype=np.float32).reshape(M, N) / 7
    np.testing.assert_allclose(oracle.gemm_f64(A, B, M, N, K), Ad @ Bd.T, rtol=1e-13, atol=1e-12)
    np.testing.assert_allclose(oracle.gemm_f64(A, B, M, N, K, 1.1, 1.2, Cm, row0=8, rows=16), (1.1 * (Ad @ Bd.T) + 1.2 * Cm.astype(np.float64))[8:24], rtol=1e-13, atol=1e-12)
    # integer-valued inputs (the reference's rand()%3 fill, src/gemm/wmma.cu:110-127): exact
    Ai = oracle.generate_f16(M * K, 5, oracle.DIST_SMALLINT)
    Bi = oracle.generate_f16(N * K, 6, oracle.DIST_SMALLINT)
    want = as_f(Ai, np.int64).reshape(M, K) @ as_f(Bi, np.int64).reshape(N, K).T
    assert np.array_equal(oracle.gemm_f64(Ai, Bi, M, N, K), want.astype(np.float64))
    # a transposed B operand would fail this: B is not symmetric in shape (N != K)


def test_offsets_reduction_against_numpy_and_the_fixed_size_oracle(oracle):
    """Segments given by begin/end offsets: numpy slices summed in float64 / sequentially in float32,
    the fixed-size functions on uniform offsets, empty and inverted segments, overlapping segments."""
    rng = np.random.default_rng(3)
    n = 20000
    x = oracle.generate_f16(n, 4, oracle.DIST_UNIFORM)
    xf = x.view(np.float16)
    begin = rng.integers(0, n, 400)
    end = np.minimum(begin + rng.integers(0, 700, 400), n)
    end[::17] = begin[::17] - 1  # inverted = empty
    got64 = oracle.seg_reduce_offsets_f64(x, begin, end)
    got16 = oracle.seg_reduce_offsets_ref(x, begin, end)
    for j in range(400):
        sl = xf[begin[j]:max(end[j], begin[j])]
        assert abs(got64[j] - math.fsum(float(v) for v in sl)) <= 1e-9
        acc = np.float32(0)
        for v in sl:
            acc = np.float32(acc + np.float32(v))
        assert got16[j] == np.float16(acc).view(np.uint16)
    seg, nseg = 125, 160
    b = np.arange(nseg) * seg
    assert np.array_equal(oracle.seg_reduce_offsets_f64(x, b, b + seg), oracle.seg_reduce_f64(x, nseg, seg))
    assert np.array_equal(oracle.seg_reduce_offsets_ref(x, b, b + seg), oracle.seg_reduce_ref(x, nseg, seg))
    # overlapping segments are independent: [0, 100) and [50, 150) share elements
    o = oracle.seg_reduce_offsets_f64(x, np.array([0, 50, 0]), np.array([100, 150, 150]))
    assert abs(o[2] - (o[0] + o[1] - oracle.seg_reduce_offsets_f64(x, np.array([50]), np.array([100]))[0])) <= 1e-9


def test_offsets_scan_against_numpy_and_the_fixed_size_oracle(oracle):
    """Prefix sums inside segments given by offsets: numpy cumsum of every slice (float64, and sequential float32
    rounded to fp16), the fixed-size functions on uniform offsets, untouched positions outside every segment,
    last prefix of a segment == its reduction."""
    rng = np.random.default_rng(5)
    n = 30000
    x = oracle.generate_f16(n, 6, oracle.DIST_UNIFORM)
    xf = x.view(np.float16)
    # disjoint ragged segments with gaps, some empty
    cuts = np.sort(rng.choice(n, 600, replace=False))
    begin, end = cuts[0::2].copy(), cuts[1::2].copy()
    end[::13] = begin[::13]
    got64 = oracle.seg_scan_offsets_f64(x, begin, end)
    got16 = oracle.seg_scan_offsets_ref(x, begin, end, fill=0xFFFF)
    covered = np.zeros(n, bool)
    for b, e in zip(begin, end):
        if e <= b:
            continue
        covered[b:e] = True
        assert np.allclose(got64[b:e], np.cumsum(xf[b:e].astype(np.float64)), rtol=0, atol=1e-9)
        acc, want = np.float32(0), []
        for v in xf[b:e]:
            acc = np.float32(acc + np.float32(v))
            want.append(np.float16(acc))
        assert np.array_equal(got16[b:e], np.array(want, np.float16).view(np.uint16))
    assert np.all(np.isnan(got64[~covered])) and np.all(got16[~covered] == 0xFFFF)
    live = end > begin
    assert np.allclose(got64[end[live] - 1], oracle.seg_reduce_offsets_f64(x, begin, end)[live], rtol=0, atol=1e-9)
    seg, nseg = 75, 400
    b = np.arange(nseg) * seg
    assert np.array_equal(oracle.seg_scan_offsets_f64(x, b, b + seg)[:nseg * seg], oracle.seg_scan_f64(x, nseg, seg))
    assert np.array_equal(oracle.seg_scan_offsets_ref(x, b, b + seg)[:nseg * seg], oracle.seg_scan_ref(x, nseg, seg))


def test_by_key_against_numpy_and_the_offsets_oracle(oracle):
    """Segments as runs of equal consecutive keys, pinned by: numpy's run boundaries (np.flatnonzero of key changes)
    with np.add.reduceat / per-run cumsum in float64, a sequential float32 loop for the fp16 path, the offsets
    functions on the same boundaries, a key that comes back later (two runs, not one), and the two extremes
    (all keys equal = full-array result, all keys distinct = identity)."""
    rng = np.random.default_rng(11)
    n = 25000
    x = oracle.generate_f16(n, 9, oracle.DIST_UNIFORM)
    xf = x.view(np.float16)
    lengths = rng.integers(1, 300, 400)
    lengths = lengths[np.cumsum(lengths) <= n]
    lengths[-1] += n - lengths.sum()
    run_key = rng.integers(-5, 5, lengths.size) * (1 << 33)
    for i in range(1, run_key.size):  # neighbours differ, repeats further apart stay
        if run_key[i] == run_key[i - 1]:
            run_key[i] += 1
    keys = np.repeat(run_key, lengths)
    starts = np.flatnonzero(np.r_[True, keys[1:] != keys[:-1]])
    assert np.array_equal(starts, np.r_[0, np.cumsum(lengths)[:-1]])
    ends = np.r_[starts[1:], n]

    ko, sums = oracle.seg_reduce_by_key_f64(keys, x)
    assert np.array_equal(ko, run_key)
    np.testing.assert_allclose(sums, np.add.reduceat(xf.astype(np.float64), starts), rtol=0, atol=1e-9)
    assert np.array_equal(sums, oracle.seg_reduce_offsets_f64(x, starts, ends))
    ko16, sums16 = oracle.seg_reduce_by_key_ref(keys, x)
    assert np.array_equal(ko16, run_key) and np.array_equal(sums16, oracle.seg_reduce_offsets_ref(x, starts, ends))

    sc = oracle.seg_scan_by_key_f64(keys, x)
    sc16 = oracle.seg_scan_by_key_ref(keys, x)
    for b, e in zip(starts[:60], ends[:60]):
        assert np.allclose(sc[b:e], np.cumsum(xf[b:e].astype(np.float64)), rtol=0, atol=1e-9)
        acc, want = np.float32(0), []
        for v in xf[b:e]:
            acc = np.float32(acc + np.float32(v))
            want.append(np.float16(acc))
        assert np.array_equal(sc16[b:e], np.array(want, np.float16).view(np.uint16))
    assert np.array_equal(sc, oracle.seg_scan_offsets_f64(x, starts, ends))
    assert np.array_equal(sc16, oracle.seg_scan_offsets_ref(x, starts, ends))
    assert np.array_equal(sc[ends - 1], sums)

    same = np.zeros(n, np.int64)
    assert np.array_equal(oracle.seg_scan_by_key_f64(same, x), oracle.seg_scan_f64(x, 1, n))
    k1, s1 = oracle.seg_reduce_by_key_f64(same, x)
    assert k1.tolist() == [0] and s1[0] == oracle.seg_reduce_f64(x, 1, n)[0]
    distinct = np.arange(n)[::-1].copy()
    assert np.array_equal(oracle.seg_scan_by_key_ref(distinct, x), x)
    k2, s2 = oracle.seg_reduce_by_key_ref(distinct, x)
    assert np.array_equal(k2, distinct) and np.array_equal(s2, x)
    k3, s3 = oracle.seg_reduce_by_key_f64(np.array([], np.int64), np.array([], np.uint16))
    assert k3.size == 0 and s3.size == 0
