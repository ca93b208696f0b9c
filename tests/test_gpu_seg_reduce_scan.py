"""GPU parity of the segmented reduction and inclusive prefix sum against the CPU oracle,
through the C ABI.  Tolerance: |out - fp64 sum| <= 2 ulp_fp16(result) + 1e-3*sqrt(segment size);
inputs on the k/2048 grid must match bit for bit (their fp32 partial sums are exact)."""
import numpy as np
import pytest

from gpu_common import expect_ok, to_dev, to_host

pytestmark = pytest.mark.gpu

SEGS = [16, 32, 64, 128, 256, 512, 1024, 2048, 4096, 16384]


@pytest.fixture(scope="module")
def tcu():
    import tcu_scope_amd as t

    t.init(0)
    return t


def variants_for(tcu, seg):
    V = tcu.Variant
    # the block families take every size the reference registers them at (16 ... for *_16N_BLOCK and cub::Block*,
    # 256 ... for *_256N_BLOCK); below 512 halves they are launch shapes of the wave kernels
    out = [V.AUTO, V.WAVE_SHUFFLE, V.MFMA_16N, V.BLOCK_LDS, V.MFMA_16N_BLOCK]
    if seg == 16:
        out.append(V.MFMA_16)
    if seg == 256:
        out.append(V.MFMA_256)
    if seg >= 256:
        out += [V.MFMA_256N, V.MFMA_256N_BLOCK]
    return out


@pytest.mark.parametrize("seg", SEGS)
def test_seg_reduce_uniform_all_variants(tcu, oracle, seg):
    n = 1 << 21
    nseg = n // seg
    x = oracle.generate_f16(n, 1, oracle.DIST_UNIFORM)
    ref = oracle.seg_reduce_f64(x, nseg, seg)
    xd = to_dev(x)
    for v in variants_for(tcu, seg):
        for u, w in [(0, 0), (1, 1), (2, 8), (4, 2), (8, 16)]:
            got = to_host(tcu.seg_reduce(xd, seg, variant=v, tiles_per_wave=u, waves_per_block=w))
            expect_ok(oracle, got, ref, seg, f"seg_reduce seg={seg} {v.name} u={u} w={w}")


@pytest.mark.parametrize("seg", SEGS)
def test_seg_scan_uniform_all_variants(tcu, oracle, seg):
    import torch

    n = 1 << 21
    nseg = n // seg
    x = oracle.generate_f16(n, 2, oracle.DIST_UNIFORM)
    ref = oracle.seg_scan_f64(x, nseg, seg)
    ref_tot = ref.reshape(nseg, seg)[:, -1]
    xd = to_dev(x)
    for v in variants_for(tcu, seg):
        for u, w in [(0, 0), (1, 1), (2, 8), (4, 2), (8, 16)]:
            tot = torch.zeros(nseg, dtype=torch.float16, device="cuda")
            got = to_host(tcu.seg_scan(xd, seg, variant=v, tiles_per_wave=u, waves_per_block=w, totals=tot))
            expect_ok(oracle, got, ref, seg, f"seg_scan seg={seg} {v.name} u={u} w={w}")
            expect_ok(oracle, to_host(tot), ref_tot, seg, f"seg_scan totals seg={seg} {v.name} u={u} w={w}")


@pytest.mark.parametrize("seg", [16, 256, 1024, 8192])
def test_exact_grid_inputs_bitwise(tcu, oracle, seg):
    n = 1 << 20
    nseg = n // seg
    x = oracle.generate_f16(n, 21, oracle.DIST_GRID)
    sc = oracle.seg_scan_f64(x, nseg, seg)
    want_scan = sc.astype(np.float16).view(np.uint16)
    want_red = want_scan.reshape(nseg, seg)[:, -1]
    assert np.array_equal(want_red, oracle.seg_reduce_ref(x, nseg, seg))  # the reference CPU path agrees bit for bit here
    xd = to_dev(x)
    for v in variants_for(tcu, seg):
        assert np.array_equal(to_host(tcu.seg_reduce(xd, seg, variant=v)), want_red), f"reduce {v.name}"
        assert np.array_equal(to_host(tcu.seg_scan(xd, seg, variant=v)), want_scan), f"scan {v.name}"


def test_cpu_reference_configuration(tcu, oracle):
    """The configuration the reference's CPU path is quoted on: N = 2^20 halves, uniform [-1, 1) from seed 0,
    contiguous segments of 16 (65536 segments), fp32 accumulation, one fp16 result per segment.  Every family that
    takes 16-half segments against the fp64 sums within the stated tolerance, and against the CPU path itself
    (fp32 running sum, one rounding): sums of 16 halves of magnitude below 1 are exact in fp32 in any order, so the
    two must agree bit for bit."""
    n, seg = 1 << 20, 16
    nseg = n // seg
    x = oracle.generate_f16(n, 0, oracle.DIST_UNIFORM)
    ref64 = oracle.seg_reduce_f64(x, nseg, seg)
    cpu_path = oracle.seg_reduce_ref(x, nseg, seg)
    expect_ok(oracle, cpu_path, ref64, seg, "the CPU path itself")
    xd = to_dev(x)
    dev = tcu.generate(n, 0, tcu.Dist.UNIFORM)  # the device generator gives the same input
    assert np.array_equal(to_host(dev), x)
    for v in (tcu.Variant.AUTO, tcu.Variant.MFMA_16, tcu.Variant.MFMA_16N, tcu.Variant.WAVE_SHUFFLE, tcu.Variant.MFMA_16N_BLOCK, tcu.Variant.BLOCK_LDS):
        got = to_host(tcu.seg_reduce(xd, seg, variant=v))
        assert got.size == 65536
        expect_ok(oracle, got, ref64, seg, f"configuration 1 {v.name}")
        assert np.array_equal(got, cpu_path), f"configuration 1 {v.name}: differs from the CPU path"


def test_reference_fixture_constant_fill(tcu, oracle):
    """The reference fills its inputs with (half)0.001f; closed forms seg*c and (i+1)*c."""
    import torch

    c = 0.00100040435791015625
    for seg in (16, 256, 2048):
        n = 1 << 18
        nseg = n // seg
        x = torch.empty(n, dtype=torch.float16, device="cuda")
        tcu.fill(x, 0.001)
        assert np.all(to_host(x) == 0x1419)
        red = to_host(tcu.seg_reduce(x, seg)).view(np.float16).astype(np.float64)
        sc = to_host(tcu.seg_scan(x, seg)).view(np.float16).astype(np.float64).reshape(nseg, seg)
        expect_ok(oracle, to_host(tcu.seg_reduce(x, seg)), np.full(nseg, seg * c), seg, "fixture reduce")
        expect_ok(oracle, to_host(tcu.seg_scan(x, seg)), np.tile((np.arange(seg) + 1) * c, nseg), seg, "fixture scan")
        assert np.all(np.abs(red - seg * c) <= 0.1) and np.all(np.abs(sc - (np.arange(seg) + 1) * c) <= 0.01)  # the reference's own tolerances


def test_results_beyond_fp16_range_become_infinity(tcu, oracle):
    """Sums past 65504 round to +/-inf exactly where the rounded fp64 sum does (the reference's constant-fill
    benchmark silently runs into this from 6.5e7 elements on): every variant, reduce, scan, full reduce and scan."""
    import torch

    seg = 1 << 17
    n = 4 * seg
    for value in (1.0, -1.0):
        x = torch.full((n,), value, dtype=torch.float16, device="cuda")
        want_red = np.full(4, value * seg)
        want_scan = np.tile(value * (np.arange(seg) + 1.0), 4)
        inf_bits = np.float16(value * np.inf).view(np.uint16)
        for v in (tcu.Variant.AUTO, tcu.Variant.WAVE_SHUFFLE, tcu.Variant.MFMA_16N, tcu.Variant.BLOCK_LDS, tcu.Variant.MFMA_256N_BLOCK):
            red = to_host(tcu.seg_reduce(x, seg, variant=v))
            assert np.all(red == inf_bits), (v.name, value)
            sc = to_host(tcu.seg_scan(x, seg, variant=v))
            expect_ok(oracle, sc, want_scan, seg, f"scan into inf {v.name}")
            first_inf = int(np.argmax(sc[:seg] == inf_bits))
            assert first_inf == 65519 and np.all(sc[first_inf:seg] == inf_bits) and np.all(sc[:first_inf] != inf_bits), (v.name, first_inf)  # 65520 is the first sum that rounds to inf
        assert to_host(tcu.full_reduce(x))[0] == inf_bits
        full = to_host(tcu.full_scan(x))
        assert np.all(full[65519:] == inf_bits) and np.all(full[:65519] != inf_bits)
        expect_ok(oracle, to_host(tcu.seg_reduce(x, seg)), want_red, seg, "reduce into inf")


@pytest.mark.parametrize("seg", [16, 256, 2048, 16384])
def test_non_finite_inputs_stay_in_their_segment(tcu, oracle, seg):
    """A NaN or an infinity in one segment reaches that segment's sum and the prefixes from its position on, and nothing
    else (AUTO and the DPP / LDS variants; the MFMA variants multiply by 0/1 matrices, where 0 * inf is NaN, and are
    only required to keep what lies outside the wave's span of at most 8 tiles clean)."""
    import torch

    n = 1 << 20
    nseg = n // seg
    x_host = oracle.generate_f16(n, 31, oracle.DIST_UNIFORM)
    ref_red = oracle.seg_reduce_f64(x_host, nseg, seg)
    ref_scan = oracle.seg_scan_f64(x_host, nseg, seg)
    for bits, name in ((0x7E00, "nan"), (0x7C00, "inf")):
        hit_seg, hit_pos = nseg // 3, seg // 2 + 3
        xh = x_host.copy()
        xh[hit_seg * seg + hit_pos] = bits
        x = to_dev(xh)
        for v in (tcu.Variant.AUTO, tcu.Variant.WAVE_SHUFFLE, tcu.Variant.BLOCK_LDS):
            try:
                red = to_host(tcu.seg_reduce(x, seg, variant=v)).view(np.float16).astype(np.float64)
                sc = to_host(tcu.seg_scan(x, seg, variant=v)).view(np.float16).astype(np.float64).reshape(nseg, seg)
            except tcu.TcuError as e:
                assert e.status == 2
                continue
            bad = (lambda a: np.isnan(a)) if name == "nan" else (lambda a: np.isinf(a) & (a > 0))
            assert bad(red[hit_seg]) and np.all(bad(sc[hit_seg, hit_pos:])), (v.name, name)
            keep = np.ones(nseg, bool)
            keep[hit_seg] = False
            assert np.all(np.isfinite(red[keep])) and np.all(np.isfinite(sc[keep])) and np.all(np.isfinite(sc[hit_seg, :hit_pos])), (v.name, name)
            assert oracle.check_f16(red[keep].astype(np.float16).view(np.uint16), ref_red[keep], seg)[0] == 0
            assert oracle.check_f16(sc[keep].astype(np.float16).view(np.uint16), ref_scan.reshape(nseg, seg)[keep], seg)[0] == 0
        # MFMA flavour: whatever lies outside the 8 tiles (4096 halves) around the value and outside its segment is untouched
        red = to_host(tcu.seg_reduce(x, seg, variant=tcu.Variant.MFMA_16N)).view(np.float16).astype(np.float64)
        sc = to_host(tcu.seg_scan(x, seg, variant=tcu.Variant.MFMA_16N)).view(np.float16).astype(np.float64)
        span = (hit_seg * seg + hit_pos) // 4096
        clean = np.ones(n, bool)
        lo = min(span * 4096, hit_seg * seg)
        hi = max((span + 1) * 4096, (hit_seg + 1) * seg)
        clean[lo:hi] = False
        assert np.all(np.isfinite(sc[clean])), name
        seg_clean = np.ones(nseg, bool)
        seg_clean[lo // seg:(hi + seg - 1) // seg] = False
        assert np.all(np.isfinite(red[seg_clean])), name


def test_ragged_and_edge_cases(tcu, oracle):
    import torch

    V = tcu.Variant
    # tails: segment counts that do not fill a tile / wave / block
    for seg, nseg in [(16, 1), (16, 3), (16, 33), (16, 257), (64, 5), (256, 7), (512, 3), (1024, 5), (2048, 3), (4096, 1)]:
        x = oracle.generate_f16(nseg * seg, 7, oracle.DIST_UNIFORM)
        xd = to_dev(x)
        for v in variants_for(tcu, seg):
            for u in (1, 8):
                out = torch.full((nseg + 64,), 7.0, dtype=torch.float16, device="cuda")  # guard words after the end
                tcu.seg_reduce(xd, seg, variant=v, tiles_per_wave=u, out=out, num_segments=nseg)
                h = to_host(out)
                expect_ok(oracle, h[:nseg], oracle.seg_reduce_f64(x, nseg, seg), seg, f"tail reduce seg={seg} nseg={nseg} {v.name}")
                assert np.all(h[nseg:] == 0x4700), f"reduce wrote past the end: seg={seg} nseg={nseg} {v.name}"
                outs = torch.full((nseg * seg + 512,), 7.0, dtype=torch.float16, device="cuda")
                tcu.seg_scan(xd, seg, variant=v, tiles_per_wave=u, out=outs, num_segments=nseg)
                h = to_host(outs)
                expect_ok(oracle, h[: nseg * seg], oracle.seg_scan_f64(x, nseg, seg), seg, f"tail scan seg={seg} nseg={nseg} {v.name}")
                assert np.all(h[nseg * seg:] == 0x4700), f"scan wrote past the end: seg={seg} nseg={nseg} {v.name}"
    # segment sizes outside the fast kernels (AUTO only)
    for seg, nseg in [(1, 100), (7, 91), (24, 50), (100, 33), (1000, 9)]:
        x = oracle.generate_f16(nseg * seg, 8, oracle.DIST_UNIFORM)
        xd = to_dev(x)
        expect_ok(oracle, to_host(tcu.seg_reduce(xd, seg)), oracle.seg_reduce_f64(x, nseg, seg), seg, f"generic reduce seg={seg}")
        expect_ok(oracle, to_host(tcu.seg_scan(xd, seg)), oracle.seg_scan_f64(x, nseg, seg), seg, f"generic scan seg={seg}")
        with pytest.raises(tcu.TcuError) as e:
            tcu.seg_reduce(xd, seg, variant=V.WAVE_SHUFFLE)
        assert e.value.status == 2
    # empty input is a no-op
    empty = torch.empty(0, dtype=torch.float16, device="cuda")
    assert tcu.seg_reduce(empty, 16).numel() == 0 and tcu.seg_scan(empty, 16).numel() == 0
    # the reference's precondition failures map to "unsupported"
    x = to_dev(oracle.generate_f16(4096, 9, oracle.DIST_UNIFORM))
    for v, seg in [(V.MFMA_16, 32), (V.MFMA_256, 16), (V.MFMA_256N, 128), (V.MFMA_256N_BLOCK, 128), (V.BLOCK_LDS, 24)]:
        with pytest.raises(tcu.TcuError) as e:
            tcu.seg_reduce(x, seg, variant=v)
        assert e.value.status == 2
        with pytest.raises(tcu.TcuError) as e:
            tcu.seg_scan(x, seg, variant=v)
        assert e.value.status == 2
    with pytest.raises(tcu.TcuError) as e:
        tcu.seg_reduce(x, 0)
    assert e.value.status == 1
    with pytest.raises(tcu.TcuError) as e:
        tcu.seg_reduce(x, 16, tiles_per_wave=3)
    assert e.value.status == 1
    with pytest.raises(tcu.TcuError) as e:
        tcu.seg_reduce(x[1:], 16, variant=V.WAVE_SHUFFLE, num_segments=8)  # misaligned
    assert e.value.status == 1
    expect_ok(oracle, to_host(tcu.seg_reduce(x[1:], 16, num_segments=8)), oracle.seg_reduce_f64(to_host(x)[1:129], 8, 16), 16, "misaligned AUTO")


def test_scan_in_place_and_structure(tcu, oracle):
    import torch

    seg, nseg = 2048, 512
    x = oracle.generate_f16(seg * nseg, 11, oracle.DIST_UNIFORM)
    xd = to_dev(x)
    want = to_host(tcu.seg_scan(xd, seg))
    y = xd.clone()
    tcu.seg_scan(y, seg, out=y)
    assert np.array_equal(to_host(y), want), "in-place scan differs"
    # one-hot input gives an exact step, zeros give zeros
    z = torch.zeros(seg * nseg, dtype=torch.float16, device="cuda")
    assert not to_host(tcu.seg_scan(z, seg)).any() and not to_host(tcu.seg_reduce(z, seg)).any()
    z[5 * seg + 1234] = 1.0
    sc = to_host(tcu.seg_scan(z, seg)).view(np.float16).reshape(nseg, seg)
    step = np.zeros((nseg, seg), np.float16)
    step[5, 1234:] = 1.0
    assert np.array_equal(sc, step)
    # changing one segment leaves every other output bit-identical
    x2 = x.copy()
    x2[7 * seg + 3] ^= 0x0100
    a, b = want.reshape(nseg, seg), to_host(tcu.seg_scan(to_dev(x2), seg)).reshape(nseg, seg)
    assert np.array_equal(np.delete(a, 7, 0), np.delete(b, 7, 0)) and not np.array_equal(a[7], b[7])


@pytest.mark.parametrize("seg", [4096, 8192, 16384])
def test_scan_blocks_capped_per_compute_unit(tcu, oracle, seg):
    """AUTO's block scan asks for LDS it never touches, so that a compute unit holds three or four of its blocks
    (option scan_lds_pad, KiB; -1 = AUTO's table).  The request changes how many blocks run side by side and nothing
    else: at 2^27 elements (and a segment count that no block shape divides) the outputs are the same bits with the
    table's cap, without one, with two blocks per unit and with a request beyond what a unit has (clipped), and they
    agree with the oracle; an explicit launch shape takes the option too."""
    nseg = (1 << 27) // seg + 3
    n = nseg * seg
    x = oracle.generate_f16(n, 31, oracle.DIST_UNIFORM)
    xd = to_dev(x)
    got = {}
    try:
        for pad in (-1, 0, 79, 400):
            tcu.set_option("scan_lds_pad", pad)
            got[pad] = to_host(tcu.seg_scan(xd, seg))
        for pad in (39, 0):  # another shape adds a segment's pieces in another order, so it is compared with itself
            tcu.set_option("scan_lds_pad", pad)
            got["explicit", pad] = to_host(tcu.seg_scan(xd, seg, variant=tcu.Variant.BLOCK_LDS, tiles_per_wave=2, waves_per_block=8))
    finally:
        tcu.set_option("scan_lds_pad", -1)
    for key in (0, 79, 400):
        assert np.array_equal(got[-1], got[key]), (seg, key)
    assert np.array_equal(got["explicit", 39], got["explicit", 0]), seg
    w = 1 << 22  # the oracle on the first and on the last stretch
    for first in (0, n - w):
        expect_ok(oracle, got[-1][first:first + w], oracle.seg_scan_f64(x[first:first + w], w // seg, seg), seg, (seg, first))


def test_device_generator_matches_oracle(tcu, oracle):
    n = (1 << 20) + 13
    for dist in (tcu.Dist.UNIFORM, tcu.Dist.GRID, tcu.Dist.SMALLINT):
        got = to_host(tcu.generate(n, 12345, dist, first=99))
        assert np.array_equal(got, oracle.generate_f16(n, 12345, int(dist), first=99)), dist.name
    g = to_host(tcu.generate(1 << 20, 3, tcu.Dist.NORMAL)).view(np.float16).astype(np.float64)
    h = oracle.generate_f16(1 << 20, 3, oracle.DIST_NORMAL).view(np.float16).astype(np.float64)
    assert np.mean(g != h) < 1e-3 and np.max(np.abs(g - h)) <= 2 ** -7  # libm differences move at most a rounding boundary


@pytest.mark.parametrize("seg", [16, 256, 1024, 4096, 16384])
def test_full_size_seg_reduce(tcu, oracle, seg):
    """N = 2^28 (the benchmark configuration): every variant against the oracle."""
    n = 1 << 28
    nseg = n // seg
    xd = tcu.generate(n, 1, tcu.Dist.UNIFORM)
    x = oracle.generate_f16(n, 1, oracle.DIST_UNIFORM)
    ref = oracle.seg_reduce_f64(x, nseg, seg)
    for v in variants_for(tcu, seg):
        expect_ok(oracle, to_host(tcu.seg_reduce(xd, seg, variant=v)), ref, seg, f"2^28 reduce seg={seg} {v.name}")


@pytest.mark.parametrize("seg", [16, 256, 2048, 16384])
def test_full_size_seg_scan(tcu, oracle, seg):
    """N = 2^28: the last element of every scanned segment against the fp64 segment sum,
    adjacent differences against the inputs, a 2^24-element window against the oracle, and
    all variants bit-identical on exact-grid inputs."""
    import torch

    n = 1 << 28
    nseg = n // seg
    xd = tcu.generate(n, 1, tcu.Dist.UNIFORM)
    x = oracle.generate_f16(n, 1, oracle.DIST_UNIFORM)
    red64 = oracle.seg_reduce_f64(x, nseg, seg)
    win = 1 << 24
    for v in variants_for(tcu, seg):
        out = tcu.seg_scan(xd, seg, variant=v)
        last = to_host(out.view(nseg, seg)[:, -1].contiguous())
        expect_ok(oracle, last, red64, seg, f"2^28 scan last element seg={seg} {v.name}")
        for lo in (0, n - win):
            got = to_host(out[lo:lo + win])
            expect_ok(oracle, got, oracle.seg_scan_f64(x[lo:lo + win], win // seg, seg), seg, f"2^28 scan window@{lo} seg={seg} {v.name}")
        # scan[i] - scan[i-1] = x[i] up to the two roundings of the outputs
        o32, x32 = out.float().view(nseg, seg), xd.float().view(nseg, seg)
        d = (o32[:, 1:] - o32[:, :-1] - x32[:, 1:]).abs()
        ulp = torch.maximum(o32[:, 1:].abs(), o32[:, :-1].abs()) * 2.0 ** -10 + 2.0 ** -24
        assert bool((d <= 2 * ulp + 2e-3 * seg ** 0.5).all()), f"difference identity seg={seg} {v.name}"
        del out, o32, x32, d, ulp
    gd = tcu.generate(n, 5, tcu.Dist.GRID)
    base = tcu.seg_scan(gd, seg, variant=tcu.Variant.WAVE_SHUFFLE)
    if seg <= 8192:
        for v in variants_for(tcu, seg):
            assert torch.equal(tcu.seg_scan(gd, seg, variant=v), base), f"grid inputs: {v.name} differs from WAVE_SHUFFLE"


@pytest.mark.parametrize("seg_log2,n_log2", [(17, 24), (19, 24), (17, 26), (20, 24), (21, 24), (24, 24), (28, 28)])
def test_segments_larger_than_a_block_can_walk(tcu, oracle, seg_log2, n_log2):
    """AUTO on segments that are cut into partitions (partition sums / look-back scan restarted at segment starts):
    2^20 (reduce) and 2^21 (scan) halves and more, up to the whole 2^28 array as one segment, and segments from 2^17
    halves on when there are fewer of them than compute units (128 and 32 segments here; 512 segments of 2^17 halves
    stay with the block that walks a segment): uniform inputs within the tolerance, exact-grid inputs bit for bit,
    per-segment totals, repeated calls."""
    import torch

    seg = 1 << seg_log2
    n = 1 << n_log2
    nseg = n // seg
    x = oracle.generate_f16(n, 3, oracle.DIST_UNIFORM)
    xd = to_dev(x)
    ref = oracle.seg_scan_f64(x, nseg, seg)
    for rep in range(2):  # the temporaries come from a pool: the second call reuses them
        expect_ok(oracle, to_host(tcu.seg_reduce(xd, seg)), ref.reshape(nseg, seg)[:, -1], seg, f"reduce seg=2^{seg_log2} call {rep}")
        tot = torch.zeros(nseg, dtype=torch.float16, device="cuda")
        got = to_host(tcu.seg_scan(xd, seg, totals=tot))
        expect_ok(oracle, got, ref, seg, f"scan seg=2^{seg_log2} call {rep}")
        expect_ok(oracle, to_host(tot), ref.reshape(nseg, seg)[:, -1], seg, f"scan totals seg=2^{seg_log2} call {rep}")
    g = oracle.generate_f16(n, 4, oracle.DIST_GRID)
    gd = to_dev(g)
    want64 = oracle.seg_scan_f64(g, nseg, seg)
    if np.abs(want64).max() < 4096:  # fp32 sums of multiples of 1/2048 are exact up to 8192
        want = want64.astype(np.float16).view(np.uint16)
        assert np.array_equal(to_host(tcu.seg_scan(gd, seg)), want)
        assert np.array_equal(to_host(tcu.seg_reduce(gd, seg)), want.reshape(nseg, seg)[:, -1])
    else:
        expect_ok(oracle, to_host(tcu.seg_scan(gd, seg)), want64, seg, f"grid scan seg=2^{seg_log2}")
        expect_ok(oracle, to_host(tcu.seg_reduce(gd, seg)), want64.reshape(nseg, seg)[:, -1], seg, f"grid reduce seg=2^{seg_log2}")


def test_segmented_reduction_over_offsets(tcu, oracle):
    """tcu_seg_reduce_offsets_f16: ragged, empty, inverted and overlapping segments with 32- and 64-bit offsets and
    every lanes-per-segment choice, against the fp64 oracle with the per-segment tolerance 2 ulp + 1e-3*sqrt(length);
    exact-grid inputs bit for bit; uniform offsets must equal tcu_seg_reduce_f16 exactly on such inputs."""
    import torch

    rng = np.random.default_rng(11)
    n = 1 << 22
    x = oracle.generate_f16(n, 8, oracle.DIST_UNIFORM)
    g = oracle.generate_f16(n, 9, oracle.DIST_GRID)
    xd, gd = to_dev(x), to_dev(g)
    for max_len, nseg in ((24, 200000), (700, 50000), (20000, 3000), (1 << 20, 40)):
        begin = rng.integers(0, n, nseg)
        end = np.minimum(begin + rng.integers(0, max_len + 1, nseg), n)
        inv = rng.random(nseg) < 0.03
        end[inv] = begin[inv] - 1
        length = np.maximum(end - begin, 0)
        ref = oracle.seg_reduce_offsets_f64(x, begin, end)
        want_grid = oracle.seg_reduce_offsets_f64(g, begin, end)
        exact = np.abs(want_grid).max() < 4096 and max_len <= 20000
        for dtype in (torch.int32, torch.int64):
            bd, ed = torch.from_numpy(begin).to(dtype).cuda(), torch.from_numpy(end).to(dtype).cuda()
            for expected in (0, 16, 100, 512, 4096, 20000, 1 << 16, 1 << 17, 1 << 20):
                got = to_host(tcu.seg_reduce_offsets(xd, bd, ed, expected_segment_size=expected)).view(np.float16).astype(np.float64)
                allow = 2 * np.maximum(np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64), 2.0 ** -24) + 1e-3 * np.sqrt(length)
                bad = np.abs(got - ref) > allow
                assert not bad.any(), (max_len, str(dtype), expected, int(bad.sum()), int(np.argmax(bad)))
                if exact:
                    gg = to_host(tcu.seg_reduce_offsets(gd, bd, ed, expected_segment_size=expected))
                    assert np.array_equal(gg, want_grid.astype(np.float16).view(np.uint16)), (max_len, str(dtype), expected)
    for seg in (16, 48, 256, 4096):
        nseg = (1 << 20) // seg
        off = (torch.arange(nseg + 1, dtype=torch.int64) * seg).to(torch.int32).cuda()
        got = tcu.seg_reduce_offsets(gd, off[:-1], off[1:], expected_segment_size=seg)
        want = oracle.seg_scan_f64(g, nseg, seg).astype(np.float16).view(np.uint16).reshape(nseg, seg)[:, -1]
        assert np.array_equal(to_host(got), want), seg
    assert tcu.seg_reduce_offsets(xd, off[:0], off[:0]).numel() == 0


def test_segmented_scan_over_offsets(tcu, oracle):
    """tcu_seg_scan_offsets_f16: disjoint ragged segments with gaps and empty segments, 32- and 64-bit offsets, every
    lanes-per-segment choice, against the fp64 oracle (2 ulp + 1e-3*sqrt(segment length)); positions outside every
    segment keep their sentinel; exact-grid inputs bit for bit; uniform offsets equal the fixed-size scan; in place."""
    import torch

    rng = np.random.default_rng(21)
    n = 1 << 22
    x = oracle.generate_f16(n, 12, oracle.DIST_UNIFORM)
    g = oracle.generate_f16(n, 13, oracle.DIST_GRID)
    xd, gd = to_dev(x), to_dev(g)
    for nseg in (150000, 20000, 500, 3):
        cuts = np.sort(rng.choice(n, 2 * nseg, replace=False))
        begin, end = cuts[0::2].astype(np.int64), cuts[1::2].astype(np.int64)
        end[::9] = begin[::9]
        ref = oracle.seg_scan_offsets_f64(x, begin, end)
        inside = ~np.isnan(ref)
        seglen = np.zeros(n)
        for b, e in zip(begin, end):  # tolerance term: sqrt of the length of the segment an element belongs to
            seglen[b:e] = e - b
        wg = oracle.seg_scan_offsets_f64(g, begin, end)
        exact = np.nanmax(np.abs(wg)) < 4096
        for dtype in (torch.int32, torch.int64):
            bd, ed = torch.from_numpy(begin).to(dtype).cuda(), torch.from_numpy(end).to(dtype).cuda()
            # the last two: several blocks per segment; 300000: slices that meet through look-back (slices longer than a
            # block holds when nseg = 3), and once more (-300000) as slice sums + a second read
            for expected in (0, 16, 40, 100, 1500, 5000) + ((1 << 16, 300000, -300000) if nseg <= 500 else ()):
                tcu.set_option("offsets_scan_chain", 0 if expected < 0 else 1)
                expected = abs(expected)
                out = torch.full((n,), -7.0, dtype=torch.float16, device="cuda")
                tcu.seg_scan_offsets(xd, bd, ed, expected_segment_size=expected, out=out)
                got = to_host(out)
                assert np.all(got[~inside] == np.float16(-7.0).view(np.uint16)), "wrote outside the segments"
                gv = got[inside].view(np.float16).astype(np.float64)
                allow = 2 * np.maximum(np.spacing(np.abs(ref[inside]).astype(np.float16)).astype(np.float64), 2.0 ** -24) + 1e-3 * np.sqrt(seglen[inside])
                bad = np.abs(gv - ref[inside]) > allow
                assert not bad.any(), (nseg, str(dtype), expected, int(bad.sum()))
                if exact:
                    og = to_host(tcu.seg_scan_offsets(gd, bd, ed, expected_segment_size=expected))
                    assert np.array_equal(og[inside], wg[inside].astype(np.float16).view(np.uint16)), (nseg, str(dtype), expected)
    for seg in (16, 48, 2048, 1 << 17):
        nseg = (1 << 20) // seg
        off = (torch.arange(nseg + 1, dtype=torch.int64) * seg).to(torch.int32).cuda()
        buf = gd[: nseg * seg].clone()
        tcu.seg_scan_offsets(buf, off[:-1], off[1:], expected_segment_size=seg, out=buf)  # in place
        assert np.array_equal(to_host(buf), oracle.seg_scan_f64(g, nseg, seg).astype(np.float16).view(np.uint16)), seg


def test_offsets_one_segment_beyond_2_to_the_31(tcu, oracle):
    """A segment of 2^31 + 11 halves that starts off a chunk boundary, 64-bit offsets, and a short one behind it: 32769
    slices that meet through look-back.  The values repeat (-3 ... 3) / 2048, so every prefix is one of seven small
    numbers and the whole output is checked against the closed form, chunk by chunk; nothing outside the segments is
    written; the reduction over the same offsets gives the two closed-form sums."""
    import torch

    if torch.cuda.mem_get_info()[0] < 40 << 30:
        pytest.skip("needs 40 GiB of free device memory")
    n = (1 << 31) + 64
    cycle = torch.tensor([-3, -2, -1, 0, 1, 2, 3], dtype=torch.float32, device="cuda") / 2048
    upto = torch.cumsum(cycle, 0)  # sum of the first r + 1 values of a cycle; whole cycles add nothing
    g = torch.empty(n, dtype=torch.float16, device="cuda")
    step = 1 << 28
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        g[lo:hi] = cycle[torch.arange(lo, hi, dtype=torch.int64, device="cuda") % 7].half()
    length = (1 << 31) + 11
    begin = torch.tensor([5, 5 + length + 3], dtype=torch.int64, device="cuda")
    end = torch.tensor([5 + length, n - 1], dtype=torch.int64, device="cuda")
    out = torch.full((n,), -7.0, dtype=torch.float16, device="cuda")
    tcu.seg_scan_offsets(g, begin, end, expected_segment_size=length, out=out)

    def prefix(i, b):  # sum of g[b .. i]
        return upto[i % 7] - (upto[(b - 1) % 7] if (b % 7) else 0.0)

    for lo in range(0, n, step):
        hi = min(n, lo + step)
        i = torch.arange(lo, hi, dtype=torch.int64, device="cuda")
        want = torch.full((hi - lo,), -7.0, dtype=torch.float32, device="cuda")
        for b, e in ((5, 5 + length), (5 + length + 3, n - 1)):
            inside = (i >= b) & (i < e)
            want = torch.where(inside, prefix(i, b), want)
        assert torch.equal(out[lo:hi].view(torch.int16), want.half().view(torch.int16)), lo
    sums = tcu.seg_reduce_offsets(g, begin, end, expected_segment_size=length)
    want = torch.stack([prefix(torch.tensor(int(e) - 1, device="cuda"), int(b)) for b, e in zip(begin.tolist(), end.tolist())]).half()
    assert torch.equal(sums.view(torch.int16), want.view(torch.int16))


def test_temporary_memory_across_streams(tcu, oracle):
    """The paths that take temporary device memory keep the block a stream gave back for that stream's next request:
    twelve streams (more than the library keeps blocks for), growing and shrinking requests on one stream, and calls
    that alternate between streams must all give the results of the default stream."""
    import torch

    seg = 1 << 20
    g = oracle.generate_f16(8 * seg, 31, oracle.DIST_GRID)
    gd = to_dev(g)
    want = {k: oracle.seg_reduce_f64(g[:k * seg], k, seg).astype(np.float16).view(np.uint16) for k in (1, 2, 4, 8)}
    streams = [torch.cuda.Stream() for _ in range(12)]
    torch.cuda.synchronize()
    outs = []
    for rep in range(3):
        for i, st in enumerate(streams):
            k = (1, 4, 2, 8)[(i + rep) % 4]  # the same stream asks for more, then for less
            with torch.cuda.stream(st):
                outs.append((k, tcu.seg_reduce(gd[:k * seg], seg, stream=st)))
    for k in (8, 1, 4):
        outs.append((k, tcu.seg_reduce(gd[:k * seg], seg)))
    torch.cuda.synchronize()
    for k, out in outs:
        assert np.array_equal(to_host(out), want[k]), k


def test_time_next_launch(tcu):
    """tcu_time_next_launch: the events are stamped by the kernel itself, only the next launch carries them, and the
    duration lies between what the bytes need at 8 TB/s and the wall-clock time of the call."""
    import time

    import torch

    n = 1 << 26
    x = tcu.generate(n, 5, tcu.Dist.UNIFORM)
    out = torch.empty_like(x)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    b.record()  # creates the handles
    tcu.seg_scan(x, 256, out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    tcu.time_next_launch(a, b)
    tcu.seg_scan(x, 256, out=out)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms = a.elapsed_time(b)
    assert 4 * n / 8e12 * 1e3 < ms < wall_ms, (ms, wall_ms)
    first = ms
    tcu.seg_scan(x, 256, out=out)  # no events any more: the stamps stay
    torch.cuda.synchronize()
    assert a.elapsed_time(b) == first
