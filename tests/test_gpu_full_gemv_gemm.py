"""GPU parity of the full-array reduction / prefix sum and of GEMV / GEMM."""
import numpy as np
import pytest

from gpu_common import expect_ok, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tcu():
    import tcu_scope_amd as t

    t.init(0)
    return t


@pytest.mark.parametrize("n", [8, 1000, 1003, 1 << 12, (1 << 20) + 8 * 37, 1 << 24])
def test_full_reduce_and_scan(tcu, oracle, n):
    S = tcu.FullStrategy
    x = oracle.generate_f16(n, 4, oracle.DIST_UNIFORM)
    ref = oracle.seg_scan_f64(x, 1, n)
    xd = to_dev(x)
    M = tcu.FULL_MFMA  # flag: the single-pass kernels add and scan on the matrix unit
    for strategy, seg, w in [(S.AUTO, 0, 0), (S.SINGLE_PASS, 2048, 4), (S.SINGLE_PASS, 1024, 1), (S.SINGLE_PASS, 65536, 8), (S.MULTI_KERNEL, 0, 0), (S.MULTI_KERNEL, 256, 2),
                             (S.AUTO | M, 0, 0), (S.SINGLE_PASS | M, 4096, 2), (S.SINGLE_PASS | M, 512, 1), (S.SINGLE_PASS | M, 65536, 16)]:
        try:
            red = to_host(tcu.full_reduce(xd, strategy, seg, w))
            sc = to_host(tcu.full_scan(xd, strategy, seg, w))
        except tcu.TcuError as e:
            assert e.status == 2 and strategy == S.MULTI_KERNEL and n % (seg or 2048) != 0, (strategy, seg, str(e))
            continue
        expect_ok(oracle, red, ref[-1:], n, f"full reduce n={n} strategy={int(strategy):#x} seg={seg}")
        expect_ok(oracle, sc, ref, n, f"full scan n={n} strategy={int(strategy):#x} seg={seg}")
    # AUTO with 4 more tiles per wave parked in LDS, which the library itself only takes up to 2^27 elements
    try:
        tcu.set_option("scan_lds_tiles", 1)
        expect_ok(oracle, to_host(tcu.full_scan(xd)), ref, n, f"full scan n={n} with tiles parked in LDS")
    finally:
        tcu.set_option("scan_lds_tiles", -1)


def test_full_exact_grid_bitwise_and_repeatable(tcu, oracle):
    import torch

    n = 1 << 22  # |prefix| stays far below 8192: every fp32 partial sum is exact
    x = oracle.generate_f16(n, 6, oracle.DIST_GRID)
    ref = oracle.seg_scan_f64(x, 1, n)
    assert np.abs(ref).max() < 8192
    xd = to_dev(x)
    want = ref.astype(np.float16).view(np.uint16)
    assert np.array_equal(to_host(tcu.full_scan(xd)), want)
    assert to_host(tcu.full_reduce(xd))[0] == want[-1]
    # same workspace reused back to back (it needs no initialisation between calls)
    ws = torch.empty(tcu.binding.full_workspace_bytes("scan", n), dtype=torch.uint8, device="cuda")
    ws.fill_(0xAB)
    for _ in range(3):
        assert np.array_equal(to_host(tcu.full_scan(xd, workspace=ws)), want)
    y = to_dev(oracle.generate_f16(n, 7, oracle.DIST_UNIFORM))
    a, b = to_host(tcu.full_reduce(y)), to_host(tcu.full_reduce(y))
    assert a[0] == b[0], "full reduction is deterministic"
    with pytest.raises(tcu.TcuError) as e:
        tcu.full_scan(xd, workspace=torch.empty(256, dtype=torch.uint8, device="cuda"))
    assert e.value.status == 4


def test_full_size_2p30(tcu, oracle):
    """N = 2^30, every single-kernel form beside AUTO: the reduction against the fp64 sum; the scan
    through its element at the end of every 2^26 piece, whole windows at both ends and the
    overflow rule (fp16 saturates to inf only where the fp64 prefix does)."""
    S = tcu.FullStrategy
    n = 1 << 30
    xd = tcu.generate(n, 1, tcu.Dist.UNIFORM)
    # fp64 prefix at the end of every piece, streamed on the host in 2^26 pieces
    piece = 1 << 26
    carry = 0.0
    ends = []
    first_ref = last_ref = None
    for p in range(n // piece):
        xp = oracle.generate_f16(piece, 1, oracle.DIST_UNIFORM, first=p * piece)
        sc = oracle.seg_scan_f64(xp, 1, piece) + carry
        if p == 0:
            first_ref = sc.copy()
        if p == n // piece - 1:
            last_ref = sc.copy()
        carry = sc[-1]
        ends.append(carry)
    ends = np.array(ends)
    out = None
    for strategy in (S.AUTO, S.SINGLE_PASS, S.SINGLE_PASS | tcu.FULL_MFMA):
        what = f"2^30 strategy={int(strategy):#x}"
        red = to_host(tcu.full_reduce(xd, strategy))
        expect_ok(oracle, red, ends[-1:], n, what + " full reduce")
        out = tcu.full_scan(xd, strategy, out=out)
        got_ends = to_host(out[piece - 1::piece].contiguous())
        expect_ok(oracle, got_ends, ends, n, what + " scan at the end of every 2^26 piece")
        expect_ok(oracle, to_host(out[:piece]), first_ref, n, what + " scan first window")
        expect_ok(oracle, to_host(out[n - piece:]), last_ref, n, what + " scan last window")
        out.zero_()


def test_a_wait_that_expires_gives_nan_not_wrong_numbers(tcu, oracle):
    """A block of a single-pass kernel that waits in vain for a value another block should have
    published must not return finite, plausible, wrong data.  The condition is forced from the
    host: one partition is told to publish nothing and the poll limit is made tiny, so the waits
    for it expire while every kernel still runs to its end.  Expected: everything up to and
    including the silent partition is right, everything that depends on it is NaN."""
    import torch

    S = tcu.FullStrategy
    n = 1 << 22
    x = oracle.generate_f16(n, 9, oracle.DIST_UNIFORM)
    ref = oracle.seg_scan_f64(x, 1, n)
    xd = to_dev(x)
    mute = 5  # partition index 4 is silent
    try:
        tcu.set_option("lookback_poll_limit", 16)
        tcu.set_option("test_mute_partition", mute)
        # (strategy, segment_size, waves) -> halves per partition
        for strategy, seg, w, part in [(S.SINGLE_PASS, 0, 0, 65536), (S.SINGLE_PASS, 8192, 4, 8192), (S.AUTO, 0, 0, 98304), (S.SINGLE_PASS | tcu.FULL_MFMA, 0, 0, 65536)]:
            tcu.set_option("scan_lds_tiles", 1 if part == 98304 else -1)  # AUTO with tiles parked in LDS: forced, the library takes it up to 2^27 elements only
            ws = torch.zeros(tcu.binding.full_workspace_bytes("scan", n, strategy, seg, w) // 4, dtype=torch.int32, device="cuda")
            got = to_host(tcu.full_scan(xd, strategy, seg, w, workspace=ws))
            # word 1 of the workspace counts the waits that gave up: the partition behind the silent one for certain,
            # later ones only if their own limit ran out before that partition published its NaN prefix
            assert 1 <= int(ws[1].item()) <= (n + part - 1) // part - mute, f"scan strategy={int(strategy):#x}: expired waits {int(ws[1].item())}"
            good = mute * part
            expect_ok(oracle, got[:good], ref[:good], n, f"scan strategy={int(strategy):#x}: partitions before the silent one")
            assert np.isnan(got[good:].view(np.float16)).all(), f"scan strategy={int(strategy):#x}: data after a wait that expired must be NaN"
            red = to_host(tcu.full_reduce(xd, S.SINGLE_PASS | (strategy & tcu.FULL_MFMA), seg, w))
            assert np.isnan(red.view(np.float16)).all(), f"reduce strategy={int(strategy):#x}: the result of a wait that expired must be NaN"
        # the look-back path of the segmented scan (segments of 2^21 halves = 32 partitions): only the silent
        # partition's segment is affected
        seg = 1 << 21
        refs = oracle.seg_scan_f64(x, n // seg, seg)
        tot = torch.zeros(n // seg, dtype=torch.float16, device="cuda")
        got = to_host(tcu.seg_scan(xd, seg, totals=tot))
        good = mute * 65536
        expect_ok(oracle, got[:good], refs[:good], seg, "segmented look-back scan: before the silent partition")
        assert np.isnan(got[good:seg].view(np.float16)).all()
        expect_ok(oracle, got[seg:], refs[seg:], seg, "segmented look-back scan: the other segment")
        th = to_host(tot)
        assert np.isnan(th[:1].view(np.float16)).all()
        expect_ok(oracle, th[1:], refs[-1:], seg, "segmented look-back scan: total of the other segment")
    finally:
        tcu.set_option("test_mute_partition", 0)
        tcu.set_option("scan_lds_tiles", -1)
        tcu.set_option("lookback_poll_limit", -1)
    # and with the defaults restored the same calls are right again
    ws = torch.ones(tcu.binding.full_workspace_bytes("scan", n, S.SINGLE_PASS) // 4, dtype=torch.int32, device="cuda")
    expect_ok(oracle, to_host(tcu.full_scan(xd, S.SINGLE_PASS, workspace=ws)), ref, n, "scan after the options were reset")
    assert int(ws[1].item()) == 0  # no wait gave up
    expect_ok(oracle, to_host(tcu.full_reduce(xd, S.SINGLE_PASS)), ref[-1:], n, "reduce after the options were reset")


def test_convert_f32_to_f16_bit_exact(tcu, oracle):
    """tcu_convert_f32_to_f16 (the reference's convertFp32ToFp16, src/utils/cuda_helpers.cuh:116-121) against the
    oracle's round-to-nearest-even conversion: random bit patterns of every exponent, dense samples around the
    subnormal / normal / overflow boundaries, every exact tie between neighbouring halves, +-65520, +-0, infinities."""
    import torch

    rng = np.random.default_rng(21)
    raw = rng.integers(0, 1 << 32, size=1 << 18, dtype=np.uint64).astype(np.uint32).view(np.float32)
    near = np.concatenate([rng.uniform(-70000, 70000, 1 << 16), rng.uniform(-1e-4, 1e-4, 1 << 16), rng.uniform(-2, 2, 1 << 16)]).astype(np.float32)
    halves = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    ties = ((halves[:-1] + halves[1:]) / 2).astype(np.float32)
    edge = np.float32([65520.0, -65520.0, 65519.996, -65519.996, 65504.0, 2.0 ** -25, -(2.0 ** -25), 2.0 ** -24, 2.0 ** -14, 6.0975552e-05, 0.0, -0.0, np.inf, -np.inf, 0.001])
    vals = np.concatenate([raw, near, ties, -ties, np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)), edge])
    vals = vals[~np.isnan(vals)]
    want = oracle.f32_to_f16_array(vals)
    got = to_host(tcu.convert_f32_to_f16(torch.from_numpy(vals).cuda()))
    assert got.shape == want.shape
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, f"{bad.size} conversions differ, first: {vals[bad[0]]!r} -> {got[bad[0]]:#06x}, oracle {want[bad[0]]:#06x}"
    # NaN in, NaN out
    nan = to_host(tcu.convert_f32_to_f16(torch.tensor([float("nan")], device="cuda")))
    assert (nan[0] & 0x7C00) == 0x7C00 and (nan[0] & 0x03FF) != 0
    # empty input: nothing is launched, nothing fails
    tcu.convert_f32_to_f16(torch.empty(0, dtype=torch.float32, device="cuda"))


def test_add_partial_sums(tcu, oracle):
    for seg, nseg in [(256, 100), (2048, 33), (24, 10)]:
        out = oracle.generate_f16(seg * nseg, 4, oracle.DIST_UNIFORM)
        ps = oracle.generate_f16(nseg, 6, oracle.DIST_UNIFORM)
        d = to_dev(out)
        tcu.add_partial_sums(d, to_dev(ps), seg)
        assert np.array_equal(to_host(d), oracle.add_partial_sums_ref(out, ps, nseg, seg))


@pytest.mark.parametrize("M,K", [(16384, 16384), (4096, 1024), (1000, 4096), (37, 264), (5, 20)])
def test_gemv(tcu, oracle, M, K):
    import torch

    A = oracle.generate_f16(M * K, 1, oracle.DIST_NORMAL)
    x = oracle.generate_f16(K, 2, oracle.DIST_NORMAL)
    y0 = np.linspace(-1, 1, M).astype(np.float32)
    Ad, xd = to_dev(A).view(M, K), to_dev(x)
    for v in (tcu.Variant.AUTO, tcu.Variant.WAVE_SHUFFLE, tcu.Variant.MFMA_16N, tcu.Variant.MFMA_256N):
        for alpha, beta in [(1.0, 0.0), (1.5, -0.5)]:
            y = torch.from_numpy(y0.copy()).cuda()
            try:
                tcu.gemv(Ad, xd, alpha, beta, y=y, variant=v)
            except tcu.TcuError as e:
                assert e.status == 2 and K % 8 != 0
                continue
            torch.cuda.synchronize()
            ref = oracle.gemv_f64(A, x, M, K, alpha, beta, y0)
            # fp32 accumulation of K products of N(0,1) values: 1e-2 relative at the scale sqrt(K)
            bad, worst, first = oracle.check_f32_rel(y.cpu().numpy(), ref, 1e-2, float(np.sqrt(K)))
            assert bad == 0, (v.name, alpha, beta, bad, worst, first)
            bad, worst, first = oracle.check_f32_rel(y.cpu().numpy(), ref, 1e-4, float(np.sqrt(K)))
            assert bad == 0, ("tight", v.name, alpha, beta, bad, worst, first)
            # fp16 y (tcu_gemv_f16_f16): the same fp32 sums, rounded once
            y0h = y0.astype(np.float16)
            yh = torch.from_numpy(y0h.copy()).cuda()
            tcu.gemv(Ad, xd, alpha, beta, y=yh, variant=v)
            torch.cuda.synchronize()
            ref = oracle.gemv_f64(A, x, M, K, alpha, beta, y0h.astype(np.float32))
            bad, worst, first = oracle.check_f16(yh.cpu().numpy().view(np.uint16), ref, K, ulps=1.0, abs_per_sqrt=1e-4)
            assert bad == 0, ("fp16 y", v.name, alpha, beta, bad, worst, first)


@pytest.mark.parametrize("M,K,lda", [(4096, 4096, 4096), (1000, 264, 1008), (2051, 1160, 2056), (513, 8, 520), (37, 24, 41), (5, 7, 5), (16384, 16384, 16384)])
def test_gemv_col_major(tcu, oracle, M, K, lda):
    """tcu_gemv_col_major_f16_f32 / _f16 (A as the reference's kernels hold it: element (m, k) at A[m + k*lda]) against the
    fp64 product (1e-4 at the scale sqrt(K), as for the row-major entry points), with rows of padding between the columns,
    ragged last slabs, the scalar kernel (lda or K not a multiple of 8), and against tcu_gemv_f16_f32 on the transposed
    copy; the same call twice gives the same bits (every sum is taken in a fixed order)."""
    import torch

    At = oracle.generate_f16(K * lda, 3, oracle.DIST_NORMAL).reshape(K, lda)
    x = oracle.generate_f16(K, 4, oracle.DIST_NORMAL)
    A = np.ascontiguousarray(At[:, :M].T).reshape(-1)
    y0 = np.linspace(-1, 1, M).astype(np.float32)
    Atd, xd = to_dev(At.reshape(-1)).view(K, lda)[:, :M], to_dev(x)
    for alpha, beta in [(1.0, 0.0), (1.5, -0.5)]:
        y = torch.from_numpy(y0.copy()).cuda()
        tcu.gemv_col_major(Atd, xd, alpha, beta, y=y)
        ref = oracle.gemv_f64(A, x, M, K, alpha, beta, y0)
        bad, worst, first = oracle.check_f32_rel(y.cpu().numpy(), ref, 1e-4, float(np.sqrt(K)))
        assert bad == 0, (alpha, beta, bad, worst, first)
        again = torch.from_numpy(y0.copy()).cuda()
        tcu.gemv_col_major(Atd, xd, alpha, beta, y=again)
        assert torch.equal(again, y)
        y0h = y0.astype(np.float16)
        yh = torch.from_numpy(y0h.copy()).cuda()
        tcu.gemv_col_major(Atd, xd, alpha, beta, y=yh)
        ref = oracle.gemv_f64(A, x, M, K, alpha, beta, y0h.astype(np.float32))
        bad, worst, first = oracle.check_f16(yh.cpu().numpy().view(np.uint16), ref, K, ulps=1.0, abs_per_sqrt=1e-4)
        assert bad == 0, ("fp16 y", alpha, beta, bad, worst, first)
    if K % 8 == 0:
        row_major = tcu.gemv(to_dev(A).view(M, K), xd)
        col_major = tcu.gemv_col_major(Atd, xd)
        assert torch.allclose(row_major, col_major, rtol=0, atol=1e-4 * float(np.sqrt(K)))
    with pytest.raises(ValueError):
        tcu.gemv_col_major(Atd.t(), xd)  # columns not contiguous


@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (512, 384, 160), (384, 640, 1088), (96, 64, 48), (33, 17, 20)])
def test_gemm_small_exact_and_normal(tcu, oracle, M, N, K):
    import torch

    C0 = (np.arange(M * N) % 7).astype(np.float32)
    for dist, exact in [(oracle.DIST_SMALLINT, True), (oracle.DIST_NORMAL, False)]:
        A = oracle.generate_f16(M * K, 5, dist)
        B = oracle.generate_f16(N * K, 6, dist)
        Ad, Bd = to_dev(A).view(M, K), to_dev(B).view(N, K)
        for v in (tcu.Variant.AUTO, tcu.Variant.BLOCK_LDS, tcu.Variant.MFMA_16N):
            for alpha, beta in [(1.0, 0.0), (2.0, 3.0)]:
                Cd = torch.from_numpy(C0.copy()).cuda().view(M, N)
                try:
                    D = tcu.gemm(Ad, Bd, alpha, beta, C=Cd, variant=v)
                except tcu.TcuError as e:
                    assert e.status == 2
                    continue
                torch.cuda.synchronize()
                ref = oracle.gemm_f64(A, B, M, N, K, alpha, beta, C0)
                got = D.cpu().numpy()
                if exact:  # the reference's rand()%3 fill: integer sums are exact in fp32
                    assert np.array_equal(got.astype(np.float64), ref), (v.name, alpha, beta)
                else:
                    bad, worst, first = oracle.check_f32_rel(got, ref, 1e-2, float(np.sqrt(K)))
                    assert bad == 0, (v.name, alpha, beta, bad, worst, first)
                # fp16 C and D (tcu_gemm_f16_f16)
                Ch = torch.from_numpy(C0.astype(np.float16)).cuda().view(M, N)
                Dh = tcu.gemm(Ad, Bd, alpha, beta, C=Ch, variant=v)
                torch.cuda.synchronize()
                assert Dh.dtype == torch.float16
                goth = Dh.cpu().numpy()
                if exact:  # the fp32 result is exact, so the output is its one rounding to fp16
                    assert np.array_equal(goth.view(np.uint16), ref.astype(np.float16).view(np.uint16)), ("fp16", v.name, alpha, beta)
                else:
                    bad, worst, first = oracle.check_f16(goth.view(np.uint16), ref, K, ulps=1.0, abs_per_sqrt=1e-4)
                    assert bad == 0, ("fp16", v.name, alpha, beta, bad, worst, first)


def test_gemm_big_tile_pipeline_shapes(tcu, oracle):
    """The 256 x 256 tile kernels (register-staged and direct-to-LDS) in every (K step, prefetch depth / buffer count) instantiation, including the
    depths the dispatcher falls back to when the step count is not a multiple of the requested
    one, and with C aliasing D.  Integer-valued inputs: results must be exact."""
    import torch

    M, N = 512, 256
    try:
        tcu.set_option("gemm_big_tiles", 1)  # two tiles: the default would take the 128 x 128 kernel
        for K in (64, 96, 160, 384, 768):
            A = oracle.generate_f16(M * K, 11, oracle.DIST_SMALLINT)
            B = oracle.generate_f16(N * K, 12, oracle.DIST_SMALLINT)
            C0 = (np.arange(M * N) % 5).astype(np.float32)
            Ad, Bd = to_dev(A).view(M, K), to_dev(B).view(N, K)
            ref0 = oracle.gemm_f64(A, B, M, N, K, 1.0, 0.0, C0)
            ref1 = oracle.gemm_f64(A, B, M, N, K, 2.0, -1.0, C0)
            # 66 (the default kernel) with its outputs turned through LDS (default) and straight from the accumulator layout
            shapes = [(0, bk64, depth, 1) for bk64 in (0, 1) for depth in (1, 2, 3, 4)] + [(3, 0, 4, 1), (4, 0, 4, 1), (64, 0, 4, 1), (65, 0, 4, 1), (66, 0, 4, 1), (66, 0, 4, 0)]
            for direct_lds, bk64, depth, staged in shapes:
                tcu.set_option("gemm_staged_epilogue", staged)
                tcu.set_option("gemm_direct_lds", direct_lds)
                tcu.set_option("gemm_bk64", bk64)
                tcu.set_option("gemm_depth", depth)
                D = tcu.gemm(Ad, Bd, 1.0, 0.0, variant=tcu.Variant.BLOCK_LDS)
                torch.cuda.synchronize()
                assert np.array_equal(D.cpu().numpy().astype(np.float64), ref0), (K, direct_lds, bk64, depth, staged)
                Cd = torch.from_numpy(C0.copy()).cuda().view(M, N)
                D = tcu.gemm(Ad, Bd, 2.0, -1.0, C=Cd, out=Cd, variant=tcu.Variant.BLOCK_LDS)  # in place
                torch.cuda.synchronize()
                assert np.array_equal(Cd.cpu().numpy().astype(np.float64), ref1), ("in place", K, direct_lds, bk64, depth, staged)
                # the same kernels with fp16 C and D, out of place and in place
                Dh = tcu.gemm(Ad, Bd, 1.0, 0.0, variant=tcu.Variant.BLOCK_LDS, out_dtype=torch.float16)
                Ch = torch.from_numpy(C0.astype(np.float16)).cuda().view(M, N)
                tcu.gemm(Ad, Bd, 2.0, -1.0, C=Ch, out=Ch, variant=tcu.Variant.BLOCK_LDS)
                torch.cuda.synchronize()
                assert np.array_equal(Dh.cpu().numpy().view(np.uint16), ref0.astype(np.float16).view(np.uint16)), ("fp16", K, direct_lds, bk64, depth, staged)
                assert np.array_equal(Ch.cpu().numpy().view(np.uint16), ref1.astype(np.float16).view(np.uint16)), ("fp16 in place", K, direct_lds, bk64, depth, staged)
        # default kernel choice with outputs that are 4-byte but not 8- or 16-byte aligned: the kernel that
        # moves four adjacent outputs per access must not be picked; aligned to 8 bytes only: not its 16-byte epilogue
        tcu.set_option("gemm_direct_lds", -1)
        tcu.set_option("gemm_staged_epilogue", 1)
        K = 384
        A = oracle.generate_f16(M * K, 13, oracle.DIST_SMALLINT)
        B = oracle.generate_f16(N * K, 14, oracle.DIST_SMALLINT)
        Ad, Bd = to_dev(A).view(M, K), to_dev(B).view(N, K)
        ref1 = oracle.gemm_f64(A, B, M, N, K, 2.0, -1.0, C0)
        buf32 = torch.zeros(M * N + 4, dtype=torch.float32, device="cuda")
        buf16 = torch.zeros(M * N + 4, dtype=torch.float16, device="cuda")
        for off32, off16 in ((0, 0), (1, 2), (2, 4)):
            Cd = buf32[off32:off32 + M * N].view(M, N)
            Cd.copy_(torch.from_numpy(C0).view(M, N))
            Ch = buf16[off16:off16 + M * N].view(M, N)
            Ch.copy_(torch.from_numpy(C0.astype(np.float16)).view(M, N))
            tcu.gemm(Ad, Bd, 2.0, -1.0, C=Cd, out=Cd)
            tcu.gemm(Ad, Bd, 2.0, -1.0, C=Ch, out=Ch)
            torch.cuda.synchronize()
            assert np.array_equal(Cd.cpu().numpy().astype(np.float64), ref1), ("offset", off32)
            assert np.array_equal(Ch.cpu().numpy().view(np.uint16), ref1.astype(np.float16).view(np.uint16)), ("offset fp16", off16)
        # the K-split tail of the grid: 264 = 256 + 8 tiles (11 x 24), the last 8 in 16 shares each (K = 8192: 128 steps
        # of 64, shares of at least 8), fp32 outputs in place and fp16 outputs.  Integer inputs: the result must equal,
        # bit for bit, that of the same launch with the split switched off, and the oracle on four rows of every tile row
        Ms, Ns, Ks = 2816, 6144, 8192
        A = oracle.generate_f16(Ms * Ks, 41, oracle.DIST_SMALLINT)
        B = oracle.generate_f16(Ns * Ks, 42, oracle.DIST_SMALLINT)
        Cs = (np.arange(Ms * Ns) % 5).astype(np.float32)
        Ad, Bd = to_dev(A).view(Ms, Ks), to_dev(B).view(Ns, Ks)
        got = {}
        for split in (1, 0):
            tcu.set_option("gemm_split_tail", split)
            Cd = torch.from_numpy(Cs.copy()).cuda().view(Ms, Ns)
            tcu.gemm(Ad, Bd, 0.5, -1.0, C=Cd, out=Cd)
            Ch = torch.from_numpy(Cs.astype(np.float16)).cuda().view(Ms, Ns)
            Dh = tcu.gemm(Ad, Bd, 0.5, -1.0, C=Ch)
            torch.cuda.synchronize()
            got[split] = (Cd.cpu().numpy(), Dh.cpu().numpy().view(np.uint16))
        tcu.set_option("gemm_split_tail", 1)
        assert np.array_equal(got[1][0], got[0][0]) and np.array_equal(got[1][1], got[0][1]), "split tail vs unsplit"
        for tm in range(Ms // 256):
            ref = oracle.gemm_f64(A, B, Ms, Ns, Ks, 0.5, -1.0, Cs, row0=tm * 256 + 37, rows=4)
            assert np.array_equal(got[1][0][tm * 256 + 37:tm * 256 + 41].astype(np.float64), ref), ("split tail", tm)
            assert np.array_equal(got[1][1][tm * 256 + 37:tm * 256 + 41], ref.astype(np.float16).view(np.uint16)), ("split tail fp16", tm)
        # 128 x 128 tiles: the 16x16x32 kernel (K a multiple of 64; outputs through LDS and straight from the accumulators),
        # the 32x32x16 transfer kernel (K step 64 and 32) and the register-staged one
        tcu.set_option("gemm_big_tiles", 0)
        tcu.set_option("gemm_bk64", 0)
        for direct_lds, K, staged in ((-1, 64, 1), (-1, 448, 1), (-1, 448, 0), (64, 448, 1), (-1, 224, 1), (0, 224, 1)):
            tcu.set_option("gemm_direct_lds", direct_lds)
            tcu.set_option("gemm_staged_epilogue", staged)
            A = oracle.generate_f16(M * K, 21, oracle.DIST_SMALLINT)
            B = oracle.generate_f16(N * K, 22, oracle.DIST_SMALLINT)
            Ad, Bd = to_dev(A).view(M, K), to_dev(B).view(N, K)
            Cd = torch.from_numpy(C0.copy()).cuda().view(M, N)
            tcu.gemm(Ad, Bd, 2.0, -1.0, C=Cd, out=Cd, variant=tcu.Variant.BLOCK_LDS)
            Dh = tcu.gemm(Ad, Bd, 1.0, 0.0, variant=tcu.Variant.BLOCK_LDS, out_dtype=torch.float16)
            torch.cuda.synchronize()
            Ch = torch.from_numpy(C0.astype(np.float16)).cuda().view(M, N)
            tcu.gemm(Ad, Bd, 2.0, -1.0, C=Ch, out=Ch, variant=tcu.Variant.BLOCK_LDS)  # fp16 in place
            torch.cuda.synchronize()
            ref1 = oracle.gemm_f64(A, B, M, N, K, 2.0, -1.0, C0)
            assert np.array_equal(Cd.cpu().numpy().astype(np.float64), ref1), ("128 tiles", direct_lds, K, staged)
            assert np.array_equal(Dh.cpu().numpy().view(np.uint16), oracle.gemm_f64(A, B, M, N, K, 1.0, 0.0, C0).astype(np.float16).view(np.uint16)), ("128 tiles fp16", direct_lds, K, staged)
            assert np.array_equal(Ch.cpu().numpy().view(np.uint16), ref1.astype(np.float16).view(np.uint16)), ("128 tiles fp16 in place", direct_lds, K, staged)
        # 192 x 192 tiles, forced (the default takes them where they fill the chip better than 256 x 256 ones): M and N need
        # not be multiples of 128
        tcu.set_option("gemm_big_tiles", 192)
        tcu.set_option("gemm_direct_lds", -1)
        M3, N3 = 576, 960
        C3 = (np.arange(M3 * N3) % 5).astype(np.float32)
        for K, staged in ((64, 1), (448, 1), (448, 0)):
            tcu.set_option("gemm_staged_epilogue", staged)
            A = oracle.generate_f16(M3 * K, 23, oracle.DIST_SMALLINT)
            B = oracle.generate_f16(N3 * K, 24, oracle.DIST_SMALLINT)
            Ad, Bd = to_dev(A).view(M3, K), to_dev(B).view(N3, K)
            Cd = torch.from_numpy(C3.copy()).cuda().view(M3, N3)
            tcu.gemm(Ad, Bd, 2.0, -1.0, C=Cd, out=Cd)
            Dh = tcu.gemm(Ad, Bd, 1.0, 0.0, out_dtype=torch.float16)
            Ch = torch.from_numpy(C3.astype(np.float16)).cuda().view(M3, N3)
            tcu.gemm(Ad, Bd, 2.0, -1.0, C=Ch, out=Ch)
            torch.cuda.synchronize()
            ref1 = oracle.gemm_f64(A, B, M3, N3, K, 2.0, -1.0, C3)
            assert np.array_equal(Cd.cpu().numpy().astype(np.float64), ref1), ("192 tiles", K, staged)
            assert np.array_equal(Dh.cpu().numpy().view(np.uint16), oracle.gemm_f64(A, B, M3, N3, K, 1.0, 0.0, C3).astype(np.float16).view(np.uint16)), ("192 tiles fp16", K, staged)
            assert np.array_equal(Ch.cpu().numpy().view(np.uint16), ref1.astype(np.float16).view(np.uint16)), ("192 tiles fp16 in place", K, staged)
    finally:
        tcu.set_option("gemm_split_tail", 1)
        tcu.set_option("gemm_staged_epilogue", 1)
        tcu.set_option("gemm_direct_lds", -1)
        tcu.set_option("gemm_bk64", 0)
        tcu.set_option("gemm_depth", 4)
        tcu.set_option("gemm_big_tiles", -1)


def test_gemm_kernels_round_alike(tcu):
    """alpha * acc + beta * c is one spelled-out rounding sequence in every GEMM epilogue: the direct kernel, the tiled
    kernel with its outputs turned through LDS and the same kernel writing straight from the accumulators agree bit
    for bit on inputs that are not integers (fp32 outputs; with fp16 outputs the two tiled forms agree bit for bit and
    the direct kernel to one unit in the last place)."""
    import torch

    M = N = 512
    K = 1024
    A = tcu.generate(M * K, 5, tcu.Dist.NORMAL).view(M, K)
    B = tcu.generate(N * K, 6, tcu.Dist.NORMAL).view(N, K)
    try:
        tcu.set_option("gemm_big_tiles", 1)
        for dt in (torch.float32, torch.float16):
            C = tcu.generate(M * N, 7, tcu.Dist.UNIFORM).view(M, N).to(dt)
            bits = torch.int32 if dt == torch.float32 else torch.int16
            got = {}
            for name, variant, staged in (("direct kernel", tcu.Variant.MFMA_16N, 1), ("tiled, through LDS", tcu.Variant.AUTO, 1), ("tiled, from the accumulators", tcu.Variant.AUTO, 0)):
                tcu.set_option("gemm_staged_epilogue", staged)
                got[name] = tcu.gemm(A, B, 1.1, 1.2, C=C, variant=variant).view(bits)
            # the same loop on 128 x 128 block tiles adds a given output's products in the same order
            tcu.set_option("gemm_big_tiles", 0)
            for staged in (1, 0):
                tcu.set_option("gemm_staged_epilogue", staged)
                got["128 tiles", staged] = tcu.gemm(A, B, 1.1, 1.2, C=C).view(bits)
            tcu.set_option("gemm_big_tiles", 1)
            torch.cuda.synchronize()
            assert torch.equal(got["tiled, through LDS"], got["tiled, from the accumulators"]), dt
            assert torch.equal(got["tiled, through LDS"], got["128 tiles", 1]) and torch.equal(got["tiled, through LDS"], got["128 tiles", 0]), dt
            if dt == torch.float32:
                assert torch.equal(got["direct kernel"], got["tiled, through LDS"])
            else:  # the compiler may narrow the fused multiply-add of one kernel in a single rounding: exact ties can fall the other way
                assert int((got["direct kernel"].int() - got["tiled, through LDS"].int()).abs().max()) <= 1
        # 192 x 192 tiles: the same loop again (768 = 3 x 256 = 4 x 192)
        M = N = 768
        A = tcu.generate(M * K, 8, tcu.Dist.NORMAL).view(M, K)
        B = tcu.generate(N * K, 9, tcu.Dist.NORMAL).view(N, K)
        for dt in (torch.float32, torch.float16):
            C = tcu.generate(M * N, 7, tcu.Dist.UNIFORM).view(M, N).to(dt)
            bits = torch.int32 if dt == torch.float32 else torch.int16
            tcu.set_option("gemm_staged_epilogue", 1)
            tcu.set_option("gemm_big_tiles", 1)
            want = tcu.gemm(A, B, 1.1, 1.2, C=C).view(bits)
            tcu.set_option("gemm_big_tiles", 192)
            for staged in (1, 0):
                tcu.set_option("gemm_staged_epilogue", staged)
                got192 = tcu.gemm(A, B, 1.1, 1.2, C=C).view(bits)
                torch.cuda.synchronize()
                assert torch.equal(want, got192), ("192 tiles", dt, staged)
    finally:
        tcu.set_option("gemm_staged_epilogue", 1)
        tcu.set_option("gemm_big_tiles", -1)


def test_gemm_8192(tcu, oracle):
    """M = N = K = 8192, N(0,1) inputs, 1e-2 relative: 64 sampled rows against the fp64 oracle."""
    import torch

    M = N = K = 8192
    Ad = tcu.generate(M * K, 11, tcu.Dist.NORMAL).view(M, K)
    Bd = tcu.generate(N * K, 12, tcu.Dist.NORMAL).view(N, K)
    D = tcu.gemm(Ad, Bd)
    torch.cuda.synchronize()
    A, B = to_host(Ad).ravel(), to_host(Bd).ravel()
    rows = [0, 1, 127, 128, 4095, 4096, 8191] + list(range(300, 8192, 997))
    for r in rows:
        ref = oracle.gemm_f64(A, B, M, N, K, row0=r, rows=1)
        bad, worst, first = oracle.check_f32_rel(D[r].cpu().numpy(), ref, 1e-2, float(np.sqrt(K)))
        assert bad == 0, (r, bad, worst, first)
        # the configuration's 1e-2 at the scale of an output (sqrt(K) = 90) would let a dropped product through: fp32
        # accumulation of K products of fp16 values keeps every output within 1e-4 * sqrt(K) of the fp64 product
        bad, worst, first = oracle.check_f32_rel(D[r].cpu().numpy(), ref, 1e-4, float(np.sqrt(K)))
        assert bad == 0, ("tight", r, bad, worst, first)
    # exact: small integers as inputs ({0, 1, 2}, the reference's rand() % 3 fill, src/gemm/wmma.cu:110-127) make every
    # fp32 partial sum exact (outputs <= 4 * 8192 < 2^24), so the default kernel must give the fp64 product bit for bit
    Ai = tcu.generate(M * K, 14, tcu.Dist.SMALLINT).view(M, K)
    Bi = tcu.generate(N * K, 15, tcu.Dist.SMALLINT).view(N, K)
    Di = tcu.gemm(Ai, Bi)
    torch.cuda.synchronize()
    Aih, Bih = to_host(Ai).ravel(), to_host(Bi).ravel()
    for r in rows[::3]:
        ref = oracle.gemm_f64(Aih, Bih, M, N, K, row0=r, rows=1)
        assert np.array_equal(Di[r].cpu().numpy().astype(np.float64), np.asarray(ref).ravel()), ("exact integers", r)
    # fp16 C and D with the benchmark's alpha and beta (reference src/gemm/wmma.cu:679-680)
    Ch = tcu.generate(M * N, 13, tcu.Dist.NORMAL).view(M, N)
    C32 = to_host(Ch).ravel().view(np.float16).astype(np.float32)
    Dh = tcu.gemm(Ad, Bd, 1.1, 1.2, C=Ch)
    torch.cuda.synchronize()
    assert Dh.dtype == torch.float16
    for r in rows[::2]:
        ref = oracle.gemm_f64(A, B, M, N, K, 1.1, 1.2, C32, row0=r, rows=1)
        bad, worst, first = oracle.check_f16(Dh[r].cpu().numpy().view(np.uint16), ref, K, ulps=1.0, abs_per_sqrt=1e-4)
        assert bad == 0, ("fp16", r, bad, worst, first)
