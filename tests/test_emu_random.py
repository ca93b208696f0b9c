"""Randomised cases over the CPU emulation of the kernels (see test_emu_kernels.py): random segment sizes, variants,
launch shapes, offsets arrays, key arrays, full-array strategies and GEMM shapes / tile families against the oracle, every
operand between guard pages.  The default run is a fixed seed and a few dozen cases; TCU_EMU_RANDOM_SEED / TCU_EMU_RANDOM_CASES run a longer
campaign by hand (5400 cases over 10 seeds passed when this file was written; 1050 more over 5 seeds with the GEMM cases)."""
import ctypes
import os

import numpy as np

import test_emu_kernels as T
from test_emu_kernels import aligned, copy_in, emu  # noqa: F401  (emu is the fixture)

SEED = int(os.environ.get("TCU_EMU_RANDOM_SEED", "2024"))
CASES = int(os.environ.get("TCU_EMU_RANDOM_CASES", "84"))
sz = ctypes.c_size_t


def fixed_size_case(rng, emu, oracle):
    seg = int(2 ** rng.integers(4, 14))
    nseg = int(rng.integers(1, max(2, min(200, 40000 // seg))))
    v, u, w = int(rng.integers(0, 9)), int(rng.choice([0, 1, 2, 4, 8])), int(rng.choice([0, 1, 2, 4, 8, 16]))
    tag = (seg, nseg, v, u, w)
    x = oracle.generate_f16(nseg * seg, int(rng.integers(1, 1000)), oracle.DIST_GRID)
    want_scan = oracle.seg_scan_f64(x, nseg, seg).astype(np.float16).view(np.uint16)
    want_red = want_scan.reshape(nseg, seg)[:, -1]
    xi = copy_in(x)
    red = aligned(nseg, np.uint16, 0xFFFF)
    rc = emu.emu_seg_reduce_f16(xi.ctypes.data, red.ctypes.data, nseg, seg, v, u, w)
    assert rc in (0, 2), (rc, emu.emu_last_error()) + tag  # 2: a family that does not take this size
    if rc == 0:
        assert np.array_equal(red, want_red), ("reduce",) + tag
    out, tot = aligned(nseg * seg, np.uint16, 0xFFFF), aligned(nseg, np.uint16, 0xFFFF)
    rc = emu.emu_seg_scan_f16(xi.ctypes.data, out.ctypes.data, tot.ctypes.data, nseg, seg, v, u, w)
    assert rc in (0, 2), (rc, emu.emu_last_error()) + tag
    if rc == 0:
        assert np.array_equal(out, want_scan) and np.array_equal(tot, want_red), ("scan",) + tag


def any_size_case(rng, emu, oracle):
    seg, nseg = int(rng.integers(1, 700)), int(rng.integers(1, 60))
    x = oracle.generate_f16(nseg * seg, int(rng.integers(1, 1000)), oracle.DIST_GRID)
    want_scan = oracle.seg_scan_f64(x, nseg, seg).astype(np.float16).view(np.uint16)
    xi = copy_in(x)
    red = aligned(nseg, np.uint16, 0xFFFF)
    assert emu.emu_seg_reduce_f16(xi.ctypes.data, red.ctypes.data, nseg, seg, 0, 0, 0) == 0, (seg, nseg)
    assert np.array_equal(red, want_scan.reshape(nseg, seg)[:, -1]), ("reduce", seg, nseg)
    out = aligned(nseg * seg, np.uint16, 0xFFFF)
    assert emu.emu_seg_scan_f16(xi.ctypes.data, out.ctypes.data, None, nseg, seg, 0, 0, 0) == 0
    assert np.array_equal(out, want_scan), ("scan", seg, nseg)


def offsets_reduce_case(rng, emu, oracle):
    expected = int(rng.choice([0, 8, 16, 64, 128, 1000, 2048, 4096, 70000, 1 << 18]))
    n = int(rng.integers(100, 40000))
    nseg = int(rng.integers(1, 8 if expected >= 65536 else 60 if expected >= 1000 else 300))
    max_len, bits = int(rng.choice([5, 40, 300, 3000, 50000])), int(rng.choice([32, 64]))
    x = oracle.generate_f16(n, int(rng.integers(1, 1000)), oracle.DIST_GRID)
    xi = copy_in(x)
    begin, end = T.ragged_offsets(rng, n, nseg, min(max_len, n))
    want = oracle.seg_reduce_offsets_f64(x, begin, end).astype(np.float16).view(np.uint16)
    dt = np.int32 if bits == 32 else np.int64
    bi, ei = copy_in(begin.astype(dt), dt), copy_in(end.astype(dt), dt)
    out = aligned(nseg, np.uint16, 0xFFFF)
    assert emu.emu_seg_reduce_offsets_f16(xi.ctypes.data, out.ctypes.data, nseg, bi.ctypes.data, ei.ctypes.data, bits, expected) == 0, emu.emu_last_error()
    assert np.array_equal(out, want), (n, nseg, max_len, expected, bits)


def offsets_scan_case(rng, emu, oracle):
    expected, bits = int(rng.choice([0, 8, 16, 64, 100, 1000, 1500, 3000, 1 << 16, 3 << 16, 1 << 19])), int(rng.choice([32, 64]))
    n = int(rng.integers(100, 40000))
    nseg = int(rng.integers(1, min(6 if expected >= 65536 else 60 if expected >= 1000 else 300, n // 4)))
    x = oracle.generate_f16(n, int(rng.integers(1, 1000)), oracle.DIST_GRID)
    xi = copy_in(x)
    begin, end = T.disjoint_offsets(rng, n, nseg, int(rng.integers(2, 20)))
    w64 = oracle.seg_scan_offsets_f64(x, begin, end)
    inside = ~np.isnan(w64)
    want = np.full(n, 0xFFFF, np.uint16)
    want[inside] = w64[inside].astype(np.float16).view(np.uint16)
    dt = np.int32 if bits == 32 else np.int64
    bi, ei = copy_in(begin.astype(dt), dt), copy_in(end.astype(dt), dt)
    out = aligned(n, np.uint16, 0xFFFF)
    assert emu.emu_seg_scan_offsets_f16(xi.ctypes.data, out.ctypes.data, nseg, bi.ctypes.data, ei.ctypes.data, bits, expected) == 0, emu.emu_last_error()
    assert np.array_equal(out, want), (n, nseg, expected, bits)


def full_array_case(rng, emu, oracle):
    n = int(rng.integers(1, 100000))
    if rng.random() < 0.5:
        n = n // 8 * 8 + 8
    strategy, wpb = int(rng.choice([0, 1, 1, 2, 0x100, 0x101])), int(rng.choice([0, 1, 2, 4, 8, 16]))
    seg = int(rng.choice([0, 256, 512, 1024, 2048, 4096, 8192, 65536]))
    x = oracle.generate_f16(n, int(rng.integers(1, 1000)), oracle.DIST_GRID)
    xi = copy_in(x)
    w64 = oracle.seg_scan_f64(x, 1, n)
    for op, fn in (("reduce", emu.emu_full_reduce_f16), ("scan", emu.emu_full_scan_f16)):
        tag = (op, n, strategy, seg, wpb)
        need = sz(0)
        rc = fn(xi.ctypes.data, None, n, None, ctypes.byref(need), strategy, seg, wpb)
        assert rc in (0, 1, 2), (rc,) + tag  # 1 / 2: a partition the block shape cannot have, n not a multiple of the segment
        if rc != 0:
            continue
        ws = aligned(need.value, np.uint8, 0xAB)
        out = aligned(n if op == "scan" else 1, np.uint16, 0xFFFF)
        assert fn(xi.ctypes.data, out.ctypes.data, n, ws.ctypes.data, ctypes.byref(need), strategy, seg, wpb) == 0, (emu.emu_last_error(),) + tag
        ref = w64 if op == "scan" else w64[-1:]
        if (strategy & 0xFF) != 2:
            assert np.array_equal(out, ref.astype(np.float16).view(np.uint16)), tag
        else:  # per-segment totals are rounded to fp16 on the way, as in the reference
            assert oracle.check_f16(out, ref, n)[0] == 0, tag


def by_key_case(rng, emu, oracle):
    n, bits, mean_run = int(rng.integers(1, 80000)), int(rng.choice([32, 64])), float(rng.choice([1, 2, 5, 17, 300, 5000, 1e9]))
    tag = (n, bits, mean_run)
    breaks = rng.random(n) < 1.0 / mean_run
    breaks[0] = True
    labels = rng.integers(-5, 6, breaks.sum())
    dt = np.int32 if bits == 32 else np.int64
    keys = labels[np.cumsum(breaks) - 1].astype(dt)
    heads = np.concatenate(([True], keys[1:] != keys[:-1]))  # runs are what the keys say: equal neighbours merge
    x = oracle.generate_f16(n, int(rng.integers(1, 1000)), oracle.DIST_GRID)
    xi, ki = copy_in(x), copy_in(keys, dt)
    want_scan = oracle.seg_scan_by_key_f64(keys, x).astype(np.float16).view(np.uint16)
    need = sz(0)
    assert emu.emu_seg_scan_by_key_f16(ki.ctypes.data, xi.ctypes.data, None, n, bits, None, ctypes.byref(need)) == 0
    ws, out = aligned(need.value, np.uint8, 0xAB), aligned(n, np.uint16, 0xFFFF)
    assert emu.emu_seg_scan_by_key_f16(ki.ctypes.data, xi.ctypes.data, out.ctypes.data, n, bits, ws.ctypes.data, ctypes.byref(need)) == 0, emu.emu_last_error()
    assert np.array_equal(out, want_scan), ("scan",) + tag
    runs = int(heads.sum())
    ko, so, nr = aligned(runs, dt, -1), aligned(runs, np.uint16, 0xFFFF), aligned(1, np.uint64, 0)
    assert emu.emu_seg_reduce_by_key_f16(None, None, None, None, None, n, bits, None, ctypes.byref(need)) == 0  # the reduction's own workspace size
    ws = aligned(need.value, np.uint8, 0xAB)
    assert emu.emu_seg_reduce_by_key_f16(ki.ctypes.data, xi.ctypes.data, ko.ctypes.data, so.ctypes.data, nr.ctypes.data, n, bits, ws.ctypes.data, ctypes.byref(need)) == 0, emu.emu_last_error()
    starts = np.flatnonzero(heads)
    assert int(nr[0]) == runs and np.array_equal(ko, keys[starts]), ("run keys",) + tag
    assert np.array_equal(so, want_scan[np.append(starts[1:], n) - 1]), ("run sums",) + tag


def gemm_case(rng, emu, oracle):
    """Random tile family (128 / 192 / 256 / none of them), K step, epilogue and scalars; integer-valued inputs, so the
    fp32 result is exact and the fp16 result is its one rounding."""
    unit = int(rng.choice([32, 64, 128, 192, 256]))
    M, N = unit * int(rng.integers(1, 4 if unit >= 128 else 7)), unit * int(rng.integers(1, 4 if unit >= 128 else 7))
    K = int(rng.choice([16, 32, 48, 64, 96, 128, 192, 320]))
    big, staged = int(rng.choice([-1, 0, 1, 192])), int(rng.integers(0, 2))
    alpha, beta = float(rng.choice([1.0, 0.5, 2.0, -1.5])), float(rng.choice([0.0, 1.0, -2.0]))
    variant = int(rng.choice([T.V_AUTO, T.V_AUTO, T.V_BLOCK, T.V_MFMA_16N]))
    tag = (M, N, K, big, staged, alpha, beta, variant)
    A, B = oracle.generate_f16(M * K, int(rng.integers(1, 1000)), oracle.DIST_SMALLINT), oracle.generate_f16(N * K, int(rng.integers(1, 1000)), oracle.DIST_SMALLINT)
    C0 = (np.arange(M * N) % 7 - 3).astype(np.float32)
    ref = oracle.gemm_f64(A, B, M, N, K, alpha, beta, C0)
    Ai, Bi = copy_in(A), copy_in(B)
    try:
        assert emu.emu_set_option(b"gemm_big_tiles", big) == 0 and emu.emu_set_option(b"gemm_staged_epilogue", staged) == 0
        D = copy_in(C0, np.float32)  # in place
        rc = emu.emu_gemm_f16_f32(Ai.ctypes.data, Bi.ctypes.data, D.ctypes.data, D.ctypes.data, M, N, K, alpha, beta, variant)
        assert rc in (0, 2), (rc, emu.emu_last_error()) + tag  # 2: a kernel family that does not take this shape
        if rc == 0:
            assert np.array_equal(D.reshape(M, N).astype(np.float64), ref), ("fp32",) + tag
        Ch = copy_in(C0.astype(np.float16).view(np.uint16))
        Dh = aligned(M * N, np.uint16, 0x7e00)
        rc = emu.emu_gemm_f16_f16(Ai.ctypes.data, Bi.ctypes.data, Ch.ctypes.data, Dh.ctypes.data, M, N, K, alpha, beta, variant)
        assert rc in (0, 2), (rc, emu.emu_last_error()) + tag
        if rc == 0:
            # by value: with beta == 0 a negative alpha times an exact zero sum is -0.0, which the fp64 reference writes as +0.0
            assert np.array_equal(Dh.view(np.float16).reshape(M, N), ref.astype(np.float16)), ("fp16",) + tag
    finally:
        emu.emu_set_option(b"gemm_big_tiles", -1)
        emu.emu_set_option(b"gemm_staged_epilogue", 1)


def test_random_cases(emu, oracle):
    emu.emu_seg_scan_by_key_f16.argtypes = [ctypes.c_void_p] * 3 + [sz, ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(sz)]
    emu.emu_seg_reduce_by_key_f16.argtypes = [ctypes.c_void_p] * 5 + [sz, ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(sz)]
    rng = np.random.default_rng(SEED)
    kinds = (fixed_size_case, any_size_case, offsets_reduce_case, offsets_scan_case, full_array_case, by_key_case, gemm_case)
    for i in range(CASES):
        kinds[i % len(kinds)](rng, emu, oracle)
