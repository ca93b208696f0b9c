"""Runs the GPU kernel SOURCES (tcu_scope_amd/csrc/*.hpp) lane by lane on the CPU, through the same
dispatch code the library uses, and compares with the oracle.  tests/emu/wave_ops_emu.hpp
replaces the wave primitives (DPP, lane swaps, MFMA, ballot) by rendezvous between 64
fibers per wave; it is strict about divergence around cross-lane operations.  This checks
indexing, lane-layout arithmetic, masks and tails without a GPU; the hardware behaviour
the emulation assumes is checked by tests/test_gpu_probe.py on the GPU."""
import ctypes
import mmap
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EMU = os.path.join(HERE, "emu")
CLANG = "/opt/rocm/llvm/bin/clang++"

V_AUTO, V_MFMA_16, V_MFMA_16N, V_MFMA_16N_BLOCK, V_MFMA_256, V_MFMA_256N, V_MFMA_256N_BLOCK, V_WAVE, V_BLOCK = range(9)


@pytest.fixture(scope="module")
def emu():
    if not os.path.exists(CLANG):
        pytest.skip("host clang++ (ROCm LLVM) not available")
    lib = os.path.join(EMU, "libtcu_emu.so")
    srcs = [os.path.join(EMU, f) for f in ("emu_driver.cpp", "wave_ops_emu.hpp")]
    csrc = os.path.join(HERE, "..", "tcu_scope_amd", "csrc")
    srcs += [os.path.join(csrc, f) for f in os.listdir(csrc) if f.endswith(".hpp")]
    if not os.path.exists(lib) or any(os.path.getmtime(s) > os.path.getmtime(lib) for s in srcs):
        subprocess.check_call([CLANG, "-x", "c++", "-std=c++17", "-O1", "-fPIC", "-shared", "-Wno-psabi", "-I" + EMU, "-o", lib, os.path.join(EMU, "emu_driver.cpp")])
    L = ctypes.CDLL(lib)
    sz, vp, ci, cf = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    L.emu_seg_reduce_f16.argtypes = [vp, vp, sz, sz, ci, ci, ci]
    L.emu_seg_scan_f16.argtypes = [vp, vp, vp, sz, sz, ci, ci, ci]
    L.emu_full_reduce_f16.argtypes = [vp, vp, sz, vp, ctypes.POINTER(sz), ci, sz, ci]
    L.emu_full_scan_f16.argtypes = [vp, vp, sz, vp, ctypes.POINTER(sz), ci, sz, ci]
    L.emu_gemv_f16_f32.argtypes = [vp, vp, vp, sz, sz, cf, cf, ci]
    L.emu_gemm_f16_f32.argtypes = [vp, vp, vp, vp, sz, sz, sz, cf, cf, ci]
    L.emu_gemv_f16_f16.argtypes = [vp, vp, vp, sz, sz, cf, cf, ci]
    L.emu_gemv_col_major_f16_f32.argtypes = [vp, sz, vp, vp, sz, sz, cf, cf]
    L.emu_gemv_col_major_f16_f16.argtypes = [vp, sz, vp, vp, sz, sz, cf, cf]
    L.emu_gemm_f16_f16.argtypes = [vp, vp, vp, vp, sz, sz, sz, cf, cf, ci]
    L.emu_set_option.argtypes = [ctypes.c_char_p, ci]
    L.emu_seg_reduce_offsets_f16.argtypes = [vp, vp, sz, vp, vp, ci, sz]
    L.emu_seg_scan_offsets_f16.argtypes = [vp, vp, sz, vp, vp, ci, sz]
    L.emu_generate_f16.argtypes = [vp, sz, ctypes.c_uint64, ci, sz]
    L.emu_last_error.restype = ctypes.c_char_p
    return L


_libc = ctypes.CDLL(None, use_errno=True)
_libc.mprotect.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
PAGE = mmap.PAGESIZE
# Every array handed to the emulated kernels lies between two inaccessible pages, so an access outside it ends the
# test run with a segmentation fault instead of reading or writing a neighbour.  "end" (default): the array's last
# byte (rounded up to 16) is the last byte before the page behind it; "start": its first byte follows the page in front.
GUARD = os.environ.get("TCU_EMU_GUARD", "end")


def aligned(n, dtype, fill=None):
    nbytes = n * np.dtype(dtype).itemsize
    body = max((nbytes + PAGE - 1) // PAGE, 1) * PAGE
    m = mmap.mmap(-1, body + 2 * PAGE)
    base = ctypes.addressof(ctypes.c_char.from_buffer(m))
    for guard in (base, base + PAGE + body):
        if _libc.mprotect(guard, PAGE, 0) != 0:  # PROT_NONE
            raise OSError(ctypes.get_errno(), "mprotect")
    off = PAGE if GUARD == "start" else PAGE + body - (nbytes + 15) // 16 * 16
    a = np.frombuffer(m, dtype=np.uint8, count=nbytes, offset=off).view(dtype)
    if fill is not None:
        a[:] = fill
    return a


def copy_in(x, dtype=np.uint16):
    a = aligned(max(x.size, 1), dtype)
    a[:x.size] = x
    return a


CASES = [  # (segment size, variants, (tiles per wave, waves per block) list, segment counts)
    (16, (V_WAVE, V_MFMA_16, V_MFMA_16N, V_AUTO, V_MFMA_16N_BLOCK, V_BLOCK), ((8, 2), (1, 1), (0, 4)), (96, 1027)),
    (64, (V_WAVE, V_MFMA_16N, V_BLOCK), ((4, 1), (0, 0)), (37,)),
    (256, (V_WAVE, V_MFMA_256, V_MFMA_256N, V_MFMA_256N_BLOCK, V_MFMA_16N_BLOCK), ((2, 2), (8, 1), (0, 2)), (19,)),
    (512, (V_WAVE, V_MFMA_16N, V_BLOCK, V_MFMA_256N_BLOCK), ((2, 1),), (9,)),
    (2048, (V_WAVE, V_MFMA_256N, V_BLOCK, V_MFMA_16N_BLOCK, V_AUTO), ((2, 2), (8, 1)), (5,)),
    (8192, (V_WAVE, V_MFMA_16N, V_MFMA_256N_BLOCK), ((4, 2),), (3,)),
    # blocks with more waves (and tiles per wave) than a segment has tiles: groups of waves take a segment each
    (512, (V_BLOCK, V_MFMA_256N_BLOCK, V_MFMA_16N_BLOCK), ((4, 4), (1, 16), (2, 2)), (9, 37)),
    (1024, (V_BLOCK, V_MFMA_16N_BLOCK), ((1, 8), (4, 4)), (7,)),
    (2048, (V_MFMA_256N_BLOCK,), ((1, 16), (8, 2)), (5,)),
]


@pytest.mark.parametrize("seg,variants,shapes,counts", CASES)
def test_segmented_kernels_bit_exact_on_grid_inputs(emu, oracle, seg, variants, shapes, counts):
    for nseg in counts:
        x = oracle.generate_f16(nseg * seg, 17 + seg, oracle.DIST_GRID)  # exact partial sums: results are fixed bit for bit
        sc = oracle.seg_scan_f64(x, nseg, seg)
        want_scan = sc.astype(np.float16).view(np.uint16)
        want_red = want_scan.reshape(nseg, seg)[:, -1]
        xi = copy_in(x)
        for v in variants:
            for u, w in shapes:
                red = aligned(nseg + 8, np.uint16, 0xFFFF)
                assert emu.emu_seg_reduce_f16(xi.ctypes.data, red.ctypes.data, nseg, seg, v, u, w) == 0, emu.emu_last_error()
                assert np.array_equal(red[:nseg], want_red) and np.all(red[nseg:] == 0xFFFF), ("reduce", seg, v, u, w, nseg)
                out = aligned(nseg * seg + 64, np.uint16, 0xFFFF)
                tot = aligned(nseg, np.uint16, 0xFFFF)
                assert emu.emu_seg_scan_f16(xi.ctypes.data, out.ctypes.data, tot.ctypes.data, nseg, seg, v, u, w) == 0, emu.emu_last_error()
                assert np.array_equal(out[:nseg * seg], want_scan) and np.all(out[nseg * seg:] == 0xFFFF), ("scan", seg, v, u, w, nseg)
                assert np.array_equal(tot, want_red), ("scan totals", seg, v, u, w, nseg)


def test_segments_larger_than_a_block_can_walk(emu, oracle):
    """AUTO cuts segments of 2^20 (reduce) / 2^21 (scan) halves and more into partitions:
    partition sums + per-segment finish, and the look-back scan restarted at segment starts."""
    seg, nseg = 1 << 20, 2
    x = oracle.generate_f16(nseg * seg, 5, oracle.DIST_GRID)
    want = oracle.seg_scan_f64(x, nseg, seg).astype(np.float16).view(np.uint16).reshape(nseg, seg)[:, -1]
    xi = copy_in(x)
    red = aligned(nseg + 8, np.uint16, 0xFFFF)
    assert emu.emu_seg_reduce_f16(xi.ctypes.data, red.ctypes.data, nseg, seg, V_AUTO, 0, 0) == 0, emu.emu_last_error()
    assert np.array_equal(red[:nseg], want) and np.all(red[nseg:] == 0xFFFF)
    seg, nseg = 1 << 21, 2
    x = oracle.generate_f16(nseg * seg, 6, oracle.DIST_GRID)
    want = oracle.seg_scan_f64(x, nseg, seg).astype(np.float16).view(np.uint16)
    xi = copy_in(x)
    out = aligned(nseg * seg + 64, np.uint16, 0xFFFF)
    tot = aligned(nseg + 8, np.uint16, 0xFFFF)
    assert emu.emu_seg_scan_f16(xi.ctypes.data, out.ctypes.data, tot.ctypes.data, nseg, seg, V_AUTO, 0, 0) == 0, emu.emu_last_error()
    assert np.array_equal(out[:nseg * seg], want) and np.all(out[nseg * seg:] == 0xFFFF)
    assert np.array_equal(tot[:nseg], want.reshape(nseg, seg)[:, -1]) and np.all(tot[nseg:] == 0xFFFF)
    # fewer segments than compute units: AUTO cuts them into partitions from 2^17 halves on (a block that walks such a
    # segment alone would leave most of the chip idle)
    seg, nseg = 1 << 17, 3
    x = oracle.generate_f16(nseg * seg, 7, oracle.DIST_GRID)
    want = oracle.seg_scan_f64(x, nseg, seg).astype(np.float16).view(np.uint16)
    xi = copy_in(x)
    red = aligned(nseg + 8, np.uint16, 0xFFFF)
    assert emu.emu_seg_reduce_f16(xi.ctypes.data, red.ctypes.data, nseg, seg, V_AUTO, 0, 0) == 0, emu.emu_last_error()
    assert np.array_equal(red[:nseg], want.reshape(nseg, seg)[:, -1]) and np.all(red[nseg:] == 0xFFFF)
    out = aligned(nseg * seg + 64, np.uint16, 0xFFFF)
    assert emu.emu_seg_scan_f16(xi.ctypes.data, out.ctypes.data, None, nseg, seg, V_AUTO, 0, 0) == 0, emu.emu_last_error()
    assert np.array_equal(out[:nseg * seg], want) and np.all(out[nseg * seg:] == 0xFFFF)


def ragged_offsets(rng, n, nseg, max_len):
    """begin/end of nseg segments inside [0, n): arbitrary starts, lengths 0..max_len, some inverted (= empty)."""
    begin = rng.integers(0, n, nseg)
    length = rng.integers(0, max_len + 1, nseg)
    end = np.minimum(begin + length, n)
    inverted = rng.random(nseg) < 0.05
    end[inverted] = begin[inverted] - rng.integers(0, 3, inverted.sum())
    return begin.astype(np.int64), end.astype(np.int64)


def test_segmented_reduction_over_offsets(emu, oracle):
    rng = np.random.default_rng(7)
    n = 50000
    x = oracle.generate_f16(n, 9, oracle.DIST_GRID)  # exact partial sums: any order gives the same bits
    xi = copy_in(x)
    for max_len, expected, bits in ((20, 16, 32), (20, 0, 64), (300, 128, 64), (3000, 0, 32), (3000, 2048, 32), (40, 64, 32), (9000, 4096, 32), (40000, 20000, 64), (3000, 100000, 32), (40000, 1 << 17, 64), (3000, 3 << 17, 32)):
        nseg = 12 if expected >= (1 << 17) else 100 if max_len > 1000 else 300
        begin, end = ragged_offsets(rng, n, nseg, max_len)
        want = oracle.seg_reduce_offsets_f64(x, begin, end).astype(np.float16).view(np.uint16)
        assert np.array_equal(want, oracle.seg_reduce_offsets_ref(x, begin, end))
        dt = np.int32 if bits == 32 else np.int64
        bi, ei = copy_in(begin.astype(dt), dt), copy_in(end.astype(dt), dt)
        out = aligned(nseg + 8, np.uint16, 0xFFFF)
        assert emu.emu_seg_reduce_offsets_f16(xi.ctypes.data, out.ctypes.data, nseg, bi.ctypes.data, ei.ctypes.data, bits, expected) == 0, emu.emu_last_error()
        assert np.array_equal(out[:nseg], want) and np.all(out[nseg:] == 0xFFFF), (max_len, expected, bits)
    # the offsets array of the reference's harness: one array, begin = offsets, end = offsets + 1
    seg, nseg = 48, 500
    off = copy_in((np.arange(nseg + 1) * seg).astype(np.int32), np.int32)
    out = aligned(nseg, np.uint16)
    assert emu.emu_seg_reduce_offsets_f16(xi.ctypes.data, out.ctypes.data, nseg, off.ctypes.data, off.ctypes.data + 4, 32, seg) == 0
    assert np.array_equal(out, oracle.seg_scan_f64(x, nseg, seg).astype(np.float16).view(np.uint16).reshape(nseg, seg)[:, -1])
    # input that is not 16-byte aligned: everything through the 2-byte path
    begin, end = ragged_offsets(rng, n - 1, 300, 100)
    want = oracle.seg_reduce_offsets_f64(x[1:], begin, end).astype(np.float16).view(np.uint16)
    bi, ei = copy_in(begin, np.int64), copy_in(end, np.int64)
    out = aligned(300, np.uint16)
    assert emu.emu_seg_reduce_offsets_f16(xi.ctypes.data + 2, out.ctypes.data, 300, bi.ctypes.data, ei.ctypes.data, 64, 64) == 0
    assert np.array_equal(out, want)
    assert emu.emu_seg_reduce_offsets_f16(xi.ctypes.data, out.ctypes.data, 300, bi.ctypes.data, ei.ctypes.data, 16, 0) == 1


def disjoint_offsets(rng, n, nseg, empty_every=11):
    """nseg disjoint ragged segments of [0, n) in increasing order with gaps between them, some empty."""
    cuts = np.sort(rng.choice(n, 2 * nseg, replace=False))
    begin, end = cuts[0::2].astype(np.int64), cuts[1::2].astype(np.int64)
    end[::empty_every] = begin[::empty_every]
    return begin, end


def test_segmented_scan_over_offsets(emu, oracle):
    rng = np.random.default_rng(12)
    n = 40000
    x = oracle.generate_f16(n, 10, oracle.DIST_GRID)  # exact partial sums: results are fixed bit for bit
    xi = copy_in(x)
    for nseg, expected, bits in ((1500, 16, 32), (1500, 0, 64), (300, 64, 32), (300, 100, 64), (40, 1000, 64), (40, 1500, 32), (40, 3000, 64), (7, 0, 32), (5, 1 << 16, 32), (4, 3 << 16, 64), (3, 1 << 19, 32)):
        begin, end = disjoint_offsets(rng, n, nseg)
        w64 = oracle.seg_scan_offsets_f64(x, begin, end)
        inside = ~np.isnan(w64)
        want = np.full(n, 0xFFFF, np.uint16)
        want[inside] = w64[inside].astype(np.float16).view(np.uint16)
        assert np.array_equal(want, oracle.seg_scan_offsets_ref(x, begin, end, fill=0xFFFF))
        dt = np.int32 if bits == 32 else np.int64
        bi, ei = copy_in(begin.astype(dt), dt), copy_in(end.astype(dt), dt)
        out = aligned(n + 64, np.uint16, 0xFFFF)
        assert emu.emu_seg_scan_offsets_f16(xi.ctypes.data, out.ctypes.data, nseg, bi.ctypes.data, ei.ctypes.data, bits, expected) == 0, emu.emu_last_error()
        assert np.array_equal(out[:n], want) and np.all(out[n:] == 0xFFFF), (nseg, expected, bits)
    # segments far longer than expected: slices that do not fit a block's registers are read twice by their block;
    # and the slice sums + second read form of the same lengths
    n2 = 200000
    x2 = oracle.generate_f16(n2, 11, oracle.DIST_GRID)
    x2i = copy_in(x2)
    begin, end = np.array([3, 199000], np.int64), np.array([198999, 199990], np.int64)
    w64 = oracle.seg_scan_offsets_f64(x2, begin, end)
    inside = ~np.isnan(w64)
    want = np.full(n2, 0xFFFF, np.uint16)
    want[inside] = w64[inside].astype(np.float16).view(np.uint16)
    bi, ei = copy_in(begin, np.int64), copy_in(end, np.int64)
    for chain, static_order in ((1, 0), (1, 1), (0, 0)):
        emu.emu_set_option(b"offsets_scan_chain", chain)
        emu.emu_set_option(b"static_order", static_order)
        out = aligned(n2 + 64, np.uint16, 0xFFFF)
        assert emu.emu_seg_scan_offsets_f16(x2i.ctypes.data, out.ctypes.data, 2, bi.ctypes.data, ei.ctypes.data, 64, 65537) == 0, emu.emu_last_error()
        assert np.array_equal(out[:n2], want) and np.all(out[n2:] == 0xFFFF), (chain, static_order)
    emu.emu_set_option(b"offsets_scan_chain", 1)
    emu.emu_set_option(b"static_order", 0)
    # uniform offsets from one array (begin = offsets, end = offsets + 1) == the fixed-size scan; in place
    seg, nseg = 200, 150
    off = copy_in((np.arange(nseg + 1) * seg).astype(np.int32), np.int32)
    buf = copy_in(x)
    assert emu.emu_seg_scan_offsets_f16(buf.ctypes.data, buf.ctypes.data, nseg, off.ctypes.data, off.ctypes.data + 4, 32, seg) == 0
    assert np.array_equal(buf[:nseg * seg], oracle.seg_scan_f64(x, nseg, seg).astype(np.float16).view(np.uint16)) and np.array_equal(buf[nseg * seg:n], x[nseg * seg:])
    # buffers that are not 16-byte aligned: the 2-byte path everywhere
    begin, end = disjoint_offsets(rng, n - 1, 200)
    w64 = oracle.seg_scan_offsets_f64(x[1:], begin, end)
    inside = ~np.isnan(w64)
    bi, ei = copy_in(begin, np.int64), copy_in(end, np.int64)
    out = aligned(n + 8, np.uint16, 0xFFFF)
    assert emu.emu_seg_scan_offsets_f16(xi.ctypes.data + 2, out.ctypes.data + 2, 200, bi.ctypes.data, ei.ctypes.data, 64, 32) == 0
    got = out[1:n]
    assert np.array_equal(got[inside], w64[inside].astype(np.float16).view(np.uint16)) and np.all(got[~inside] == 0xFFFF)


def test_generic_segment_sizes_and_preconditions(emu, oracle):
    for seg, nseg in ((1, 70), (7, 33), (100, 5)):
        x = oracle.generate_f16(nseg * seg, 3, oracle.DIST_GRID)
        sc = oracle.seg_scan_f64(x, nseg, seg).astype(np.float16).view(np.uint16)
        xi = copy_in(x)
        red = aligned(nseg, np.uint16)
        out = aligned(nseg * seg, np.uint16)
        assert emu.emu_seg_reduce_f16(xi.ctypes.data, red.ctypes.data, nseg, seg, V_AUTO, 0, 0) == 0
        assert emu.emu_seg_scan_f16(xi.ctypes.data, out.ctypes.data, None, nseg, seg, V_AUTO, 0, 0) == 0
        assert np.array_equal(out, sc) and np.array_equal(red, sc.reshape(nseg, seg)[:, -1])
        assert emu.emu_seg_reduce_f16(xi.ctypes.data, red.ctypes.data, nseg, seg, V_WAVE, 0, 0) == 2
    xi = copy_in(np.zeros(512, np.uint16))
    assert emu.emu_seg_reduce_f16(xi.ctypes.data, xi.ctypes.data, 4, 32, V_MFMA_16, 0, 0) == 2 and b"must be 16" in emu.emu_last_error()
    assert emu.emu_seg_scan_f16(xi.ctypes.data, xi.ctypes.data, None, 4, 128, V_MFMA_256N_BLOCK, 0, 0) == 2 and b"256" in emu.emu_last_error()
    assert emu.emu_seg_scan_f16(xi.ctypes.data, xi.ctypes.data, None, 2, 24, V_BLOCK, 0, 0) == 2


def test_full_array_kernels(emu, oracle):
    sz = ctypes.c_size_t
    for n in (8, 1003, 8192 * 3 + 1024, (1 << 16) + 56, 2 * 98304 + 8 * 37):
        x = oracle.generate_f16(n, 5, oracle.DIST_GRID)
        w64 = oracle.seg_scan_f64(x, 1, n)
        xi = copy_in(x)
        # 0x100 = TCU_FULL_MFMA: the single-pass kernels on the matrix unit
        # -1 as the first entry's last field: AUTO with 4 more tiles per wave parked in LDS, which the library itself only takes up to 2^27 elements
        for strategy, seg, wpb in ((0, 0, -1), (0, 0, 0), (1, 2048, 4), (1, 1024, 1), (2, 0, 0), (2, 256, 2), (0x100, 0, 0), (0x101, 2048, 4), (0x101, 512, 1)):
            emu.emu_set_option(b"scan_lds_tiles", 1 if wpb < 0 else -1)
            wpb = max(wpb, 0)
            for op, fn in (("reduce", emu.emu_full_reduce_f16), ("scan", emu.emu_full_scan_f16)):
                need = sz(0)
                rc = fn(xi.ctypes.data, None, n, None, ctypes.byref(need), strategy, seg, wpb)
                if rc == 2:
                    assert strategy == 2 and n % (seg or 2048)
                    continue
                assert rc == 0
                ws = aligned(need.value, np.uint8, 0xAB)  # the workspace needs no initialisation
                out = aligned(n if op == "scan" else 1, np.uint16, 0xFFFF)
                assert fn(xi.ctypes.data, out.ctypes.data, n, ws.ctypes.data, ctypes.byref(need), strategy, seg, wpb) == 0, emu.emu_last_error()
                ref = w64 if op == "scan" else w64[-1:]
                if strategy != 2:
                    assert np.array_equal(out, ref.astype(np.float16).view(np.uint16)), (op, n, strategy, seg, wpb)
                else:  # per-segment totals are rounded to fp16 on the way, as in the reference
                    assert oracle.check_f16(out, ref, n)[0] == 0, (op, n, strategy, seg, wpb)


def test_multi_kernel_sequences_with_many_totals(emu, oracle):
    """From `many_totals` per-segment totals on (65536; lowered here), the middle step of the reference's 2- and
    3-kernel sequences runs the partition sums / the single-pass scan on the totals instead of one block."""
    sz = ctypes.c_size_t
    try:
        assert emu.emu_set_option(b"many_totals", 64) == 0
        for op, fn, seg, nseg in (("reduce", emu.emu_full_reduce_f16, 16, 4096 + 8), ("reduce", emu.emu_full_reduce_f16, 16, 64 + 3), ("scan", emu.emu_full_scan_f16, 256, 64 + 8),
                                  ("scan", emu.emu_full_scan_f16, 256, 64 + 9), ("scan", emu.emu_full_scan_f16, 256, 63)):
            n = seg * nseg
            x = oracle.generate_f16(n, 9, oracle.DIST_GRID)
            w64 = oracle.seg_scan_f64(x, 1, n)
            xi = copy_in(x)
            need = sz(0)
            assert fn(xi.ctypes.data, None, n, None, ctypes.byref(need), 2, seg, 0) == 0
            nested = nseg >= 64 and (op == "reduce" or nseg % 8 == 0)
            assert (need.value > 2 * nseg + 256) == nested  # the totals, and the nested call's own workspace behind them
            ws = aligned(need.value, np.uint8, 0xAB)
            out = aligned(n if op == "scan" else 1, np.uint16, 0xFFFF)
            assert fn(xi.ctypes.data, out.ctypes.data, n, ws.ctypes.data, ctypes.byref(need), 2, seg, 0) == 0, emu.emu_last_error()
            ref = w64 if op == "scan" else w64[-1:]
            assert oracle.check_f16(out, ref, n)[0] == 0, (op, seg, nseg)
    finally:
        assert emu.emu_set_option(b"many_totals", 0) == 0


def test_a_wait_that_expires_gives_nan(emu, oracle):
    """A partition that publishes nothing (test option) with a small poll limit: the scan is right up to and
    including that partition and NaN after it, the reduction's result is NaN, every kernel returns."""
    sz = ctypes.c_size_t
    n = 8 * 2048 + 1024
    x = oracle.generate_f16(n, 5, oracle.DIST_GRID)
    want = oracle.seg_scan_f64(x, 1, n).astype(np.float16).view(np.uint16)
    xi = copy_in(x)
    mute = 3  # partition index 2
    try:
        assert emu.emu_set_option(b"lookback_poll_limit", 4) == 0
        assert emu.emu_set_option(b"test_mute_partition", mute) == 0
        for strategy in (1, 0x101):
            need = sz(0)
            assert emu.emu_full_scan_f16(xi.ctypes.data, None, n, None, ctypes.byref(need), strategy, 2048, 4) == 0
            ws = aligned(need.value, np.uint8, 0xAB)
            out = aligned(n, np.uint16, 0xFFFF)
            assert emu.emu_full_scan_f16(xi.ctypes.data, out.ctypes.data, n, ws.ctypes.data, ctypes.byref(need), strategy, 2048, 4) == 0, emu.emu_last_error()
            good = mute * 2048
            assert np.array_equal(out[:good], want[:good])
            assert np.isnan(out[good:].view(np.float16)).all()
            assert emu.emu_full_reduce_f16(xi.ctypes.data, None, n, None, ctypes.byref(need), strategy, 2048, 4) == 0
            ws = aligned(need.value, np.uint8, 0xAB)
            red = aligned(1, np.uint16, 0x1234)
            assert emu.emu_full_reduce_f16(xi.ctypes.data, red.ctypes.data, n, ws.ctypes.data, ctypes.byref(need), strategy, 2048, 4) == 0, emu.emu_last_error()
            assert np.isnan(red.view(np.float16)).all()
    finally:
        assert emu.emu_set_option(b"test_mute_partition", 0) == 0
        assert emu.emu_set_option(b"lookback_poll_limit", -1) == 0
    need = sz(0)
    assert emu.emu_full_scan_f16(xi.ctypes.data, None, n, None, ctypes.byref(need), 1, 2048, 4) == 0
    ws = aligned(need.value, np.uint8, 0xAB)
    out = aligned(n, np.uint16, 0xFFFF)
    assert emu.emu_full_scan_f16(xi.ctypes.data, out.ctypes.data, n, ws.ctypes.data, ctypes.byref(need), 1, 2048, 4) == 0
    assert np.array_equal(out, want)


def test_gemv_gemm_and_generator(emu, oracle):
    for dist in (0, 1, 3):
        out = aligned(5000, np.uint16)
        assert emu.emu_generate_f16(out.ctypes.data, 5000, 42, dist, 77) == 0
        assert np.array_equal(out, oracle.generate_f16(5000, 42, dist, first=77))
    for M, K in ((64, 512), (37, 256), (5, 24), (7, 4608), (3, 8192 + 264)):
        A, x = oracle.generate_f16(M * K, 1, oracle.DIST_NORMAL), oracle.generate_f16(K, 2, oracle.DIST_NORMAL)
        y0 = np.linspace(-1, 1, M).astype(np.float32)
        Ai, xi = copy_in(A), copy_in(x)
        for v in (V_AUTO, V_WAVE, V_MFMA_16N, V_MFMA_256N):
            y = copy_in(y0, np.float32)
            rc = emu.emu_gemv_f16_f32(Ai.ctypes.data, xi.ctypes.data, y.ctypes.data, M, K, 1.5, -0.5, v)
            if rc == 2:
                assert K % 8
                continue
            assert rc == 0 and oracle.check_f32_rel(y[:M], oracle.gemv_f64(A, x, M, K, 1.5, -0.5, y0), 1e-4, float(np.sqrt(K)))[0] == 0, (M, K, v)
            # fp16 y: same sums, rounded once
            y0h = y0.astype(np.float16)
            yh = copy_in(y0h.view(np.uint16))
            rc = emu.emu_gemv_f16_f16(Ai.ctypes.data, xi.ctypes.data, yh.ctypes.data, M, K, 1.5, -0.5, v)
            ref = oracle.gemv_f64(A, x, M, K, 1.5, -0.5, y0h.astype(np.float32))
            assert rc == 0 and oracle.check_f16(yh[:M], ref, K)[0] == 0, (M, K, v)
    # A column-major with a leading dimension: 512-row slabs with a ragged last one, several stretches of K, and the
    # scalar kernel (lda or K not a multiple of 8); the oracle's row-major product of the transposed copy is the reference
    for M, K, lda in ((64, 512, 64), (520, 136, 528), (513, 8, 520), (37, 24, 41), (5, 7, 5)):
        At = oracle.generate_f16(K * lda, 3, oracle.DIST_NORMAL).reshape(K, lda)  # row k = column k of A, lda - M values of padding
        x = oracle.generate_f16(K, 4, oracle.DIST_NORMAL)
        A = np.ascontiguousarray(At[:, :M].T).reshape(-1)
        y0 = np.linspace(-1, 1, M).astype(np.float32)
        Ati, xi = copy_in(At.reshape(-1)), copy_in(x)
        y = copy_in(y0, np.float32)
        assert emu.emu_gemv_col_major_f16_f32(Ati.ctypes.data, lda, xi.ctypes.data, y.ctypes.data, M, K, 1.5, -0.5) == 0, emu.emu_last_error()
        assert oracle.check_f32_rel(y[:M], oracle.gemv_f64(A, x, M, K, 1.5, -0.5, y0), 1e-4, float(np.sqrt(K)))[0] == 0, (M, K, lda)
        y0h = y0.astype(np.float16)
        yh = copy_in(y0h.view(np.uint16))
        assert emu.emu_gemv_col_major_f16_f16(Ati.ctypes.data, lda, xi.ctypes.data, yh.ctypes.data, M, K, 1.5, -0.5) == 0
        assert oracle.check_f16(yh[:M], oracle.gemv_f64(A, x, M, K, 1.5, -0.5, y0h.astype(np.float32)), K)[0] == 0, (M, K, lda)
    assert emu.emu_gemv_col_major_f16_f32(Ati.ctypes.data, 3, xi.ctypes.data, y.ctypes.data, 5, 7, 1.0, 0.0) == 1  # lda < M
    for M, N, K in ((128, 128, 64), (256, 512, 64), (128, 256, 96), (64, 32, 48), (33, 17, 20)):
        A, B = oracle.generate_f16(M * K, 5, oracle.DIST_SMALLINT), oracle.generate_f16(N * K, 6, oracle.DIST_SMALLINT)
        C0 = (np.arange(M * N) % 7).astype(np.float32)
        Ai, Bi, Ci = copy_in(A), copy_in(B), copy_in(C0, np.float32)
        for v in (V_AUTO, V_BLOCK, V_MFMA_16N):
            D = aligned(M * N, np.float32, -777)
            rc = emu.emu_gemm_f16_f32(Ai.ctypes.data, Bi.ctypes.data, Ci.ctypes.data, D.ctypes.data, M, N, K, 2.0, 3.0, v)
            if rc == 2:
                continue
            assert rc == 0 and np.array_equal(D.reshape(M, N).astype(np.float64), oracle.gemm_f64(A, B, M, N, K, 2.0, 3.0, C0)), (M, N, K, v)
            # fp16 C and D: the fp32 result is exact for these inputs, so D is its one rounding
            Ch = copy_in(C0.astype(np.float16).view(np.uint16))
            Dh = aligned(M * N, np.uint16, 0x7e00)
            rc = emu.emu_gemm_f16_f16(Ai.ctypes.data, Bi.ctypes.data, Ch.ctypes.data, Dh.ctypes.data, M, N, K, 1.5, 3.0, v)
            assert rc == 0 and np.array_equal(Dh.reshape(M, N), oracle.gemm_f64(A, B, M, N, K, 1.5, 3.0, C0).astype(np.float16).view(np.uint16)), (M, N, K, v)
    # the 256 x 256 tile kernels: register-staged (K step 32 / 64, every prefetch depth that
    # divides the step count) and direct-to-LDS (3 and 4 buffers)
    M, N, K = 256, 256, 192
    A, B = oracle.generate_f16(M * K, 7, oracle.DIST_SMALLINT), oracle.generate_f16(N * K, 8, oracle.DIST_SMALLINT)
    C0 = (np.arange(M * N) % 5).astype(np.float32)
    Ai, Bi, Ci = copy_in(A), copy_in(B), copy_in(C0, np.float32)
    ref = oracle.gemm_f64(A, B, M, N, K, 1.5, 2.0, C0)
    try:
        assert emu.emu_set_option(b"gemm_big_tiles", 1) == 0  # one tile: the default would take the 128 x 128 kernel
        assert emu.emu_set_option(b"gemm_staged_epilogue", 0) == 0  # outputs straight from the accumulator layout (default: through LDS, below)
        for direct_lds, bk64, depth in ((3, 0, 4), (4, 0, 4), (64, 0, 4), (65, 0, 4), (66, 0, 4), (0, 0, 1), (0, 0, 2), (0, 0, 3), (0, 0, 4), (0, 1, 1), (0, 1, 2)):
            for name, val in ((b"gemm_direct_lds", direct_lds), (b"gemm_bk64", bk64), (b"gemm_depth", depth)):
                assert emu.emu_set_option(name, val) == 0
            D = aligned(M * N, np.float32, -777)
            rc = emu.emu_gemm_f16_f32(Ai.ctypes.data, Bi.ctypes.data, Ci.ctypes.data, D.ctypes.data, M, N, K, 1.5, 2.0, V_BLOCK)
            assert rc == 0 and np.array_equal(D.reshape(M, N).astype(np.float64), ref), (direct_lds, bk64, depth)
            Dh = copy_in(C0.astype(np.float16).view(np.uint16))  # in place: C == D
            rc = emu.emu_gemm_f16_f16(Ai.ctypes.data, Bi.ctypes.data, Dh.ctypes.data, Dh.ctypes.data, M, N, K, 1.5, 2.0, V_BLOCK)
            assert rc == 0 and np.array_equal(Dh.reshape(M, N), ref.astype(np.float16).view(np.uint16)), (direct_lds, bk64, depth)
        # the same kernel with the outputs turned through LDS (whole rows per store): two tiles, fp32 and fp16 outputs,
        # in place and not, with and without C
        assert emu.emu_set_option(b"gemm_direct_lds", -1) == 0 and emu.emu_set_option(b"gemm_staged_epilogue", 1) == 0
        Mt, Nt, Kt = 512, 256, 128
        At, Bt = oracle.generate_f16(Mt * Kt, 21, oracle.DIST_SMALLINT), oracle.generate_f16(Nt * Kt, 22, oracle.DIST_SMALLINT)
        Ct = (np.arange(Mt * Nt) % 7).astype(np.float32)
        Ati, Bti = copy_in(At), copy_in(Bt)
        for beta in (2.0, 0.0):
            reft = oracle.gemm_f64(At, Bt, Mt, Nt, Kt, 1.5, beta, Ct)
            Cti = copy_in(Ct, np.float32)
            Dt = aligned(Mt * Nt, np.float32, -777)
            rc = emu.emu_gemm_f16_f32(Ati.ctypes.data, Bti.ctypes.data, Cti.ctypes.data, Dt.ctypes.data, Mt, Nt, Kt, 1.5, beta, V_BLOCK)
            assert rc == 0 and np.array_equal(Dt.reshape(Mt, Nt).astype(np.float64), reft), ("staged fp32", beta)
            rc = emu.emu_gemm_f16_f32(Ati.ctypes.data, Bti.ctypes.data, Cti.ctypes.data, Cti.ctypes.data, Mt, Nt, Kt, 1.5, beta, V_BLOCK)
            assert rc == 0 and np.array_equal(Cti.reshape(Mt, Nt).astype(np.float64), reft), ("staged fp32 in place", beta)
            Cht = copy_in(Ct.astype(np.float16).view(np.uint16))
            Dht = aligned(Mt * Nt, np.uint16, 0x7e00)
            rc = emu.emu_gemm_f16_f16(Ati.ctypes.data, Bti.ctypes.data, Cht.ctypes.data, Dht.ctypes.data, Mt, Nt, Kt, 1.5, beta, V_BLOCK)
            assert rc == 0 and np.array_equal(Dht.reshape(Mt, Nt), reft.astype(np.float16).view(np.uint16)), ("staged fp16", beta)
            rc = emu.emu_gemm_f16_f16(Ati.ctypes.data, Bti.ctypes.data, Cht.ctypes.data, Cht.ctypes.data, Mt, Nt, Kt, 1.5, beta, V_BLOCK)
            assert rc == 0 and np.array_equal(Cht.reshape(Mt, Nt), reft.astype(np.float16).view(np.uint16)), ("staged fp16 in place", beta)
            # fp16 outputs aligned to 8 bytes only: the direct epilogue takes over
            Dho = aligned(Mt * Nt + 4, np.uint16, 0x7e00)
            Cho = copy_in(Ct.astype(np.float16).view(np.uint16))
            rc = emu.emu_gemm_f16_f16(Ati.ctypes.data, Bti.ctypes.data, Cho.ctypes.data, Dho.ctypes.data + 8, Mt, Nt, Kt, 1.5, beta, V_BLOCK)
            assert rc == 0 and np.array_equal(Dho[4:].reshape(Mt, Nt), reft.astype(np.float16).view(np.uint16)) and np.all(Dho[:4] == 0x7e00), ("fp16 at 8 bytes", beta)
        # the K-split tail on a device of 4 units: 7 tiles -> the 48 K steps of the last 3 in 4 runs of 12, three of
        # which cross from one tile into the next; 9 tiles -> the last one in 2 runs (tile ids regrouped for 8 XCDs);
        # fp32 outputs in place, fp16 outputs with C
        assert emu.emu_set_option(b"gemm_direct_lds", -1) == 0 and emu.emu_set_option(b"compute_units", 4) == 0 and emu.emu_set_option(b"gemm_split_tail", 2) == 0
        for Ms, Ns, Ks in ((1792, 256, 1024), (768, 768, 1024)):
            As, Bs = oracle.generate_f16(Ms * Ks, 15, oracle.DIST_SMALLINT), oracle.generate_f16(Ns * Ks, 16, oracle.DIST_SMALLINT)
            Cs = (np.arange(Ms * Ns) % 5).astype(np.float32)
            Asi, Bsi = copy_in(As), copy_in(Bs)
            refs = oracle.gemm_f64(As, Bs, Ms, Ns, Ks, 0.5, 2.0, Cs)
            Ds = copy_in(Cs, np.float32)
            rc = emu.emu_gemm_f16_f32(Asi.ctypes.data, Bsi.ctypes.data, Ds.ctypes.data, Ds.ctypes.data, Ms, Ns, Ks, 0.5, 2.0, V_BLOCK)
            assert rc == 0 and np.array_equal(Ds.reshape(Ms, Ns).astype(np.float64), refs), ("split tail", Ms, Ns, Ks)
            if Ms == Ns:
                continue  # fp16 outputs once is enough: the two cases differ in the tile mapping only
            Chs = copy_in(Cs.astype(np.float16).view(np.uint16))
            Dhs = aligned(Ms * Ns, np.uint16, 0x7e00)
            rc = emu.emu_gemm_f16_f16(Asi.ctypes.data, Bsi.ctypes.data, Chs.ctypes.data, Dhs.ctypes.data, Ms, Ns, Ks, 0.5, 2.0, V_BLOCK)
            assert rc == 0 and np.array_equal(Dhs.reshape(Ms, Ns), refs.astype(np.float16).view(np.uint16)), ("split tail fp16", Ms, Ns, Ks)
        assert emu.emu_set_option(b"compute_units", 256) == 0 and emu.emu_set_option(b"gemm_split_tail", 1) == 0
        # 128 x 128 tiles: the 16x16x32 kernel (K a multiple of 64; outputs through LDS or straight from the accumulators,
        # fp16 outputs in place), the 32x32x16 transfer kernel (K step 64 and 32) and the register-staged one
        assert emu.emu_set_option(b"gemm_big_tiles", 0) == 0
        for direct_lds, Ks, staged in ((-1, 192, 1), (-1, 192, 0), (-1, 64, 1), (64, 192, 1), (-1, 96, 1), (0, 96, 1)):
            assert emu.emu_set_option(b"gemm_direct_lds", direct_lds) == 0 and emu.emu_set_option(b"gemm_staged_epilogue", staged) == 0
            A2, B2 = oracle.generate_f16(M * Ks, 9, oracle.DIST_SMALLINT), oracle.generate_f16(N * Ks, 10, oracle.DIST_SMALLINT)
            A2i, B2i = copy_in(A2), copy_in(B2)
            ref2 = oracle.gemm_f64(A2, B2, M, N, Ks, 1.5, 2.0, C0)
            D = aligned(M * N, np.float32, -777)
            rc = emu.emu_gemm_f16_f32(A2i.ctypes.data, B2i.ctypes.data, Ci.ctypes.data, D.ctypes.data, M, N, Ks, 1.5, 2.0, V_BLOCK)
            assert rc == 0 and np.array_equal(D.reshape(M, N).astype(np.float64), ref2), (direct_lds, Ks, staged)
            if direct_lds == -1 and Ks % 64 == 0:
                Dh = copy_in(C0.astype(np.float16).view(np.uint16))  # in place: C == D
                rc = emu.emu_gemm_f16_f16(A2i.ctypes.data, B2i.ctypes.data, Dh.ctypes.data, Dh.ctypes.data, M, N, Ks, 1.5, 2.0, V_BLOCK)
                assert rc == 0 and np.array_equal(Dh.reshape(M, N), ref2.astype(np.float16).view(np.uint16)), ("fp16", Ks, staged)
                D = aligned(M * N, np.float32, -777)  # beta = 0: C is not read
                rc = emu.emu_gemm_f16_f32(A2i.ctypes.data, B2i.ctypes.data, None, D.ctypes.data, M, N, Ks, 1.5, 0.0, V_BLOCK)
                assert rc == 0 and np.array_equal(D.reshape(M, N).astype(np.float64), oracle.gemm_f64(A2, B2, M, N, Ks, 1.5, 0.0, C0)), ("beta 0", Ks, staged)
        # 192 x 192 tiles (waves of 96 x 96; 48 of 64 lanes move the outputs that went through LDS): six and two tiles,
        # one and three K steps, outputs through LDS and straight from the accumulators, fp16 outputs in place, beta = 0
        assert emu.emu_set_option(b"gemm_big_tiles", 192) == 0 and emu.emu_set_option(b"gemm_direct_lds", -1) == 0
        for M3, N3, K3, staged in ((384, 576, 192, 1), (384, 576, 192, 0), (384, 192, 64, 1)):
            assert emu.emu_set_option(b"gemm_staged_epilogue", staged) == 0
            A3, B3 = oracle.generate_f16(M3 * K3, 17, oracle.DIST_SMALLINT), oracle.generate_f16(N3 * K3, 18, oracle.DIST_SMALLINT)
            C3 = (np.arange(M3 * N3) % 5).astype(np.float32)
            A3i, B3i = copy_in(A3), copy_in(B3)
            ref3 = oracle.gemm_f64(A3, B3, M3, N3, K3, 1.5, 2.0, C3)
            D3 = copy_in(C3, np.float32)  # in place
            rc = emu.emu_gemm_f16_f32(A3i.ctypes.data, B3i.ctypes.data, D3.ctypes.data, D3.ctypes.data, M3, N3, K3, 1.5, 2.0, V_AUTO)
            assert rc == 0 and np.array_equal(D3.reshape(M3, N3).astype(np.float64), ref3), ("192 tiles", M3, N3, K3, staged)
            Dh3 = copy_in(C3.astype(np.float16).view(np.uint16))
            rc = emu.emu_gemm_f16_f16(A3i.ctypes.data, B3i.ctypes.data, Dh3.ctypes.data, Dh3.ctypes.data, M3, N3, K3, 1.5, 2.0, V_AUTO)
            assert rc == 0 and np.array_equal(Dh3.reshape(M3, N3), ref3.astype(np.float16).view(np.uint16)), ("192 tiles fp16", M3, N3, K3, staged)
            D3 = aligned(M3 * N3, np.float32, -777)
            rc = emu.emu_gemm_f16_f32(A3i.ctypes.data, B3i.ctypes.data, None, D3.ctypes.data, M3, N3, K3, 1.5, 0.0, V_AUTO)
            assert rc == 0 and np.array_equal(D3.reshape(M3, N3).astype(np.float64), oracle.gemm_f64(A3, B3, M3, N3, K3, 1.5, 0.0, C3)), ("192 tiles beta 0", M3, N3, K3, staged)
    finally:
        for name, val in ((b"gemm_direct_lds", -1), (b"gemm_bk64", 0), (b"gemm_depth", 4), (b"gemm_big_tiles", -1), (b"compute_units", 256), (b"gemm_split_tail", 1), (b"gemm_staged_epilogue", 1)):
            emu.emu_set_option(name, val)


def run_keys(rng, n, mean_run):
    """Keys whose runs have geometric lengths around mean_run; equal keys may come back in later runs."""
    heads = rng.random(n) < 1.0 / mean_run
    ids = np.cumsum(heads)
    return (ids * 7919) % 1013 - 500 + (ids % 2) * (1 << 40)  # neighbours always differ; values need 64 bits


@pytest.mark.parametrize("bits", [32, 64])
def test_segments_given_by_keys(emu, oracle, bits):
    sz = ctypes.c_size_t
    emu.emu_seg_scan_by_key_f16.argtypes = [ctypes.c_void_p] * 3 + [sz, ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(sz)]
    emu.emu_seg_reduce_by_key_f16.argtypes = [ctypes.c_void_p] * 5 + [sz, ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(sz)]
    kt = np.int32 if bits == 32 else np.int64
    rng = np.random.default_rng(bits)
    part = 4 * 16 * 512
    cases = ((1, 1), (7, 2), (513, 1), (part - 3, 40), (part + 1, 5000), (2 * part + 77, 3), (2 * part + 77, 300), (2 * part, 10 ** 9))
    if bits == 64:  # the key width changes how keys are loaded and compared, nothing else: half of the cases cover it
        cases = ((7, 2), (part - 3, 40), (2 * part + 77, 3), (2 * part, 10 ** 9))
    for n, mean_run in cases:
        keys = run_keys(rng, n, mean_run)
        if bits == 32:
            keys = keys % (1 << 20)
        keys = keys.astype(kt)
        x = oracle.generate_f16(n, 5 + n, oracle.DIST_GRID)
        want_scan = oracle.seg_scan_by_key_f64(keys, x).astype(np.float16).view(np.uint16)
        want_keys, want_sums = oracle.seg_reduce_by_key_f64(keys, x)
        want_sums = want_sums.astype(np.float16).view(np.uint16)
        # the reduction in four launches that wait for nothing (one wave and four waves per block), then both
        # operations on the one-pass look-back kernel with tickets and in block-index order
        for static_order, chain, waves in ((0, 0, 0), (0, 0, 4), (0, 1, 0), (1, 1, 0)):
            if static_order and n > part + 1:
                continue  # block-index order: the smaller cases are enough (the emulator runs blocks in that order anyway)
            emu.emu_set_option(b"static_order", static_order)
            emu.emu_set_option(b"by_key_reduce_chain", chain)
            emu.emu_set_option(b"by_key_waves", waves)
            d_keys, d_x = copy_in(keys, kt), copy_in(x)
            need = sz(0)
            if chain:  # the scan has the one form: once with tickets, once in block-index order
                assert emu.emu_seg_scan_by_key_f16(None, None, None, n, bits, None, ctypes.byref(need)) == 0
                ws = aligned(need.value, np.uint8, 0xAB)
                out = aligned(n, np.uint16, 0xFFFF)
                assert emu.emu_seg_scan_by_key_f16(d_keys.ctypes.data, d_x.ctypes.data, out.ctypes.data, n, bits, ws.ctypes.data, ctypes.byref(need)) == 0, emu.emu_last_error()
                assert np.array_equal(out, want_scan), (n, mean_run, static_order, chain)
                # in place
                assert emu.emu_seg_scan_by_key_f16(d_keys.ctypes.data, d_x.ctypes.data, d_x.ctypes.data, n, bits, ws.ctypes.data, ctypes.byref(need)) == 0
                assert np.array_equal(d_x[:n], want_scan)
                d_x = copy_in(x)
            assert emu.emu_seg_reduce_by_key_f16(None, None, None, None, None, n, bits, None, ctypes.byref(need)) == 0
            ws = aligned(need.value, np.uint8, 0xCD)
            sums, keys_out, runs = aligned(n, np.uint16, 0xFFFF), aligned(n, kt, -1), aligned(1, np.uint64, 99)
            assert emu.emu_seg_reduce_by_key_f16(d_keys.ctypes.data, d_x.ctypes.data, keys_out.ctypes.data, sums.ctypes.data, runs.ctypes.data, n, bits, ws.ctypes.data, ctypes.byref(need)) == 0, emu.emu_last_error()
            r = int(runs[0])
            assert r == want_keys.size, (n, mean_run)
            assert np.array_equal(sums[:r], want_sums) and np.array_equal(keys_out[:r], want_keys.astype(kt))
            assert np.all(sums[r:] == 0xFFFF)  # nothing written past the runs
            # without the keys
            sums2 = aligned(n, np.uint16, 0xFFFF)
            assert emu.emu_seg_reduce_by_key_f16(d_keys.ctypes.data, d_x.ctypes.data, None, sums2.ctypes.data, None, n, bits, ws.ctypes.data, ctypes.byref(need)) == 0, emu.emu_last_error()
            assert np.array_equal(sums2, sums)
    emu.emu_set_option(b"static_order", 0)
    emu.emu_set_option(b"by_key_reduce_chain", 0)
    emu.emu_set_option(b"by_key_waves", 0)
    # empty input: no launch needed, the run count is cleared
    need, runs = sz(1 << 20), aligned(1, np.uint64, 99)
    ws = aligned(1 << 12, np.uint8)
    assert emu.emu_seg_reduce_by_key_f16(None, None, None, None, runs.ctypes.data, 0, bits, ws.ctypes.data, ctypes.byref(need)) == 0
    assert runs[0] == 0
    assert emu.emu_seg_scan_by_key_f16(None, None, None, 8, 48, ws.ctypes.data, ctypes.byref(need)) == 1  # key width
