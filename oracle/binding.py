"""ctypes binding of the CPU oracle (test infrastructure only).

Only tests, the smoke check and the CPU-baseline leg of the benchmark import this
module; the GPU library and its Python mirror never do.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtcu_oracle.so")

DIST_UNIFORM, DIST_GRID, DIST_NORMAL, DIST_SMALLINT = 0, 1, 2, 3


def build(force=False):
    """Compile oracle/tcu_oracle.c with gcc (make)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        u16p, f64p, f32p = c.POINTER(c.c_uint16), c.POINTER(c.c_double), c.POINTER(c.c_float)
        sz = c.c_size_t
        L.tcu_oracle_f16_to_f32.restype = c.c_float
        L.tcu_oracle_f16_to_f32.argtypes = [c.c_uint16]
        L.tcu_oracle_f32_to_f16.restype = c.c_uint16
        L.tcu_oracle_f32_to_f16.argtypes = [c.c_float]
        L.tcu_oracle_f64_to_f16.restype = c.c_uint16
        L.tcu_oracle_f64_to_f16.argtypes = [c.c_double]
        L.tcu_oracle_ulp_f16.restype = c.c_double
        L.tcu_oracle_ulp_f16.argtypes = [c.c_double]
        L.tcu_oracle_splitmix64.restype = c.c_uint64
        L.tcu_oracle_splitmix64.argtypes = [c.c_uint64, c.c_uint64]
        L.tcu_oracle_generate_f16.argtypes = [u16p, sz, c.c_uint64, c.c_int]
        L.tcu_oracle_generate_f16_range.argtypes = [u16p, sz, sz, c.c_uint64, c.c_int]
        L.tcu_oracle_fill_f16.argtypes = [u16p, c.c_float, sz]
        L.tcu_oracle_convert_f32_to_f16.argtypes = [u16p, f32p, sz]
        for name in ("seg_reduce_ref", "seg_scan_ref"):
            getattr(L, "tcu_oracle_" + name).argtypes = [u16p, u16p, sz, sz]
            getattr(L, "tcu_oracle_" + name + "_mt").argtypes = [u16p, u16p, sz, sz, c.c_int]
        L.tcu_oracle_full_reduce_ref.argtypes = [u16p, u16p, sz]
        L.tcu_oracle_full_scan_ref.argtypes = [u16p, u16p, sz]
        L.tcu_oracle_add_partial_sums_ref.argtypes = [u16p, u16p, sz, sz]
        L.tcu_oracle_seg_reduce_f64.argtypes = [u16p, f64p, sz, sz]
        i64p = c.POINTER(c.c_int64)
        L.tcu_oracle_seg_reduce_offsets_ref.argtypes = [u16p, u16p, sz, i64p, i64p]
        L.tcu_oracle_seg_reduce_offsets_f64.argtypes = [u16p, f64p, sz, i64p, i64p]
        L.tcu_oracle_seg_scan_offsets_ref.argtypes = [u16p, u16p, sz, i64p, i64p]
        L.tcu_oracle_seg_scan_offsets_f64.argtypes = [u16p, f64p, sz, i64p, i64p]
        L.tcu_oracle_seg_scan_f64.argtypes = [u16p, f64p, sz, sz]
        L.tcu_oracle_seg_scan_by_key_ref.argtypes = [i64p, u16p, u16p, sz]
        L.tcu_oracle_seg_scan_by_key_f64.argtypes = [i64p, u16p, f64p, sz]
        L.tcu_oracle_seg_reduce_by_key_ref.restype = sz
        L.tcu_oracle_seg_reduce_by_key_ref.argtypes = [i64p, u16p, i64p, u16p, sz]
        L.tcu_oracle_seg_reduce_by_key_f64.restype = sz
        L.tcu_oracle_seg_reduce_by_key_f64.argtypes = [i64p, u16p, i64p, f64p, sz]
        L.tcu_oracle_gemv_f64.argtypes = [u16p, u16p, f32p, f64p, sz, sz, c.c_double, c.c_double]
        L.tcu_oracle_gemm_f64.argtypes = [u16p, u16p, f32p, f64p, sz, sz, sz, c.c_double, c.c_double, sz, sz]
        L.tcu_oracle_check_f16.restype = sz
        L.tcu_oracle_check_f16.argtypes = [u16p, f64p, sz, c.c_double, c.c_double, sz, f64p, c.POINTER(sz)]
        L.tcu_oracle_check_f32_rel.restype = sz
        L.tcu_oracle_check_f32_rel.argtypes = [f32p, f64p, sz, c.c_double, c.c_double, f64p, c.POINTER(sz)]
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def _u16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16
    return a


def f16_to_f32(h):
    return lib().tcu_oracle_f16_to_f32(int(h))


def f32_to_f16(f):
    return lib().tcu_oracle_f32_to_f16(float(np.float32(f)))


def f32_to_f16_array(values):
    """Element-wise float32 -> fp16 bit patterns (the reference's convertFp32ToFp16)."""
    a = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().tcu_oracle_convert_f32_to_f16(_p(out, ctypes.c_uint16), _p(a, ctypes.c_float), a.size)
    return out


def f64_to_f16(d):
    return lib().tcu_oracle_f64_to_f16(float(d))


def ulp_f16(v):
    return lib().tcu_oracle_ulp_f16(float(v))


def splitmix64(seed, i):
    return lib().tcu_oracle_splitmix64(seed & 0xFFFFFFFFFFFFFFFF, i)


_THREADS = min(16, os.cpu_count() or 1)
_PAR_MIN = 1 << 22


def _split(n_items, fn):
    """Runs fn(lo, hi) over contiguous pieces of range(n_items) on a few threads (the C
    functions release the GIL; every piece is computed independently, so results do not
    depend on the split)."""
    from concurrent.futures import ThreadPoolExecutor

    t = _THREADS
    bounds = [n_items * i // t for i in range(t + 1)]
    with ThreadPoolExecutor(t) as ex:
        list(ex.map(lambda i: fn(bounds[i], bounds[i + 1]), range(t)))


def generate_f16(n, seed, dist=DIST_UNIFORM, first=0):
    """n fp16 bit patterns (uint16) of the counter-based generator."""
    out = np.empty(n, dtype=np.uint16)
    L = lib()
    seed &= 0xFFFFFFFFFFFFFFFF
    if n >= _PAR_MIN:
        _split(n, lambda lo, hi: L.tcu_oracle_generate_f16_range(_p(out[lo:hi], ctypes.c_uint16), first + lo, hi - lo, seed, dist))
    else:
        L.tcu_oracle_generate_f16_range(_p(out, ctypes.c_uint16), first, n, seed, dist)
    return out


def fill_f16(n, value):
    out = np.empty(n, dtype=np.uint16)
    lib().tcu_oracle_fill_f16(_p(out, ctypes.c_uint16), value, n)
    return out


def seg_reduce_ref(x, num_segments, segment_size, nthreads=1):
    x = _u16(x)
    assert x.size >= num_segments * segment_size
    out = np.empty(num_segments, dtype=np.uint16)
    if nthreads == 1:
        lib().tcu_oracle_seg_reduce_ref(_p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), num_segments, segment_size)
    else:
        lib().tcu_oracle_seg_reduce_ref_mt(_p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), num_segments, segment_size, nthreads)
    return out


def seg_scan_ref(x, num_segments, segment_size, nthreads=1):
    x = _u16(x)
    assert x.size >= num_segments * segment_size
    out = np.empty(num_segments * segment_size, dtype=np.uint16)
    if nthreads == 1:
        lib().tcu_oracle_seg_scan_ref(_p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), num_segments, segment_size)
    else:
        lib().tcu_oracle_seg_scan_ref_mt(_p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), num_segments, segment_size, nthreads)
    return out


def full_reduce_ref(x):
    x = _u16(x)
    out = np.empty(1, dtype=np.uint16)
    lib().tcu_oracle_full_reduce_ref(_p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), x.size)
    return out


def full_scan_ref(x):
    x = _u16(x)
    out = np.empty(x.size, dtype=np.uint16)
    lib().tcu_oracle_full_scan_ref(_p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), x.size)
    return out


def add_partial_sums_ref(out, partial_sums, num_segments, segment_size):
    out = _u16(out).copy()
    ps = _u16(partial_sums)
    lib().tcu_oracle_add_partial_sums_ref(_p(out, ctypes.c_uint16), _p(ps, ctypes.c_uint16), num_segments, segment_size)
    return out


def seg_reduce_f64(x, num_segments, segment_size):
    x = _u16(x)
    assert x.size >= num_segments * segment_size
    out = np.empty(num_segments, dtype=np.float64)
    L, S = lib(), segment_size
    if num_segments * S >= _PAR_MIN and num_segments >= 64:
        _split(num_segments, lambda lo, hi: L.tcu_oracle_seg_reduce_f64(_p(x[lo * S:], ctypes.c_uint16), _p(out[lo:], ctypes.c_double), hi - lo, S))
    else:
        L.tcu_oracle_seg_reduce_f64(_p(x, ctypes.c_uint16), _p(out, ctypes.c_double), num_segments, S)
    return out


def _offsets(x, begin, end):
    begin = np.ascontiguousarray(begin, dtype=np.int64)
    end = np.ascontiguousarray(end, dtype=np.int64)
    assert begin.shape == end.shape and begin.ndim == 1
    live = end > begin
    assert not live.any() or (begin[live].min() >= 0 and end[live].max() <= x.size)
    return begin, end


def seg_reduce_offsets_ref(x, begin, end):
    """fp32 sequential sum of x[begin[j]:end[j]] per segment, fp16 bits out."""
    x = _u16(x)
    begin, end = _offsets(x, begin, end)
    out = np.empty(begin.size, dtype=np.uint16)
    lib().tcu_oracle_seg_reduce_offsets_ref(_p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), begin.size, _p(begin, ctypes.c_int64), _p(end, ctypes.c_int64))
    return out


def seg_reduce_offsets_f64(x, begin, end):
    x = _u16(x)
    begin, end = _offsets(x, begin, end)
    out = np.empty(begin.size, dtype=np.float64)
    lib().tcu_oracle_seg_reduce_offsets_f64(_p(x, ctypes.c_uint16), _p(out, ctypes.c_double), begin.size, _p(begin, ctypes.c_int64), _p(end, ctypes.c_int64))
    return out


def seg_scan_offsets_ref(x, begin, end, fill=0xFFFF):
    """fp32 running sums inside x[begin[j]:end[j]], fp16 bits; positions outside every segment hold `fill`."""
    x = _u16(x)
    begin, end = _offsets(x, begin, end)
    out = np.full(x.size, fill, dtype=np.uint16)
    lib().tcu_oracle_seg_scan_offsets_ref(_p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), begin.size, _p(begin, ctypes.c_int64), _p(end, ctypes.c_int64))
    return out


def seg_scan_offsets_f64(x, begin, end):
    """fp64 running sums inside every segment; NaN outside every segment."""
    x = _u16(x)
    begin, end = _offsets(x, begin, end)
    out = np.full(x.size, np.nan, dtype=np.float64)
    lib().tcu_oracle_seg_scan_offsets_f64(_p(x, ctypes.c_uint16), _p(out, ctypes.c_double), begin.size, _p(begin, ctypes.c_int64), _p(end, ctypes.c_int64))
    return out


def _keys64(keys):
    return np.ascontiguousarray(keys, dtype=np.int64)


def seg_scan_by_key_ref(keys, x):
    """Inclusive prefix sums inside runs of equal consecutive keys: fp32 running sum, fp16 results (uint16 bit patterns)."""
    k, x = _keys64(keys), _u16(x)
    out = np.empty(x.size, dtype=np.uint16)
    lib().tcu_oracle_seg_scan_by_key_ref(_p(k, ctypes.c_int64), _p(x, ctypes.c_uint16), _p(out, ctypes.c_uint16), x.size)
    return out


def seg_scan_by_key_f64(keys, x):
    k, x = _keys64(keys), _u16(x)
    out = np.empty(x.size, dtype=np.float64)
    lib().tcu_oracle_seg_scan_by_key_f64(_p(k, ctypes.c_int64), _p(x, ctypes.c_uint16), _p(out, ctypes.c_double), x.size)
    return out


def seg_reduce_by_key_ref(keys, x):
    """(keys of the runs, fp16 bit patterns of their sums): fp32 running sum per run."""
    k, x = _keys64(keys), _u16(x)
    ko, out = np.empty(max(x.size, 1), dtype=np.int64), np.empty(max(x.size, 1), dtype=np.uint16)
    runs = lib().tcu_oracle_seg_reduce_by_key_ref(_p(k, ctypes.c_int64), _p(x, ctypes.c_uint16), _p(ko, ctypes.c_int64), _p(out, ctypes.c_uint16), x.size)
    return ko[:runs].copy(), out[:runs].copy()


def seg_reduce_by_key_f64(keys, x):
    k, x = _keys64(keys), _u16(x)
    ko, out = np.empty(max(x.size, 1), dtype=np.int64), np.empty(max(x.size, 1), dtype=np.float64)
    runs = lib().tcu_oracle_seg_reduce_by_key_f64(_p(k, ctypes.c_int64), _p(x, ctypes.c_uint16), _p(ko, ctypes.c_int64), _p(out, ctypes.c_double), x.size)
    return ko[:runs].copy(), out[:runs].copy()


def seg_scan_f64(x, num_segments, segment_size):
    x = _u16(x)
    assert x.size >= num_segments * segment_size
    out = np.empty(num_segments * segment_size, dtype=np.float64)
    L, S = lib(), segment_size
    if num_segments * S >= _PAR_MIN and num_segments >= 64:
        _split(num_segments, lambda lo, hi: L.tcu_oracle_seg_scan_f64(_p(x[lo * S:], ctypes.c_uint16), _p(out[lo * S:], ctypes.c_double), hi - lo, S))
    else:
        L.tcu_oracle_seg_scan_f64(_p(x, ctypes.c_uint16), _p(out, ctypes.c_double), num_segments, S)
    return out


def gemv_f64(A, x, M, K, alpha=1.0, beta=0.0, y0=None):
    A, x = _u16(A), _u16(x)
    y = np.empty(M, dtype=np.float64)
    y0p = None
    if y0 is not None:
        y0 = np.ascontiguousarray(y0, dtype=np.float32)
        y0p = _p(y0, ctypes.c_float)
    lib().tcu_oracle_gemv_f64(_p(A, ctypes.c_uint16), _p(x, ctypes.c_uint16), y0p, _p(y, ctypes.c_double), M, K, alpha, beta)
    return y


def gemm_f64(A, B, M, N, K, alpha=1.0, beta=0.0, C=None, row0=0, rows=None):
    """A: M x K row-major, B: K x N column-major (stored as N rows of K), C: M x N row-major."""
    A, B = _u16(A), _u16(B)
    rows = M - row0 if rows is None else rows
    D = np.empty(rows * N, dtype=np.float64)
    Cp = None
    if C is not None:
        C = np.ascontiguousarray(C, dtype=np.float32)
        Cp = _p(C, ctypes.c_float)
    lib().tcu_oracle_gemm_f64(_p(A, ctypes.c_uint16), _p(B, ctypes.c_uint16), Cp, _p(D, ctypes.c_double), M, N, K, alpha, beta, row0, rows)
    return D.reshape(rows, N)


def check_f16(got, ref, segment_size, ulps=2.0, abs_per_sqrt=1e-3):
    """Tolerance rule |got-ref| <= ulps*ulp16(ref) + abs_per_sqrt*sqrt(segment_size).

    Returns (violations, worst_excess, first_bad_index)."""
    got = _u16(got).ravel()
    ref = np.ascontiguousarray(ref, dtype=np.float64).ravel()
    assert got.size == ref.size, (got.size, ref.size)
    L = lib()
    if got.size >= _PAR_MIN:
        res = []

        def piece(lo, hi):
            w, f = ctypes.c_double(), ctypes.c_size_t()
            b = L.tcu_oracle_check_f16(_p(got[lo:hi], ctypes.c_uint16), _p(ref[lo:hi], ctypes.c_double), hi - lo, ulps, abs_per_sqrt, segment_size, ctypes.byref(w), ctypes.byref(f))
            res.append((b, w.value, lo + f.value if b else got.size))

        _split(got.size, piece)
        return sum(r[0] for r in res), max(r[1] for r in res), min(r[2] for r in res)
    worst = ctypes.c_double()
    fb = ctypes.c_size_t()
    bad = L.tcu_oracle_check_f16(_p(got, ctypes.c_uint16), _p(ref, ctypes.c_double), got.size, ulps, abs_per_sqrt, segment_size, ctypes.byref(worst), ctypes.byref(fb))
    return bad, worst.value, fb.value


def check_f32_rel(got, ref, rel, scale):
    got = np.ascontiguousarray(got, dtype=np.float32).ravel()
    ref = np.ascontiguousarray(ref, dtype=np.float64).ravel()
    assert got.size == ref.size
    worst = ctypes.c_double()
    fb = ctypes.c_size_t()
    bad = lib().tcu_oracle_check_f32_rel(_p(got, ctypes.c_float), _p(ref, ctypes.c_double), got.size, rel, scale, ctypes.byref(worst), ctypes.byref(fb))
    return bad, worst.value, fb.value
