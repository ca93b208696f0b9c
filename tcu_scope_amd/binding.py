"""ctypes binding of libtcu_scope_amd.so; every function takes torch CUDA tensors and
launches on torch's current stream unless told otherwise."""
import ctypes
import enum
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.environ.get("TCU_SCOPE_AMD_LIBRARY") or os.path.join(_HERE, "libtcu_scope_amd.so")
_CSRC = os.path.join(_HERE, "csrc")

EXPORTS = [
    "tcu_abi_version", "tcu_last_error", "tcu_init", "tcu_device_info", "tcu_set_option",
    "tcu_seg_reduce_f16", "tcu_seg_reduce_offsets_f16", "tcu_seg_scan_f16", "tcu_seg_scan_f16_noalloc", "tcu_seg_scan_offsets_f16", "tcu_seg_scan_by_key_f16", "tcu_seg_reduce_by_key_f16", "tcu_add_partial_sums_f16",
    "tcu_full_reduce_f16", "tcu_full_scan_f16", "tcu_gemv_f16_f32", "tcu_gemm_f16_f32", "tcu_gemv_f16_f16", "tcu_gemm_f16_f16", "tcu_gemv_col_major_f16_f32", "tcu_gemv_col_major_f16_f16",
    "tcu_fill_f16", "tcu_convert_f32_to_f16", "tcu_generate_f16", "tcu_stream_probe", "tcu_time_next_launch", "tcu_lane_probe", "tcu_temporary_allocations",
]


class Variant(enum.IntEnum):
    AUTO = 0
    MFMA_16 = 1
    MFMA_16N = 2
    MFMA_16N_BLOCK = 3
    MFMA_256 = 4
    MFMA_256N = 5
    MFMA_256N_BLOCK = 6
    WAVE_SHUFFLE = 7
    BLOCK_LDS = 8


VARIANTS = list(Variant)


class FullStrategy(enum.IntEnum):
    AUTO = 0
    SINGLE_PASS = 1
    MULTI_KERNEL = 2


# flag OR-ed onto a FullStrategy: the single-pass full-array kernels work on the matrix unit
FULL_MFMA = 0x100


class Dist(enum.IntEnum):
    UNIFORM = 0
    GRID = 1
    NORMAL = 2
    SMALLINT = 3


class TcuError(RuntimeError):
    """A non-zero tcu_status; .status is 1 invalid argument, 2 unsupported, 3 runtime, 4 workspace."""

    def __init__(self, status, message):
        super().__init__(f"tcu_status {status}: {message}")
        self.status = status


def library_path():
    return _LIB


def build():
    """Compile the HIP sources for gfx950 into libtcu_scope_amd.so (needs hipcc, no GPU)."""
    subprocess.check_call(["make", "-C", _CSRC, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _CSRC], stdout=subprocess.DEVNULL)
    return _LIB


_lib = None


def lib():
    """The loaded shared library.  Raises when it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise ImportError(f"{_LIB} is missing: build it with `make -C {_CSRC}` (python -c 'import __graft_entry__ as g; g.build()')")
        L = ctypes.CDLL(_LIB)
        c = ctypes
        vp, sz, ci, cf = c.c_void_p, c.c_size_t, c.c_int, c.c_float
        L.tcu_abi_version.restype = ci
        L.tcu_last_error.restype = c.c_char_p
        L.tcu_init.argtypes = [ci]
        L.tcu_device_info.argtypes = [c.POINTER(ci)] * 4
        L.tcu_set_option.argtypes = [c.c_char_p, ci]
        L.tcu_seg_reduce_f16.argtypes = [vp, vp, sz, sz, ci, ci, ci, vp]
        L.tcu_seg_reduce_offsets_f16.argtypes = [vp, vp, sz, vp, vp, ci, sz, vp]
        L.tcu_seg_scan_f16.argtypes = [vp, vp, vp, sz, sz, ci, ci, ci, vp]
        L.tcu_seg_scan_f16_noalloc.argtypes = [vp, vp, vp, sz, sz, ci, ci, ci, vp]
        L.tcu_seg_scan_offsets_f16.argtypes = [vp, vp, sz, vp, vp, ci, sz, vp]
        L.tcu_seg_scan_by_key_f16.argtypes = [vp, vp, vp, sz, ci, vp, c.POINTER(sz), vp]
        L.tcu_seg_reduce_by_key_f16.argtypes = [vp, vp, vp, vp, vp, sz, ci, vp, c.POINTER(sz), vp]
        L.tcu_add_partial_sums_f16.argtypes = [vp, vp, sz, sz, vp]
        L.tcu_full_reduce_f16.argtypes = [vp, vp, sz, vp, c.POINTER(sz), ci, sz, ci, vp]
        L.tcu_full_scan_f16.argtypes = [vp, vp, sz, vp, c.POINTER(sz), ci, sz, ci, vp]
        L.tcu_gemv_f16_f32.argtypes = [vp, vp, vp, sz, sz, cf, cf, ci, vp]
        L.tcu_gemm_f16_f32.argtypes = [vp, vp, vp, vp, sz, sz, sz, cf, cf, ci, vp]
        L.tcu_gemv_f16_f16.argtypes = [vp, vp, vp, sz, sz, cf, cf, ci, vp]
        L.tcu_gemv_col_major_f16_f32.argtypes = [vp, sz, vp, vp, sz, sz, cf, cf, vp]
        L.tcu_gemv_col_major_f16_f16.argtypes = [vp, sz, vp, vp, sz, sz, cf, cf, vp]
        L.tcu_gemm_f16_f16.argtypes = [vp, vp, vp, vp, sz, sz, sz, cf, cf, ci, vp]
        L.tcu_fill_f16.argtypes = [vp, cf, sz, vp]
        L.tcu_convert_f32_to_f16.argtypes = [vp, vp, sz, vp]
        L.tcu_generate_f16.argtypes = [vp, sz, c.c_uint64, ci, sz, vp]
        L.tcu_stream_probe.argtypes = [vp, vp, sz, ci, ci, ci, vp]
        L.tcu_lane_probe.argtypes = [vp, c.POINTER(sz), vp]
        L.tcu_time_next_launch.argtypes = [vp, vp]
        L.tcu_temporary_allocations.argtypes = []
        L.tcu_temporary_allocations.restype = c.c_ulong
        for name in EXPORTS:
            if name not in ("tcu_last_error", "tcu_temporary_allocations"):
                getattr(L, name).restype = ci
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise TcuError(rc, lib().tcu_last_error().decode())


def _torch():
    import torch

    return torch


def _stream(stream):
    torch = _torch()
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _need_f16(t, name):
    torch = _torch()
    if t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous CUDA float16 tensor")


def init(device_id=0):
    _check(lib().tcu_init(device_id))


def device_info():
    vals = [ctypes.c_int() for _ in range(4)]
    _check(lib().tcu_device_info(*[ctypes.byref(v) for v in vals]))
    return {"compute_units": vals[0].value, "wavefront_size": vals[1].value, "lds_bytes": vals[2].value, "is_gfx950": bool(vals[3].value)}


def set_option(name, value):
    _check(lib().tcu_set_option(name.encode(), int(value)))


def seg_reduce(x, segment_size, variant=Variant.AUTO, tiles_per_wave=0, waves_per_block=0, out=None, num_segments=None, stream=None):
    """out[j] = sum of x[j*S:(j+1)*S] (fp32 accumulate, fp16 result)."""
    torch = _torch()
    _need_f16(x, "x")
    nseg = (x.numel() // segment_size if segment_size > 0 else 1) if num_segments is None else num_segments
    if out is None:
        out = torch.empty(nseg, dtype=torch.float16, device=x.device)
    _check(lib().tcu_seg_reduce_f16(_ptr(x), _ptr(out), nseg, segment_size, int(variant), tiles_per_wave, waves_per_block, _stream(stream)))
    return out


def seg_reduce_offsets(x, begin, end, expected_segment_size=0, out=None, stream=None):
    """out[j] = sum of x[begin[j]:end[j]] (empty when end[j] <= begin[j]); begin/end are int32 or int64
    device tensors of equal length (two views of one offsets tensor are fine)."""
    torch = _torch()
    _need_f16(x, "x")
    if begin.dtype != end.dtype or begin.dtype not in (torch.int32, torch.int64) or begin.numel() != end.numel():
        raise ValueError("begin and end must be int32 or int64 tensors of the same length")
    if not (begin.is_contiguous() and end.is_contiguous()):
        raise ValueError("begin and end must be contiguous")
    nseg = begin.numel()
    if out is None:
        out = torch.empty(nseg, dtype=torch.float16, device=x.device)
    bits = 32 if begin.dtype == torch.int32 else 64
    _check(lib().tcu_seg_reduce_offsets_f16(_ptr(x), _ptr(out), nseg, _ptr(begin), _ptr(end), bits, expected_segment_size, _stream(stream)))
    return out


def seg_scan(x, segment_size, variant=Variant.AUTO, tiles_per_wave=0, waves_per_block=0, out=None, totals=None, num_segments=None, stream=None):
    """Inclusive prefix sum inside every segment; `totals` (optional tensor) receives the segment totals."""
    torch = _torch()
    _need_f16(x, "x")
    nseg = (x.numel() // segment_size if segment_size > 0 else 1) if num_segments is None else num_segments
    if out is None:
        out = torch.empty(nseg * max(segment_size, 0), dtype=torch.float16, device=x.device)
    _check(lib().tcu_seg_scan_f16(_ptr(x), _ptr(out), _ptr(totals), nseg, segment_size, int(variant), tiles_per_wave, waves_per_block, _stream(stream)))
    return out


def seg_scan_noalloc(x, segment_size, out, variant=Variant.AUTO, tiles_per_wave=0, waves_per_block=0, totals=None, num_segments=None, stream=None):
    """seg_scan through tcu_seg_scan_f16_noalloc: the caller brings `out`, nothing is allocated on the way
    (the look-back path keeps its partition descriptors in an array inside the library's device code)."""
    _need_f16(x, "x")
    _need_f16(out, "out")
    nseg = (x.numel() // segment_size if segment_size > 0 else 1) if num_segments is None else num_segments
    _check(lib().tcu_seg_scan_f16_noalloc(_ptr(x), _ptr(out), _ptr(totals), nseg, segment_size, int(variant), tiles_per_wave, waves_per_block, _stream(stream)))
    return out


def seg_scan_offsets(x, begin, end, expected_segment_size=0, out=None, stream=None):
    """Inclusive prefix sums inside every x[begin[j]:end[j]] (non-overlapping); the rest of `out` is not written."""
    torch = _torch()
    _need_f16(x, "x")
    if begin.dtype != end.dtype or begin.dtype not in (torch.int32, torch.int64) or begin.numel() != end.numel():
        raise ValueError("begin and end must be int32 or int64 tensors of the same length")
    if not (begin.is_contiguous() and end.is_contiguous()):
        raise ValueError("begin and end must be contiguous")
    if out is None:
        out = torch.zeros_like(x)
    bits = 32 if begin.dtype == torch.int32 else 64
    _check(lib().tcu_seg_scan_offsets_f16(_ptr(x), _ptr(out), begin.numel(), _ptr(begin), _ptr(end), bits, expected_segment_size, _stream(stream)))
    return out


def _key_bits(keys):
    torch = _torch()
    if keys.dtype not in (torch.int32, torch.int64) or not keys.is_cuda or not keys.is_contiguous():
        raise ValueError("keys must be a contiguous CUDA int32 or int64 tensor")
    return 32 if keys.dtype == torch.int32 else 64


def seg_scan_by_key(keys, x, out=None, workspace=None, stream=None):
    """Inclusive prefix sums inside runs of equal consecutive keys (thrust::inclusive_scan_by_key)."""
    torch = _torch()
    _need_f16(x, "x")
    bits = _key_bits(keys)
    n = x.numel()
    if keys.numel() != n:
        raise ValueError("keys and x must have the same length")
    if out is None:
        out = torch.empty_like(x)
    need = ctypes.c_size_t(0)
    _check(lib().tcu_seg_scan_by_key_f16(None, None, None, n, bits, None, ctypes.byref(need), None))
    if workspace is None:
        workspace = torch.empty(max(need.value, 256), dtype=torch.uint8, device=x.device)
    have = ctypes.c_size_t(workspace.numel())
    _check(lib().tcu_seg_scan_by_key_f16(_ptr(keys), _ptr(x), _ptr(out), n, bits, _ptr(workspace), ctypes.byref(have), _stream(stream)))
    return out


def seg_reduce_by_key(keys, x, workspace=None, stream=None):
    """One sum per run of equal consecutive keys (thrust::reduce_by_key): returns (keys_out, sums, num_runs tensor);
    the first two have room for x.numel() entries, of which the first num_runs.item() are written."""
    torch = _torch()
    _need_f16(x, "x")
    bits = _key_bits(keys)
    n = x.numel()
    if keys.numel() != n:
        raise ValueError("keys and x must have the same length")
    keys_out = torch.empty_like(keys)
    out = torch.empty_like(x)
    num_runs = torch.zeros(1, dtype=torch.int64, device=x.device)
    need = ctypes.c_size_t(0)
    _check(lib().tcu_seg_reduce_by_key_f16(None, None, None, None, None, n, bits, None, ctypes.byref(need), None))
    if workspace is None:
        workspace = torch.empty(max(need.value, 256), dtype=torch.uint8, device=x.device)
    have = ctypes.c_size_t(workspace.numel())
    _check(lib().tcu_seg_reduce_by_key_f16(_ptr(keys), _ptr(x), _ptr(keys_out), _ptr(out), _ptr(num_runs), n, bits, _ptr(workspace), ctypes.byref(have), _stream(stream)))
    return keys_out, out, num_runs


def add_partial_sums(out, partial_sums, segment_size, stream=None):
    _need_f16(out, "out")
    _need_f16(partial_sums, "partial_sums")
    _check(lib().tcu_add_partial_sums_f16(_ptr(out), _ptr(partial_sums), partial_sums.numel(), segment_size, _stream(stream)))
    return out


def _workspace(fn, x, out, n, strategy, segment_size, waves_per_block, workspace, stream):
    torch = _torch()
    need = ctypes.c_size_t(0)
    _check(fn(_ptr(x), None, n, None, ctypes.byref(need), int(strategy), segment_size, waves_per_block, _stream(stream)))
    if workspace is None:
        workspace = torch.empty(max(need.value, 256), dtype=torch.uint8, device=x.device)
    have = ctypes.c_size_t(workspace.numel() * workspace.element_size())
    _check(fn(_ptr(x), _ptr(out), n, _ptr(workspace), ctypes.byref(have), int(strategy), segment_size, waves_per_block, _stream(stream)))
    return workspace


def full_reduce(x, strategy=FullStrategy.AUTO, segment_size=0, waves_per_block=0, out=None, workspace=None, stream=None):
    torch = _torch()
    _need_f16(x, "x")
    if out is None:
        out = torch.empty(1, dtype=torch.float16, device=x.device)
    _workspace(lib().tcu_full_reduce_f16, x, out, x.numel(), strategy, segment_size, waves_per_block, workspace, stream)
    return out


def full_scan(x, strategy=FullStrategy.AUTO, segment_size=0, waves_per_block=0, out=None, workspace=None, stream=None):
    torch = _torch()
    _need_f16(x, "x")
    if out is None:
        out = torch.empty_like(x)
    _workspace(lib().tcu_full_scan_f16, x, out, x.numel(), strategy, segment_size, waves_per_block, workspace, stream)
    return out


def full_workspace_bytes(kind, n, strategy=FullStrategy.AUTO, segment_size=0, waves_per_block=0):
    fn = lib().tcu_full_reduce_f16 if kind == "reduce" else lib().tcu_full_scan_f16
    need = ctypes.c_size_t(0)
    _check(fn(None, None, n, None, ctypes.byref(need), int(strategy), segment_size, waves_per_block, None))
    return need.value


def _out_entry(t, what, f32_entry, f16_entry):
    torch = _torch()
    if t.dtype == torch.float32:
        return f32_entry
    if t.dtype == torch.float16:
        return f16_entry
    raise TypeError(f"{what} must be a float32 or float16 tensor")


def gemv(A, x, alpha=1.0, beta=0.0, y=None, variant=Variant.AUTO, stream=None, out_dtype=None):
    """y = alpha*A@x + beta*y; A (M,K) row-major fp16, x (K,) fp16, y (M,) fp32 or fp16.

    The dtype of `y` (or `out_dtype` when y is None; default float32) selects
    tcu_gemv_f16_f32 or tcu_gemv_f16_f16."""
    torch = _torch()
    _need_f16(A, "A")
    _need_f16(x, "x")
    M, K = A.shape
    if y is None:
        y = torch.zeros(M, dtype=out_dtype or torch.float32, device=A.device)
    entry = _out_entry(y, "y", lib().tcu_gemv_f16_f32, lib().tcu_gemv_f16_f16)
    _check(entry(_ptr(A), _ptr(x), _ptr(y), M, K, alpha, beta, int(variant), _stream(stream)))
    return y


def gemv_col_major(At, x, alpha=1.0, beta=0.0, y=None, stream=None, out_dtype=None):
    """y = alpha*A@x + beta*y with A column-major: `At` is the (K, M) fp16 tensor whose row k is column k of A (rows may be
    further apart than M elements: lda = At.stride(0)); x (K,) fp16, y (M,) fp32 or fp16 (tcu_gemv_col_major_f16_f32 / _f16)."""
    torch = _torch()
    _need_f16(x, "x")
    if At.dtype != torch.float16 or not At.is_cuda or At.dim() != 2 or At.stride(1) != 1:
        raise ValueError("At must be a CUDA float16 matrix that holds the columns of A contiguously (stride 1 along its second dimension)")
    K, M = At.shape
    if y is None:
        y = torch.zeros(M, dtype=out_dtype or torch.float32, device=At.device)
    entry = _out_entry(y, "y", lib().tcu_gemv_col_major_f16_f32, lib().tcu_gemv_col_major_f16_f16)
    _check(entry(ctypes.c_void_p(At.data_ptr()), At.stride(0) if K > 1 else M, _ptr(x), _ptr(y), M, K, alpha, beta, _stream(stream)))
    return y


def gemm(A, Bt, alpha=1.0, beta=0.0, C=None, out=None, variant=Variant.AUTO, stream=None, out_dtype=None):
    """D = alpha*A@B + beta*C with A (M,K) fp16 and B given column-major, i.e. as Bt (N,K) fp16.

    C and D are float32 (tcu_gemm_f16_f32) or float16 (tcu_gemm_f16_f16): the dtype of `out`,
    else of `C`, else `out_dtype` (default float32)."""
    torch = _torch()
    _need_f16(A, "A")
    _need_f16(Bt, "Bt")
    M, K = A.shape
    N, K2 = Bt.shape
    if K != K2:
        raise ValueError("A and Bt disagree on K")
    if out is None:
        out = torch.empty(M, N, dtype=C.dtype if C is not None else (out_dtype or torch.float32), device=A.device)
    if C is not None and C.dtype != out.dtype:
        raise TypeError("C and out must have the same dtype")
    entry = _out_entry(out, "out", lib().tcu_gemm_f16_f32, lib().tcu_gemm_f16_f16)
    _check(entry(_ptr(A), _ptr(Bt), _ptr(C), _ptr(out), M, N, K, alpha, beta, int(variant), _stream(stream)))
    return out


def fill(t, value, stream=None):
    _need_f16(t, "t")
    _check(lib().tcu_fill_f16(_ptr(t), value, t.numel(), _stream(stream)))
    return t


def convert_f32_to_f16(src, out=None, stream=None):
    torch = _torch()
    if out is None:
        out = torch.empty(src.shape, dtype=torch.float16, device=src.device)
    _check(lib().tcu_convert_f32_to_f16(_ptr(out), _ptr(src), src.numel(), _stream(stream)))
    return out


def generate(n, seed, dist=Dist.UNIFORM, first=0, out=None, device="cuda", stream=None):
    torch = _torch()
    if out is None:
        out = torch.empty(n, dtype=torch.float16, device=device)
    _check(lib().tcu_generate_f16(_ptr(out), n, seed & 0xFFFFFFFFFFFFFFFF, int(dist), first, _stream(stream)))
    return out


def stream_probe(dst, src, nbytes, mode, tiles_per_wave=0, waves_per_block=0, stream=None):
    _check(lib().tcu_stream_probe(_ptr(dst), _ptr(src), nbytes, mode, tiles_per_wave, waves_per_block, _stream(stream)))


def temporary_allocations():
    """How many times the library has taken temporary device memory since the process began."""
    return int(lib().tcu_temporary_allocations())


def time_next_launch(start, stop):
    """The next kernel launched through the library stamps the torch events `start` and `stop`
    (enable_timing=True, already recorded once so that their handles exist) with its own begin
    and end: start.elapsed_time(stop) is then the kernel's duration."""
    _check(lib().tcu_time_next_launch(start.cuda_event, stop.cuda_event))


def lane_probe(device="cuda", stream=None):
    torch = _torch()
    words = ctypes.c_size_t(0)
    _check(lib().tcu_lane_probe(None, ctypes.byref(words), None))
    out = torch.zeros(words.value, dtype=torch.int32, device=device)
    _check(lib().tcu_lane_probe(_ptr(out), ctypes.byref(words), _stream(stream)))
    return out
