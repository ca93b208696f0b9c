"""CPU-side checks of the C ABI: the library loads, exports every symbol the header
declares, and validates arguments without touching a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    import tcu_scope_amd

    if not os.path.exists(tcu_scope_amd.library_path()):
        tcu_scope_amd.build()
    return tcu_scope_amd.lib()


def test_header_and_library_agree(lib):
    import tcu_scope_amd.binding as b

    declared = {}
    for header in ("tcu_scope.h", "tcu_scope_dev.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        declared[header] = set(re.findall(r"\b(tcu_[a-z0-9_]+)\s*\(", text))
    # the reference-facing header carries no tuning switch, test hook or measurement aid
    assert declared["tcu_scope_dev.h"] == {"tcu_set_option", "tcu_stream_probe", "tcu_time_next_launch", "tcu_lane_probe", "tcu_temporary_allocations"}
    assert not (declared["tcu_scope.h"] & declared["tcu_scope_dev.h"])
    assert declared["tcu_scope.h"] | declared["tcu_scope_dev.h"] == set(b.EXPORTS)
    for name in b.EXPORTS:
        assert hasattr(lib, name), name
    # the version the header states is the one the library reports; 2 = the contract with the offsets / by-key /
    # no-alloc entry points and 256-byte look-back descriptors (a workspace size cached from version 1 is too small)
    version = int(re.search(r"#define TCU_SCOPE_ABI_VERSION (\d+)", open(os.path.join(ROOT, "include", "tcu_scope.h")).read()).group(1))
    assert version == 3 and lib.tcu_abi_version() == version


def test_argument_validation_needs_no_gpu(lib):
    sz = ctypes.c_size_t
    err = lambda: lib.tcu_last_error().decode()
    buf = ctypes.create_string_buffer(4096 + 16)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)
    assert lib.tcu_seg_reduce_f16(p, p, 0, 16, 0, 0, 0, None) == 0          # empty: no launch
    assert lib.tcu_seg_reduce_f16(p, p, 4, 0, 0, 0, 0, None) == 1 and "segment_size" in err()
    assert lib.tcu_seg_reduce_f16(p, p, 4, 32, 1, 0, 0, None) == 2 and "must be 16" in err()
    assert lib.tcu_seg_reduce_f16(p, p, 4, 16, 4, 0, 0, None) == 2 and "must be 256" in err()
    assert lib.tcu_seg_reduce_f16(p, p, 4, 16, 99, 0, 0, None) == 1
    assert lib.tcu_seg_reduce_f16(None, p, 4, 16, 0, 0, 0, None) == 1
    assert lib.tcu_seg_scan_f16(p, p, None, 4, 48, 7, 0, 0, None) == 2
    assert lib.tcu_seg_scan_f16(p, p, None, 4, 16, 7, 5, 0, None) == 1
    need = sz(0)
    assert lib.tcu_full_scan_f16(None, None, 1 << 30, None, ctypes.byref(need), 0, 0, 0, None) == 0
    assert need.value == 256 + 256 * ((1 << 30) // 65536)  # one look-back descriptor per 256 bytes
    assert lib.tcu_full_reduce_f16(None, None, 1 << 30, None, ctypes.byref(need), 0, 0, 0, None) == 0 and need.value > 0
    assert lib.tcu_full_reduce_f16(None, None, 1000, None, ctypes.byref(need), 2, 2048, 0, None) == 2  # n % segment_size
    assert lib.tcu_full_scan_f16(None, None, 1 << 20, None, None, 0, 0, 0, None) == 1
    assert lib.tcu_full_scan_f16(None, None, 1 << 20, None, ctypes.byref(need), 0x101, 0, 0, None) == 0  # SINGLE_PASS | MFMA
    assert lib.tcu_full_reduce_f16(None, None, 1 << 20, None, ctypes.byref(need), 0x103, 0, 0, None) == 1 and "strategy" in err()
    assert lib.tcu_gemv_f16_f32(p, p, p, 4, 8, 1.0, 0.0, 6, None) == 2
    assert lib.tcu_gemm_f16_f32(p, p, None, p, 64, 64, 64, 1.0, 0.0, 8, None) == 2  # LDS kernel needs multiples of 128
    assert lib.tcu_gemv_f16_f16(p, p, p, 4, 8, 1.0, 0.0, 6, None) == 2
    assert lib.tcu_gemm_f16_f16(p, p, None, p, 64, 64, 64, 1.0, 0.0, 8, None) == 2
    assert lib.tcu_gemm_f16_f16(p, p, None, p, 64, 64, 64, 1.0, 1.0, 0, None) == 1 and "tcu_gemm_f16_f16" in err()  # beta != 0 needs C
    assert lib.tcu_gemv_f16_f16(None, p, p, 4, 8, 1.0, 0.0, 0, None) == 1 and "tcu_gemv_f16_f16" in err()
    assert lib.tcu_seg_reduce_offsets_f16(p, p, 0, p, p, 32, 0, None) == 0      # no segments: no launch
    assert lib.tcu_seg_reduce_offsets_f16(p, p, 4, p, p, 16, 0, None) == 1 and "offset_bits" in err()
    assert lib.tcu_seg_reduce_offsets_f16(p, p, 4, None, p, 64, 0, None) == 1 and "null" in err()
    for name in (b"static_order", b"scan_lds_tiles", b"gemm_big_tiles", b"gemm_direct_lds", b"gemm_bk64", b"gemm_staged_epilogue", b"gemm_depth", b"gemm_split_tail", b"compute_units", b"gemv_rows", b"gemv_tiles", b"gemv_waves", b"lookback_poll_limit",
                 b"test_mute_partition", b"scan_store_policy", b"by_key_reduce_chain", b"by_key_waves", b"by_key_key_tiles", b"offsets_scan_chain", b"gemv_col_shape", b"gemv_col_blocks"):
        assert lib.tcu_set_option(name, 0) == 0  # every switch the header documents exists
    for name, default in ((b"scan_lds_tiles", -1), (b"gemm_big_tiles", -1), (b"gemm_direct_lds", -1), (b"gemm_depth", 4), (b"gemm_staged_epilogue", 1), (b"gemm_split_tail", 1), (b"compute_units", 256), (b"lookback_poll_limit", -1), (b"scan_store_policy", 2), (b"offsets_scan_chain", 1), (b"gemv_col_shape", 82), (b"gemv_col_blocks", 1024), (b"xcd_run", 7),
                          (b"xcd_run", -1)):
        assert lib.tcu_set_option(name, default) == 0
    assert lib.tcu_set_option(b"no_such_option", 1) == 1
    assert lib.tcu_set_option(b"nontemporal", 1) == 0
    words = sz(0)
    assert lib.tcu_lane_probe(None, ctypes.byref(words), None) == 0 and words.value == 2560


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    import tcu_scope_amd.binding as b

    monkeypatch.setattr(b, "_lib", None)
    monkeypatch.setattr(b, "_LIB", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError):
        b.lib()
