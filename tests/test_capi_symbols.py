"""The C-ABI library loads and exports every symbol include/dlfx.h declares
(no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

from dlf_amd import hip_backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "dlfx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dlfx_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_agree():
    assert declared_symbols() == sorted(hip_backend.EXPORTS)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(hip_backend.LIB_PATH), "run __graft_entry__.build() first"
    lib = ctypes.CDLL(hip_backend.LIB_PATH)
    for name in declared_symbols():
        assert getattr(lib, name) is not None


def test_host_only_calls():
    lib = hip_backend.load_library()
    assert lib.dlfx_version() >= 100
    assert lib.dlfx_status_string(0) == b"ok"
    assert b"scratch" in lib.dlfx_status_string(-4)
    # scratch queries are pure host arithmetic
    assert lib.dlfx_scan_scratch_bytes(0, 64, 1 << 20) > 0
    assert lib.dlfx_scan_scratch_bytes(0, 64, 100) == 0
    assert 0 < lib.dlfx_top_k_scratch_bytes(0, 4096, 32000, 256) <= 4096 * (4096 * 8 + 4) + 1024
    assert lib.dlfx_top_k_scratch_bytes(0, 256, 1000, 5) <= 1024
    # rows longer than the selection kernel takes: winners of 16 segments per row, far below a full argsort
    assert 0 < lib.dlfx_top_k_scratch_bytes(0, 8, 1 << 20, 5) < 8 * (1 << 20)
    # limits the selection does not take still need room for the argsort
    assert lib.dlfx_top_k_scratch_bytes(0, 8, 1 << 20, 5000) > 8 * (1 << 20) * 8
    # the softmax family needs scratch only for few rows that are too long for one workgroup's registers
    assert lib.dlfx_softmax_scratch_bytes(0, 4096, 32000) == 0
    assert lib.dlfx_softmax_scratch_bytes(0, 8, 32768) == 0
    assert 0 < lib.dlfx_softmax_scratch_bytes(0, 8, 262144) <= 8 * 32 * 32
    assert lib.dlfx_softmax_scratch_bytes(1, 8, 20000) > 0
    assert lib.dlfx_softmax_scratch_bytes(0, 255, 262144) > 0
    assert lib.dlfx_softmax_scratch_bytes(0, 256, 262144) == 0
    assert lib.dlfx_softmax_scratch_bytes(2, 8, 262144) > 0            # hardmax of int32
    assert lib.dlfx_softmax_scratch_bytes(5, 8, 262144) == 0           # no int16 softmax family
    # long rows on the bucket route: one pair of ping-pong buffers (with indices: at most 1.6 x the input)
    keys = 256 * (1 << 20) * 8
    assert keys <= lib.dlfx_sort_scratch_bytes(3, 256, 1 << 20) < int(1.1 * keys)
    assert keys + keys // 2 <= lib.dlfx_argsort_scratch_bytes(3, 256, 1 << 20) <= int(1.6 * keys)
    # 16-bit keys keep the digit passes and both pairs
    assert lib.dlfx_sort_scratch_bytes(5, 64, 1 << 16) >= 2 * 64 * (1 << 16) * 2
    assert lib.dlfx_set_tuning(b"no_such_knob", 1) == -3
    assert lib.dlfx_set_tuning(b"scan_poll_limit", 2048) == 0
    for knob, value in ((b"sort_poll_limit", 2048), (b"sort_wave_rows", 512), (b"sort_buckets", 1), (b"sort_compare_max", 32), (b"topk_thread_rows", 256),
                        (b"topk_cols_waves", 0), (b"scan_cols_per_lane", 0)):
        assert lib.dlfx_set_tuning(knob, value) == 0
    assert lib.dlfx_set_tuning(b"sort_wave_rows", 100000) == -3
    assert lib.dlfx_set_tuning(b"topk_cols_waves", 3) == -3 and lib.dlfx_set_tuning(b"scan_cols_per_lane", 4) == -3


def test_argument_errors_are_reported_without_a_gpu():
    lib = hip_backend.load_library()
    dims = (ctypes.c_int64 * 2)(4, 8)
    st = (ctypes.c_int64 * 2)(8, 1)
    one = (ctypes.c_int64 * 1)(4)
    s1 = (ctypes.c_int64 * 1)(1)
    fake = ctypes.c_void_p(0x1000)
    # m * n does not match the view
    assert lib.dlfx_reduce(None, b"reduce_sum", 0, 4, 9, 2, dims, st, fake, 0, 1, one, s1, fake, 0, None, 0) == -1
    assert lib.dlfx_reduce(None, b"nope", 0, 4, 8, 2, dims, st, fake, 0, 1, one, s1, fake, 0, None, 0) == -3
    assert lib.dlfx_reduce(None, b"reduce_sum", 9, 4, 8, 2, dims, st, fake, 0, 1, one, s1, fake, 0, None, 0) == -2
    assert lib.dlfx_reduce(None, b"reduce_sum", 0, 4, 8, 2, dims, st, None, 0, 1, one, s1, fake, 0, None, 0) == -1
    assert lib.dlfx_scan(None, b"cumsum", 0, 4, 7, 0, 2, dims, fake, 0, st, fake, 0, st, None, 0) == -1
    assert lib.dlfx_scan(None, b"cumavg", 0, 4, 8, 0, 2, dims, fake, 0, st, fake, 0, st, None, 0) == -3
    ydims = (ctypes.c_int64 * 2)(4, 9)
    assert lib.dlfx_top_k(None, 9, 1, 0, 2, 2, dims, ydims, fake, 0, st, fake, 0, st, fake, 0, st, None, 0) == -1
    big = (ctypes.c_int64 * 2)(2, 1 << 20)
    bst = (ctypes.c_int64 * 2)(1 << 20, 1)
    assert lib.dlfx_sort(None, 0, 0, 2, big, fake, 0, bst, fake, 0, bst, None, 0) == -4     # scratch missing
