"""The C-ABI library loads without a GPU and exports every function the headers under include/ declare."""
import ctypes
import os
import re

import tvm_amd
from tvm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = "".join(open(os.path.join(ROOT, "include", name)).read() for name in ("tvmkv.h", "tvmkv_dlpack.h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tvmkv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 55
    handle = ctypes.CDLL(tvm_amd.LIB_PATH)
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, f"declared under include/ but not exported: {missing}"


def test_bench_library_exports_every_declared_symbol():
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "tvmkv_bench.h")).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(tvmkvb_[a-z0-9_]+)\s*\(", text)))
    assert names == sorted(_lib.BENCH_SIGNATURES)
    handle = ctypes.CDLL(_lib.BENCH_LIB_PATH)
    assert not [n for n in names if not hasattr(handle, n)]
    product = ctypes.CDLL(tvm_amd.LIB_PATH)
    assert not [n for n in ("tvmkv_mfma_loop", "tvmkv_stream_read", "tvmkv_prefill_clock_probe") if hasattr(product, n)], \
        "measurement aids belong to libtvmkv_bench.so, not to the product library"


def test_scratch_epochs_skip_zero_at_the_wrap():
    """The epoch that tags a launch's arrival counters is the low half of a 64-bit launch count and never 0."""
    from tvm_amd._lib import lib

    fn = lib().tvmkv_debug_next_scratch_epoch
    fn.argtypes = [ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_int32)]
    fn.restype = ctypes.c_uint32
    count, wrapped = ctypes.c_uint64((1 << 32) - 3), ctypes.c_int32(0)
    seen = []
    for _ in range(5):
        seen.append((fn(ctypes.byref(count), ctypes.byref(wrapped)), wrapped.value))
    assert seen == [(0xfffffffe, 0), (0xffffffff, 0), (1, 1), (2, 0), (3, 0)]
    assert count.value == (1 << 32) + 3


def test_python_signatures_cover_the_header():
    names = set(declared_functions()) - {"tvmkv_last_error", "tvmkv_version", "tvmkv_cache_destroy",
                                         "tvmkv_debug_next_scratch_epoch"}
    assert names == set(_lib.SIGNATURES), names ^ set(_lib.SIGNATURES)


def test_version_and_error_channel():
    lib = tvm_amd.lib()
    assert b"gfx950" in lib.tvmkv_version()
    # argument validation happens before any device work, so it can be exercised without a GPU
    rc = lib.tvmkv_batch_decode_paged_kv(None, None, None, None, None, None, None, None, None, 1, 1.0, 1e4, 1.0,
                                         1, 1, 1, 8, 2, 72, 16, 0, None)
    assert rc == -2 and b"multiple of 16, got 72" in lib.tvmkv_last_error()
    rc = lib.tvmkv_batch_decode_paged_kv(None, None, None, None, None, None, None, None, None, 0, 1.0, 1e4, 1.0,
                                         1, 1, 1, 8, 2, 128, 16, 0, None)
    assert rc == -1 and b"NULL tensor" in lib.tvmkv_last_error()
    rc = lib.tvmkv_merge_state_inplace(None, None, None, None, 1, 1, 100, None)
    assert rc == -2 and b"head dim 100" in lib.tvmkv_last_error()
    rc = lib.tvmkv_fused_rope(None, None, None, None, None, 1, 0, 8, 2, 128, 1.0, 1e4, None)
    assert rc == 0  # empty input is a no-op


def test_public_headers_are_plain_c(tmp_path):
    """The boundary is a C ABI: the three public headers compile as C99 and as C++11 on their own, warnings as
    errors (a binding generator -- cgo, JNI, ctypes codegen -- reads them as C)."""
    import shutil
    import subprocess

    src = tmp_path / "headers.c"
    src.write_text('#include "tvmkv.h"\n#include "tvmkv_dlpack.h"\n#include "tvmkv_bench.h"\n'
                   "int main(void) { return tvmkv_version() == 0; }\n")
    include = os.path.join(ROOT, "include")
    flags = ["-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", include]
    if shutil.which("gcc"):
        subprocess.check_call(["gcc", "-std=c99"] + flags + [str(src)])
    if shutil.which("g++"):
        subprocess.check_call(["g++", "-std=c++11", "-x", "c++"] + flags + [str(src)])
