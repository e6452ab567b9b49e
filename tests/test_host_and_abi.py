"""CPU tests of the host-side C++ mirror and of the C ABI surface of libwarp34_kernels.so.

The host tests are a C++ program (tests/host/kv_host_test.cpp) restating the reference's own
unit tests for this path (crates/warp34-host/src/cache.rs:628-826, model/graph_io.rs:1286);
it is compiled with the host compiler, with address and undefined-behaviour sanitizers, and run here.
The ABI tests check that the shared library loads without a GPU, exports every symbol
the headers under include/ declare, and that the descriptor structs have the sizes the reference
static_asserts (warp34_cuda.h:57,80,101).  No compute entry point is called.
"""
import ctypes as C
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXPECTED_HOST_TESTS = 22  # "ok <name>" lines of tests/host/kv_host_test.cpp


def test_host_mirror_cpp(tmp_path):
    exe = str(tmp_path / "kv_host_test")
    # sanitizer runtimes linked statically: they need no place of their own in the library load order
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-Wall", "-Wextra", "-Werror", "-fsanitize=address,undefined",
           "-static-libasan", "-static-libubsan",
           os.path.join(ROOT, "tests", "host", "kv_host_test.cpp"),
           os.path.join(ROOT, "warp34_amd", "host", "kv_host.cpp"),
           os.path.join(ROOT, "warp34_amd", "host", "prefix_cache.cpp"),
           os.path.join(ROOT, "warp34_amd", "host", "graph_io.cpp"), "-o", exe]
    subprocess.run(cmd, check=True)
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert p.returncode == 0, p.stdout
    oks = [l for l in p.stdout.splitlines() if l.startswith("ok ")]
    assert len(oks) == EXPECTED_HOST_TESTS and "all host tests passed" in p.stdout, p.stdout


def _declared_symbols():
    import glob

    text = "".join(open(h).read() for h in sorted(glob.glob(os.path.join(ROOT, "include", "*.h"))))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(warp34_[a-z0-9_]+)\s*\(", text)))


def _lib_path():
    from warp34_amd import ffi

    path = ffi.LIB_PATH
    if not os.path.exists(path):
        pytest.fail("libwarp34_kernels.so is not built (run __graft_entry__.build())")
    return path


def test_header_and_binding_table_agree():
    from warp34_amd import ffi

    declared = _declared_symbols()
    assert len(declared) >= 20
    assert sorted(ffi.SIGNATURES) == declared


def test_library_loads_and_exports_every_declared_symbol():
    lib = C.CDLL(_lib_path())
    for name in _declared_symbols():
        assert hasattr(lib, name), "missing export " + name
    # the dynamic symbol table holds them as plain C names (no mangling)
    out = subprocess.run(["nm", "-D", "--defined-only", _lib_path()], stdout=subprocess.PIPE, text=True,
                         check=True).stdout
    exported = set(l.split()[-1] for l in out.splitlines() if l.strip())
    assert set(_declared_symbols()) <= exported


def test_descriptor_struct_sizes_and_enums():
    from warp34_amd import ffi

    assert C.sizeof(ffi.Warp34Exec) == 32
    assert C.sizeof(ffi.Warp34KvLayerLayout) == 104
    assert C.sizeof(ffi.Warp34AttentionBatch) == 96
    assert (ffi.WARP34_KV_FORMAT_FP16, ffi.WARP34_KV_FORMAT_BF16, ffi.WARP34_KV_FORMAT_TQ4) == (0, 1, 2)
    assert (ffi.WARP34_KV_TRANSFORM_IDENTITY, ffi.WARP34_KV_TRANSFORM_RADEMACHER_WHT256) == (0, 1)
    # field offsets the kernels rely on (by-value copies of the host structs)
    L, B = ffi.Warp34KvLayerLayout, ffi.Warp34AttentionBatch
    assert L.k_base.offset == 0 and L.v_base.offset == 8 and L.k_page_stride_bytes.offset == 16
    assert B.query_start_loc.offset == 0 and B.block_tables.offset == 24 and B.num_reqs.offset == 56


def test_error_string_needs_no_gpu():
    """warp34_cuda_error_string is a pure lookup: callable on a box without a GPU."""
    from warp34_amd import ffi

    lib = ffi.load()
    s = lib.warp34_cuda_error_string(1)
    assert s and b"invalid" in s.lower()


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU; asked for more it says so and exits without touching a GPU."""
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)
    assert not any(ln.startswith("{") for ln in r.stdout.splitlines())
