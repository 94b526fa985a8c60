"""CPU tests of the drop-in boundary: the shared library loads without a GPU and exports
exactly the functions include/thrust_amd.h declares; the Python binding declares them all;
argument validation returns status codes (no compute, no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "thrust_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(thrust_amd_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from thrust_amd import capi
    if not os.path.exists(capi.LIB_PATH):
        from thrust_amd import build
        build.build(verbose=False)
    return capi.load()


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("thrust_amd_reduce", "thrust_amd_inclusive_scan", "thrust_amd_exclusive_scan",
                 "thrust_amd_sort_keys", "thrust_amd_sort_pairs", "thrust_amd_copy_if",
                 "thrust_amd_partition_copy", "thrust_amd_stable_partition", "thrust_amd_unique",
                 "thrust_amd_unique_by_key", "thrust_amd_reduce_by_key", "thrust_amd_merge",
                 "thrust_amd_merge_by_key", "thrust_amd_malloc", "thrust_amd_free", "thrust_amd_memcpy"):
        assert must in names


def test_library_exports_every_declared_symbol(lib):
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in thrust_amd.h but not exported"


def test_binding_covers_every_declared_symbol():
    from thrust_amd import capi
    assert sorted(capi.SIGNATURES) == declared_functions()


def test_metadata_entry_points(lib):
    assert lib.thrust_amd_version() == 100
    sizes = [lib.thrust_amd_dtype_size(d) for d in range(10)]
    assert sizes == [1, 1, 2, 2, 4, 4, 8, 8, 4, 8] and lib.thrust_amd_dtype_size(10) == 0
    assert lib.thrust_amd_error_string(0)


def test_size_queries_and_argument_errors_need_no_gpu(lib):
    """temp == NULL only computes sizes; bad arguments give a non-zero status."""
    n = ctypes.c_size_t(0)
    assert lib.thrust_amd_reduce(None, ctypes.byref(n), None, 1 << 20, 4, 0, None, None, None) == 0 and n.value > 0
    assert lib.thrust_amd_inclusive_scan(None, ctypes.byref(n), None, None, 1 << 20, 4, 0, None) == 0 and n.value > 0
    assert lib.thrust_amd_sort_keys(None, ctypes.byref(n), None, 1 << 20, 5, 0, 0, 32, None) == 0
    assert n.value >= (1 << 20) * 4  # the alternate key buffer lives in temp storage
    assert lib.thrust_amd_merge(None, ctypes.byref(n), None, 10, None, 10, None, 5, 0, None) == 0
    assert lib.thrust_amd_reduce(None, ctypes.byref(n), None, 10, 99, 0, None, None, None) != 0   # bad dtype
    assert lib.thrust_amd_reduce(None, ctypes.byref(n), None, 10, 4, 99, None, None, None) != 0   # bad op
    assert lib.thrust_amd_sort_keys(None, ctypes.byref(n), None, 10, 5, 0, 8, 40, None) != 0       # bad bit range
    assert lib.thrust_amd_sort_keys(None, ctypes.byref(n), None, 1 << 31, 5, 0, 0, 32, None) == 0  # wide descriptors
    assert lib.thrust_amd_sort_keys(None, ctypes.byref(n), None, 1 << 32, 5, 0, 0, 32, None) != 0  # n too large
    assert lib.thrust_amd_copy_if(None, ctypes.byref(n), None, None, None, None, 10, 3, 8, 0, None, None) != 0  # item size
    assert lib.thrust_amd_reduce(None, None, None, 10, 4, 0, None, None, None) != 0                # no size slot


def test_sort_pass_tickets_take_every_tile_once_and_never_get_stuck():
    """tests/cpp/test_sort_tickets.cpp compiles the rule by which the workgroups of a radix-sort pass take
    their tiles (thrust_amd/csrc/sort_tickets.hpp, the function the kernel calls) for the host: every tile
    exactly once for every tile count, and no schedule of two dispatcher models leaves a pass stuck."""
    import subprocess
    cpp = os.path.join(ROOT, "tests", "cpp")
    prog = os.path.join(cpp, "bin", "test_sort_tickets")
    subprocess.run(["make", "-C", cpp, prog], check=True, capture_output=True)
    res = subprocess.run([prog], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0 and "PASSED" in res.stdout, res.stdout + res.stderr

