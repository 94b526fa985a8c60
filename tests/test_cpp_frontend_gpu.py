"""Runs the C++ front-end test programs (the thrust:: API over the C ABI) on the GPU.

The programs are built by tests/cpp/Makefile (driven by __graft_entry__.build) with the
plain host compiler (one of them, for user comparators, with hipcc); they replay the reference's literal known-answer vectors and its
host-vs-device differential pattern through device_vector.
"""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "bin")


def _run(name, *args, timeout=300):
    path = os.path.join(BIN, name)
    assert os.path.exists(path), f"{path} is not built (python -c 'import __graft_entry__ as g; g.build()')"
    r = subprocess.run([path, *args], capture_output=True, text=True, timeout=timeout)
    print(r.stdout[-4000:])
    print(r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-4000:]
    return r.stdout


def test_thrust_api_known_answers_and_differential():
    out = _run("test_thrust_api")
    assert "PASSED" in out


def test_containers_and_pointers_as_the_reference_tests_use_them():
    # host_vector / device_vector (construction, assignment across systems, insert, erase, resize, reserve, comparisons
    # with std::vector in either order, reverse iterators, large elements), device_ptr, device_reference
    out = _run("test_containers")
    assert "PASSED" in out


def test_c_abi_from_plain_c():
    out = _run("test_thrust_c11")
    assert "PASS" in out


def test_user_comparators_and_struct_keys_compiled_with_hipcc():
    # thrust::sort with user comparators: the merge sort kernels are instantiated in the test's own translation unit
    out = _run("test_user_comparator")
    assert "PASSED" in out


def test_fancy_iterators_and_user_functors_compiled_with_hipcc():
    # counting / constant / transform / permutation iterators as inputs, transform, for_each, sequence, gather, scatter
    out = _run("test_fancy_iterators")
    assert "PASSED" in out


@pytest.mark.parametrize("log2_n", ["12", "22"])
def test_user_functors_and_library_functors_give_the_same_output(log2_n):
    # every algorithm once with a functor of the caller's own (kernels instantiated in the test's translation unit) and
    # once with the library's (kernels of libthrust_amd.so): sizes and contents must agree; the times it prints are
    # informative only
    out = _run("test_user_functor_paths", log2_n)
    assert "PASSED" in out and "0 mismatches" in out


def test_reference_cases_with_unusual_inputs_and_outputs():
    # bool keys, std::vector / std::list / vector<bool> sources, discard_iterator outputs of the by-key and partition
    # families, zip iterators as partitioned range and as stencil, predicates that return numbers, table-driven
    # operators, elements of 4 to 256 bytes under the default plus
    out = _run("test_reference_cases")
    assert "PASSED" in out


def test_reference_cases_of_sorts_scans_merges_and_set_operations():
    # sorts through permutation iterators and of keys / values up to 1 KiB, keys that use few bits; scan_by_key with
    # head-flag predicates, transform-iterator values, mixed types, discard output, wide values; merges and set operations
    # into discard iterators, descending, on equal ranges and multisets; remove_copy into zip / discard outputs; transform
    # scans from structs, counting iterators and with thrust::identity<> / maximum<>
    out = _run("test_reference_cases_sorts_scans")
    assert "PASSED" in out


def test_placeholder_expressions_as_functors():
    # thrust::placeholders: arithmetic, bitwise, logical, relational, compound assignment and increment forms through
    # thrust::transform on both systems, and as predicates / operators of count_if, copy_if, partition, reduce, inner_product
    out = _run("test_placeholders")
    assert "PASSED" in out


def test_searches_and_extrema():
    # min_element / max_element / minmax_element (first of equivalent extremes), find / find_if / find_if_not,
    # all_of / any_of / none_of, mismatch and equal: the reference's literal vectors on both systems, then the device
    # system against the host system over the size list
    out = _run("test_searches_and_extrema")
    assert "PASSED" in out


def test_elementwise_callers_and_order_checks():
    # is_sorted / is_sorted_until, is_partitioned / partition_point, adjacent_difference (also in place), the replace
    # family with and without stencils, generate(_n), tabulate, reverse(_copy), swap_ranges, uninitialized_fill / _copy:
    # the reference's literal vectors on both systems, then the device system against the host system
    out = _run("test_elementwise_callers")
    assert "PASSED" in out


def test_binary_searches():
    # lower_bound / upper_bound / binary_search / equal_range for one value and for ranges of values, ascending and
    # under thrust::greater: the reference's literal vectors on both systems, then device against host on sorted inputs
    out = _run("test_binary_search")
    assert "PASSED" in out


def test_conditional_forms_and_reverse_iterator():
    # transform_if (input decides / stencil decides / two inputs), gather_if, scatter_if, for_each_n, and
    # thrust::reverse_iterator as input and output of copy, transform, reduce, scan and sort
    out = _run("test_conditional_forms")
    assert "PASSED" in out


def test_random_engines_and_distributions():
    # thrust::random: the 10000th draw of minstd_rand0 / minstd_rand (the standard's validation values) on the host and
    # in device code, discard against drawing, equality, the ranges of uniform_real / uniform_int, normal deviates, and
    # the stream made by one seed-discard-draw functor per element (identical on both sides); the 10000th draw of
    # ranlux24_base, ranlux48_base, ranlux24, ranlux48 and taus88 on both sides; thrust::shuffle / shuffle_copy: a
    # permutation, the same on host and device, the one the reference draws for five elements and seed 2, the generator
    # advanced by sixteen draws, and the Feistel network a bijection of the same images on both sides
    out = _run("test_random")
    assert "PASSED" in out


def test_reference_idioms():
    # what programs written for the reference lean on beside the algorithms: thrust::min / max, distance, the storage
    # calls of thrust/memory.h, transform_input_output_iterator, transform_iterator with named types, device_vector
    # iterators dereferenced inside a functor, fill through a strided view, callables that are not const, unique over
    # tuples, allocators over run-time chosen resources, and the algorithms the vector headers bring along
    out = _run("test_reference_idioms")
    assert "PASSED" in out


def test_bandwidth_ceiling_kernels_run():
    # plain read / write / copy kernels over 1 GiB: the ceiling the library's bandwidth fractions can be read against
    # (profiles/copy_ceiling.txt holds their rocprofv3 durations); here only that they run and give sane rates
    out = _run("bandwidth_ceiling")
    assert "PASSED" in out and "best copy" in out


def test_pass_pattern_ceiling_kernels_run():
    # the memory accesses of one radix-sort pass and nothing else (tiles read in order, written as 256 runs): the
    # ceiling the sort pass can be read against (profiles/scatter_ceiling.txt holds the rocprofv3 durations); every
    # variant is checked to be a permutation of its input
    out = _run("scatter_ceiling")
    assert "PASSED" in out and "NOT A PERMUTATION" not in out and "256 runs of 72 keys" in out

