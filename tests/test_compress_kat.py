"""Known-answer tests: the hand-traced tiles of tests/golden/reorder_kat.py
against the C oracle, the Python restatement and the product compressor."""
import numpy as np
import pytest

from golden import reorder_kat as kat
import py_restatement


def _check(case, items, offsets):
    assert list(offsets) == case["offsets"]
    assert [int(x) for x in items] == kat.expected_stream(case)


@pytest.mark.parametrize("name", sorted(kat.CASES))
def test_oracle_reorder_kat(oracle, name):
    case = kat.CASES[name]
    n, items, offsets = oracle.compress_reorder(kat.build_matrix(case))
    assert n == len(case["offsets"])
    _check(case, items, offsets)


@pytest.mark.parametrize("name", sorted(kat.CASES))
def test_python_restatement_kat(name):
    case = kat.CASES[name]
    items, offsets = py_restatement.compress_reorder(kat.build_matrix(case))
    _check(case, items, offsets)


@pytest.mark.parametrize("name", sorted(kat.CASES))
def test_product_reorder_kat(product, name):
    case = kat.CASES[name]
    items, offsets = product.init_sparse_matrix_a(kat.build_matrix(case))
    _check(case, items, offsets)


@pytest.mark.parametrize("name", sorted(kat.NOREORDER_CASES))
def test_noreorder_kat(oracle, product, name):
    case = kat.NOREORDER_CASES[name]
    a = kat.build_matrix(case)
    _, items, offsets = oracle.compress_noreorder(a)
    _check(case, items, offsets)
    items, offsets = product.init_sparse_matrix_a_noreorder(a)
    _check(case, items, offsets)


def test_swizzle_positions_spelled_out():
    case = kat.CASES["swizzle"]
    assert [x >> 16 for x in kat.expected_stream(case)] == case["positions"]
