"""Pins the CPU oracle (oracle/tc_oracle.c) before anything is compared with it.

The reference ships no golden vectors for this path (it has no test suite); its only check is
the nested host loop of post_Correctness() in every driver.  So the oracle is pinned
  1. bit for bit against THOSE loops, compiled from the reference's own driver sources by
     oracle/Makefile (oracle/_ref/*.so; skipped where that directory was not built),
  2. bit for bit against small fixtures written from those loops (tests/golden/, always run),
  3. against numpy einsum on Fortran-ordered arrays, closed forms and a brute-force Python loop,
chosen so that a swapped index, a wrong stride, a dropped term or a wrong sign fails.
"""
import ctypes
import itertools
import json
import os

import numpy as np
import pytest

import helpers
from helpers import parse_expression, uniform, tensor_sizes, ref_lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXPR_DIR = os.path.join(ROOT, "cgo2019-ae_amd", "expressions")
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# distinct small extents per index position, so that a transposed pair of indices changes the result
SMALL = [3, 4, 5, 2, 6, 3, 4]

# the reference's drivers 33 and 34 add although their expression files say "-="
# (cogent/drivers/tccg/code_main_tccg_33.c:132 vs cogent/input_strings/tccg/input_tccg_33.in:4)
DRIVER_OPERATOR = {33: "+=", 34: "+="}


def tccg_expr(n):
    with open(os.path.join(EXPR_DIR, "tccg_%02d.in" % n)) as f:
        return parse_expression(f.read())


def run_reference_loop(lib, dtype, sizes, C, A, B):
    """post_Correctness(h_C, h_C_chk, h_A, h_B, sizes...) accumulates into h_C_chk."""
    dummy = np.zeros_like(C)
    args = [dummy.ctypes.data_as(ctypes.c_void_p), C.ctypes.data_as(ctypes.c_void_p),
            A.ctypes.data_as(ctypes.c_void_p), B.ctypes.data_as(ctypes.c_void_p)] + [ctypes.c_int(s) for s in sizes]
    lib.post_Correctness(*args)
    return C


def inputs(expr, sizes, dtype, c_seeded=True):
    nC, nA, nB = tensor_sizes(expr, sizes)
    A = uniform(nA, 1, dtype)
    B = uniform(nB, 2, dtype)
    C = uniform(nC, 3, dtype) if c_seeded else np.zeros(nC, dtype=dtype)
    return C, A, B


@pytest.mark.parametrize("n", range(1, 49))
def test_oracle_equals_reference_loop_fp64(n, oracle):
    lib = ref_lib("ref_tccg_%02d" % n)
    if lib is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    expr = tccg_expr(n)
    expr["op"] = DRIVER_OPERATOR.get(n, expr["op"])
    sizes = SMALL[:len(expr["all_idx"])]
    C, A, B = inputs(expr, sizes, np.float64)
    want = run_reference_loop(lib, np.float64, sizes, C.copy(), A, B)
    got = oracle.contract(expr, sizes, C.copy(), A, B)
    assert np.array_equal(got, want)
    assert not np.array_equal(got, C)      # something was accumulated


@pytest.mark.parametrize("n", range(40, 49))
def test_oracle_equals_reference_loop_fp32(n, oracle):
    lib = ref_lib("ref_float_tccg_%02d" % n)
    if lib is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    expr = tccg_expr(n)
    sizes = SMALL[:7]
    C, A, B = inputs(expr, sizes, np.float32)
    want = run_reference_loop(lib, np.float32, sizes, C.copy(), A, B)
    got = oracle.contract(expr, sizes, C.copy(), A, B)
    assert got.dtype == np.float32 and np.array_equal(got, want)


SD2_1 = "t3 [h3,4,h2,4,h1,4,p6,4,p5,4,p4,4] -= sum(p7,4) * t2 [p7,p4,h1,h2] * v2 [p7,h3,p6,p5];"


def test_oracle_equals_reference_loop_minus_operator(oracle):
    """cogent/drivers/ccsd_t/code_main_sd2_1.c:562-575: explicit stride tables and '-='."""
    lib = ref_lib("ref_ccsd_sd2_1")
    if lib is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    expr = parse_expression(SD2_1)
    sizes = SMALL[:7]
    C, A, B = inputs(expr, sizes, np.float64)
    chk = C.copy()
    dummy = np.zeros_like(C)
    p = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    lib.post_Correctness(p(dummy), p(chk), *([p(A), p(B)] * 9), *[ctypes.c_int(s) for s in sizes])
    got = oracle.contract(expr, sizes, C.copy(), A, B)
    assert np.array_equal(got, chk)


def golden_cases():
    with open(os.path.join(GOLDEN, "cases.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", golden_cases(), ids=lambda c: c["name"])
def test_oracle_equals_golden_fixture(case, oracle):
    """Fixtures written by tests/golden/make_golden.py from the reference's compiled loops."""
    z = np.load(os.path.join(GOLDEN, case["file"]))
    expr = parse_expression(case["expression"])
    got = oracle.contract(expr, case["sizes"], z["C_in"].copy(), z["A"], z["B"])
    assert got.dtype == z["C_out"].dtype and np.array_equal(got, z["C_out"])


EINSUM_CASES = [
    ("t3 [a,5,b,4,c,3] += sum(d,6) * t2 [b,d,a] * v2 [d,c];", [5, 4, 3, 6]),
    ("t3 [a,3,b,4] += sum(c,5,d,2) * t2 [a,c,d] * v2 [d,b,c];", [3, 4, 5, 2]),
    ("t3 [d,3,c,4,b,2,a,5] -= sum(e,3,f,4) * t2 [c,f,a,e] * v2 [e,b,f,d];", [3, 4, 2, 5, 3, 4]),
    ("t3 [f,2,e,3,d,4,c,2,b,3,a,2] += sum(g,5) * t2 [e,c,a,g] * v2 [d,f,g,b];", [2, 3, 4, 2, 3, 2, 5]),
]


@pytest.mark.parametrize("text,sizes", EINSUM_CASES)
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_oracle_matches_einsum(text, sizes, dtype, oracle):
    expr = parse_expression(text)
    C, A, B = inputs(expr, sizes, dtype)
    got = oracle.contract(expr, sizes, C.copy(), A, B)
    want = helpers.einsum_reference(expr, sizes, C, A, B)
    tol = 1e-13 if dtype == np.float64 else 2e-6
    assert helpers.rel_error(got, want) < tol
    acc64 = oracle.contract_f32_acc64(expr, sizes, C.astype(np.float32), A.astype(np.float32), B.astype(np.float32))
    want32 = helpers.einsum_reference(expr, sizes, C.astype(np.float32), A.astype(np.float32), B.astype(np.float32))
    assert helpers.rel_error(acc64, want32) < 1e-13


def test_oracle_brute_force_python(oracle):
    """Loop nest written out by hand for one 2-contracted-index case, same summation order: bit-exact."""
    text = "t3 [a,3,b,2,c,4] += sum(e,3,d,2) * t2 [a,d,e,c] * v2 [e,b,d];"
    expr = parse_expression(text)
    a_, b_, c_, e_, d_ = sizes = [3, 2, 4, 3, 2]
    C, A, B = inputs(expr, sizes, np.float64)
    want = C.copy()
    for a, b, c in itertools.product(range(a_), range(b_), range(c_)):
        idx = a + a_ * (b + b_ * c)
        for e in range(e_):
            for d in range(d_):
                want[idx] += A[a + a_ * (d + d_ * (e + e_ * c))] * B[e + e_ * (b + b_ * d)]
    got = oracle.contract(expr, sizes, C.copy(), A, B)
    assert np.array_equal(got, want)


def test_oracle_three_contracted_indices_brute_force(oracle):
    """The generic branch (three or more summed indices: an odometer with the FIRST listed index outermost): a loop nest
    written out by hand with that order, distinct extents and the summed indices in different places of the two inputs,
    bit-exact in both element types and for both operators.  A swapped pair of input strides or a reversed odometer
    changes the summation order or the operands and fails the comparison."""
    for op, dtype in (("+=", np.float64), ("-=", np.float64), ("+=", np.float32), ("-=", np.float32)):
        text = "t3 [a,3,b,2] %s sum(e,4,d,2,f,3) * t2 [d,a,f,e] * v2 [f,e,b,d];" % op
        expr = parse_expression(text)
        a_, b_, e_, d_, f_ = sizes = [3, 2, 4, 2, 3]
        C, A, B = inputs(expr, sizes, dtype)
        want = C.copy()
        for a, b in itertools.product(range(a_), range(b_)):
            idx = a + a_ * b
            for e in range(e_):                  # sum() order: e outermost, then d, then f
                for d in range(d_):
                    for f in range(f_):
                        p = A[d + d_ * (a + a_ * (f + f_ * e))] * B[f + f_ * (e + e_ * (b + b_ * d))]
                        want[idx] = want[idx] - p if op == "-=" else want[idx] + p
        got = oracle.contract(expr, sizes, C.copy(), A, B)
        assert got.dtype == dtype and np.array_equal(got, want), (op, dtype)
        # the other summation order (f outermost) gives other bits for at least one element: the check above can tell them apart
        other = C.copy()
        for a, b in itertools.product(range(a_), range(b_)):
            for f in range(f_):
                for d in range(d_):
                    for e in range(e_):
                        p = A[d + d_ * (a + a_ * (f + f_ * e))] * B[f + f_ * (e + e_ * (b + b_ * d))]
                        other[a + a_ * b] = other[a + a_ * b] - p if op == "-=" else other[a + a_ * b] + p
        assert not np.array_equal(other, want)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_oracle_three_and_four_contracted_indices_vs_einsum_and_vs_the_two_index_loop(dtype, oracle):
    """Generic branch against numpy einsum (values) and, with a unit extent added to the sum, against the two-index
    branch that the reference's own loops pin (bits: the unit index adds no term and does not reorder the others)."""
    text3 = "t3 [c,3,a,4,b,2] += sum(d,3,e,2,f,4) * t2 [e,a,d,f] * v2 [b,f,c,d,e];"
    expr3 = parse_expression(text3)
    sizes3 = [3, 4, 2, 3, 2, 4]
    C, A, B = inputs(expr3, sizes3, dtype)
    got = oracle.contract(expr3, sizes3, C.copy(), A, B)
    assert helpers.rel_error(got, helpers.einsum_reference(expr3, sizes3, C, A, B)) < (1e-13 if dtype == np.float64 else 2e-6)
    text4 = "t3 [a,2,b,3] -= sum(d,2,e,3,f,2,g,3) * t2 [g,a,e,d,f] * v2 [f,d,b,g,e];"
    expr4 = parse_expression(text4)
    sizes4 = [2, 3, 2, 3, 2, 3]
    C, A, B = inputs(expr4, sizes4, dtype)
    got = oracle.contract(expr4, sizes4, C.copy(), A, B)
    assert helpers.rel_error(got, helpers.einsum_reference(expr4, sizes4, C, A, B)) < (1e-13 if dtype == np.float64 else 2e-6)
    # sum(e, u, d) with extent(u) = 1 in either input  ==  sum(e, d), bit for bit
    two = parse_expression("t3 [a,3,b,2,c,4] += sum(e,3,d,2) * t2 [a,d,e,c] * v2 [e,b,d];")
    three = parse_expression("t3 [a,3,b,2,c,4] += sum(e,3,u,1,d,2) * t2 [a,u,d,e,c] * v2 [e,b,d,u];")
    C, A, B = inputs(two, [3, 2, 4, 3, 2], dtype)
    assert np.array_equal(oracle.contract(three, [3, 2, 4, 3, 1, 2], C.copy(), A, B), oracle.contract(two, [3, 2, 4, 3, 2], C.copy(), A, B))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_oracle_without_contracted_index_is_the_outer_product(dtype, oracle):
    """No summed index (the grammar cannot say it, the descriptor can): C[a,b,c] +/-= A[c,a] * B[b], one multiply and one
    add per element, which numpy does with the same two roundings."""
    for op in ("+=", "-="):
        expr = {"out": "t3", "op": op, "a": "t2", "b": "v2", "out_idx": ["a", "b", "c"], "sum_idx": [],
                "a_idx": ["c", "a"], "b_idx": ["b"], "all_idx": ["a", "b", "c"]}
        sizes = [3, 4, 2]
        C, A, B = inputs(expr, sizes, dtype)
        got = oracle.contract(expr, sizes, C.copy(), A, B).reshape((3, 4, 2), order="F")
        Af, Cf = A.reshape((2, 3), order="F"), C.reshape((3, 4, 2), order="F")
        prod = (Af.T[:, None, :] * B[None, :, None]).astype(dtype)              # [a, b, c], rounded once
        want = (Cf - prod if op == "-=" else Cf + prod).astype(dtype)
        assert got.dtype == dtype and np.array_equal(got, want)


def test_oracle_closed_forms(oracle):
    text = "t3 [a,4,b,3,c,5] += sum(d,7) * t2 [b,d,a] * v2 [d,c];"
    expr = parse_expression(text)
    sizes = [4, 3, 5, 7]
    nC, nA, nB = tensor_sizes(expr, sizes)
    # all ones: every element equals the contracted extent
    got = oracle.contract(expr, sizes, np.zeros(nC), np.ones(nA), np.ones(nB))
    assert np.array_equal(got, np.full(nC, 7.0))
    # one-hot B[d0, c0]: C[:, :, c0] is A[:, d0, :] transposed, everything else untouched
    A = uniform(nA, 5, np.float64)
    B = np.zeros(nB)
    d0, c0 = 2, 3
    B[d0 + 7 * c0] = 1.0
    got = oracle.contract(expr, sizes, np.zeros(nC), A, B).reshape((4, 3, 5), order="F")
    Af = A.reshape((3, 7, 4), order="F")
    want = np.zeros((4, 3, 5))
    want[:, :, c0] = Af[:, d0, :].T
    assert np.array_equal(got, want)


def test_oracle_linearity_and_sign(oracle):
    text = "t3 [a,4,b,3] += sum(c,5) * t2 [c,a] * v2 [b,c];"
    plus = parse_expression(text)
    minus = parse_expression(text.replace("+=", "-="))
    sizes = [4, 3, 5]
    C, A, B = inputs(plus, sizes, np.float64)
    r1 = oracle.contract(plus, sizes, C.copy(), A, B)
    back = oracle.contract(minus, sizes, r1.copy(), A, B)
    assert helpers.rel_error(back, C) < 1e-15
    r2 = oracle.contract(plus, sizes, np.zeros_like(C), 2.0 * A, B)
    r3 = oracle.contract(plus, sizes, np.zeros_like(C), A, B)
    assert np.array_equal(r2, 2.0 * r3)      # scaling by 2 is exact in binary floating point


def test_oracle_thread_count_does_not_change_bits(oracle):
    expr = parse_expression(EINSUM_CASES[3][0])
    sizes = [6, 5, 4, 3, 4, 5, 7]
    C, A, B = inputs(expr, sizes, np.float32)
    one = oracle.contract(expr, sizes, C.copy(), A, B, threads=1)
    many = oracle.contract(expr, sizes, C.copy(), A, B, threads=8)
    assert np.array_equal(one, many)


def test_oracle_sub_range_of_last_index(oracle):
    expr = parse_expression(EINSUM_CASES[0][0])
    sizes = [5, 4, 3, 6]
    C, A, B = inputs(expr, sizes, np.float64)
    full = oracle.contract(expr, sizes, C.copy(), A, B)
    part = oracle.contract(expr, sizes, C.copy(), A, B, last_range=(1, 2))
    slab = slice(5 * 4 * 1, 5 * 4 * 2)
    assert np.array_equal(part[slab], full[slab])
    assert np.array_equal(part[:slab.start], C[:slab.start]) and np.array_equal(part[slab.stop:], C[slab.stop:])


def test_fill_matches_numpy_stream(tools):
    for dtype in (np.float64, np.float32):
        a = np.empty(1000, dtype=dtype)
        tools.fill_uniform(a, 12345)
        assert np.array_equal(a, uniform(1000, 12345, dtype))
        assert a.min() >= -1.0 and a.max() < 1.0
