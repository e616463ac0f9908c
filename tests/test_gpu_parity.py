"""GPU parity: every compiled expression, called through its C-ABI entry point, against the CPU oracle.

Tolerances (stated by the task): max relative error <= 1e-12 for fp64 and <= 1e-5 for fp32, with
relative error = |gpu - ref| / max(|ref|, rms(ref)).  The plain kernel keeps the reference loop's
summation order with separately rounded multiply and add, so it must match the oracle bit for bit.
"""
import os
import sys

import numpy as np
import pytest

import helpers
from gpu_common import make_inputs, run_entry

pytestmark = pytest.mark.gpu

TOL = {"f64": 1e-12, "f32": 1e-5}
SMALL = [3, 4, 5, 2, 6, 3, 4, 2, 3, 5, 2, 3]
ODD = [17, 5, 3, 9, 2, 7, 19, 3, 6, 5, 4, 2]


def _pkg():
    import cogent_mi355
    return cogent_mi355


def all_names():
    import json
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "cgo2019-ae_amd", "expressions", "manifest.json")) as f:
        return [e["name"] for e in json.load(f)["expressions"]]


def tile_sizes(ex, expr, mult):
    """Extents that are exact multiples of the compiled tiles (exercises the unpredicated kernels)."""
    tiles = {}
    for side in ("x", "y", "k"):
        for name, t in ex.info[side]:
            tiles[name] = t
    return [tiles[n] * mult.get(n, 1) for n in expr["all_idx"]]


def check(name, sizes, tools, oracle, c_mode="seeded", variant=None, exact=False):
    pkg = _pkg()
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    dtype = np.float64 if ex.dtype == "f64" else np.float32
    print("[gpu] %s sizes=%s variant=%s" % (name, sizes, variant), flush=True)
    C, A, B = make_inputs(tools, expr, sizes, dtype, c_mode)
    got = run_entry(ex, sizes, C, A, B, variant)
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    if exact:
        assert np.array_equal(got, want)
    else:
        err = helpers.rel_error(got, want)
        assert err <= TOL[ex.dtype], "%s %s: max rel err %.3g" % (name, sizes, err)
    return ex


@pytest.mark.parametrize("name", all_names())
def test_small_ragged_extents(name, tools, oracle):
    """Extents that divide no tile: the predicated kernel on every index; C starts from a nonzero seed."""
    n = _pkg().Expression(name).n
    check(name, SMALL[:n], tools, oracle)


@pytest.mark.parametrize("name", all_names())
def test_plain_kernel_is_bit_exact(name, tools, oracle):
    n = _pkg().Expression(name).n
    check(name, SMALL[:n], tools, oracle, variant=1, exact=True)


@pytest.mark.parametrize("name", all_names())
def test_valu_streaming_kernel_is_bit_exact(name, tools, oracle):
    """variant 3: blocks walk C in memory order, every lane sums its elements' terms in sum() order with separately
    rounded multiply and add.  Ragged sizes (scalar accesses) and sizes whose fastest extent allows 16-byte accesses."""
    pkg = _pkg()
    n = pkg.Expression(name).n
    ex = check(name, SMALL[:n], tools, oracle, variant=3, exact=True)
    assert ex.last_kernel() == "valu"
    check(name, ([8] + SMALL[1:])[:n], tools, oracle, variant=3, exact=True)


@pytest.mark.parametrize("name", all_names())
def test_exact_tile_multiples(name, tools, oracle):
    """Extents equal to the compiled tiles (twice the tile on the first and the last index when small)."""
    pkg = _pkg()
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    sizes = tile_sizes(ex, expr, {})
    first, last = expr["all_idx"][0], expr["all_idx"][-1]
    vol = float(np.prod(sizes, dtype=np.float64))
    mult = {}
    if vol * 2 <= 4e7:
        mult[last] = 2
    if vol * 4 <= 4e7:
        mult[first] = 2
    sizes = tile_sizes(ex, expr, mult)
    if float(np.prod(sizes, dtype=np.float64)) > 3e8:
        pytest.skip("tile volume too large for the CPU oracle in a unit test")
    check(name, sizes, tools, oracle)


@pytest.mark.parametrize("name", [n for n in all_names() if n.startswith("cfg")])
def test_odd_extents_mixed_full_and_partial(name, tools, oracle):
    """Externals partial / contracted full and the other way round."""
    pkg = _pkg()
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    full = tile_sizes(ex, expr, {})
    n_out = len(expr["out_idx"])
    odd = ODD[:len(full)]
    cap = lambda v: [min(x, 24) for x in v]
    ext_partial = cap(odd[:n_out]) + [min(f, 48) for f in full[n_out:]]
    int_partial = [min(f, 16) for f in full[:n_out]] + cap(odd[n_out:])
    check(name, ext_partial, tools, oracle)
    check(name, int_partial, tools, oracle)


@pytest.mark.parametrize("name", [n for n in all_names() if n.startswith("rand_")])
def test_random_expressions_at_their_own_and_at_odd_sizes(name, tools, oracle):
    """The seeded random expressions (written by tests/golden/make_random_expressions.py): at the sizes they were mapped for, and
    at odd sizes that divide none of their tiles."""
    pkg = _pkg()
    n = pkg.Expression(name).n
    check(name, pkg.manifest_entry(name)["bench_sizes"], tools, oracle)
    check(name, ODD[:n], tools, oracle)


@pytest.mark.parametrize("name", ["cfg1_f64", "cfg3_f64", "cfg4_f32", "cfg5_3_f64"])
def test_zero_initialised_output_and_unit_extents(name, tools, oracle):
    n = _pkg().Expression(name).n
    check(name, SMALL[:n], tools, oracle, c_mode="zero")
    check(name, [1] * n, tools, oracle)
    sizes = [1] * n
    sizes[0] = 33
    sizes[-1] = 5
    check(name, sizes, tools, oracle)
