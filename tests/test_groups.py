"""Fused groups: several contractions into one output, one kernel that keeps the output tile on chip.

Reference: expressions with an identical output index list form one group
(cogent/src/algs/bases/tc_gen_inputs.py:113-123); the fused entry point takes one pair of inputs and one
flag per term (cogent/src/codes/kernels/tc_interface.py:1494-1511); the nine sd_t_d2 terms and their signs
are those of cogent/drivers/ccsd_t/code_main_sd2_1.c:573-606.  The expected result is the oracle applied
term by term to the same output (the reference's check adds the terms inside one loop nest; the two differ
only in rounding, and the reference ships that loop with eight of the nine terms commented out).
"""
import ctypes
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import helpers

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "cgo2019-ae_amd")
sys.path.insert(0, PKG)
GEN = os.path.join(PKG, "bin", "cogent_gen")
FUSED = os.path.join(PKG, "expressions", "fused_sd2_f64.in")


def plan_json(path, dtype="DOUBLE", spec=None):
    cmd = [GEN, "g", path, "-1", "-1", dtype, "-o", os.devnull, "--json"] + (["--map", spec] if spec else [])
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    return r.returncode, (json.loads(r.stdout) if r.returncode == 0 else r.stderr)


def test_group_plan_shares_one_tile_and_gives_each_term_its_own_roles():
    rc, j = plan_json(FUSED)
    assert rc == 0 and j["group"] and j["n_terms"] == 9 and j["threads"] == 512           # 4096-element tile: eight wavefronts
    assert j["out_idx"] == ["h3", "h2", "h1", "p6", "p5", "p4"] and j["sum_idx"] == ["p7"]
    tile = dict(zip(j["out_idx"], j["c_tile"]))
    vol = int(np.prod(j["c_tile"]))
    assert 256 <= vol * 8 <= 32768 and j["lds_bytes"] <= 160 * 1024          # dynamic LDS: the CU's 160 KB is the limit
    for term in j["terms"]:
        m = term["mapping"]
        # every output index is tiled exactly once, with the group's tile, on the side of the input that holds it
        got = {n: t for n, t in m["x"] + m["y"]}
        assert got == tile
        assert m["x"][0][0] == "h3"                         # the output's fastest index leads the X side
        assert m["block_tile"][0] * m["block_tile"][1] == vol
        assert m["threads"] == 512 and m["split_k"] == 1
    # the nine terms do not agree on which input is the X side, nor on the split of the externals
    assert len({tuple(n for n, _ in t["mapping"]["x"]) for t in j["terms"]}) > 1


def test_group_tile_spec_and_rejections(tmp_path):
    rc, j = plan_json(FUSED, spec="ct=16,2,2,4,2,2")
    assert rc == 0 and j["c_tile"] == [16, 2, 2, 4, 2, 2] and j["spec"] == "ct=16,2,2,4,2,2;kt=32;nw=4;nr=1"
    rc, j = plan_json(FUSED, spec="ct=16,4,4,2,2,2;kt=8;nw=8")                 # K depth per block, wavefronts per workgroup
    assert rc == 0 and j["threads"] == 512 and all(t["mapping"]["block_tile"][2] == 8 for t in j["terms"])
    rc, j = plan_json(FUSED, spec="ct=16,4,4,2,2,2;kt=16;nw=4;nr=1;ps=1")     # persistent workgroups (opt-in)
    assert rc == 0 and j["spec"].endswith(";ps=1")
    for nr in (0, 1, 2):                                               # operand regions of the pipelined kernel; 0 = the per-term kernel
        rc, j = plan_json(FUSED, spec="ct=16,4,4,2,2,2;kt=16;nw=4;nr=%d" % nr)
        assert rc == 0 and j["spec"].endswith(";nr=%d" % nr)
    rc, err = plan_json(FUSED, spec="tile=3")
    assert rc == 3 and "fields are" in err
    rc, err = plan_json(FUSED, spec="ct=16,16,16,16,1,1")              # 64 K elements of C: does not fit
    assert rc == 3 and "does not fit" in err
    rc, err = plan_json(FUSED, spec="ct=16,2,2")
    assert rc == 3 and "one tile per output index" in err
    # expressions with different outputs are not a group
    bad = tmp_path / "bad.in"
    bad.write_text("t3 [a,8,b,8] += sum(c,8) * t2 [a,c] * v2 [c,b];\nt3 [b,8,a,8] += sum(c,8) * t2 [a,c] * v2 [c,b];\n")
    rc, err = plan_json(str(bad))
    assert rc == 3 and "must share the output" in err


@pytest.mark.parametrize("name", ["fused_sd2_f64", "fused_sd1_f32"])
def test_group_object_exports_the_fused_entry_points(name):
    so = os.path.join(PKG, "lib", name + ".so")
    out = subprocess.run(["nm", "-D", "--defined-only", so], stdout=subprocess.PIPE, text=True, check=True).stdout
    for sym in ("sd_t_d2_fusion_", "sd_t_d2_fusion_host_", "cogent_run_group", "cogent_%s_run_group" % name,
                "cogent_num_indices", "cogent_num_terms", "cogent_last_error", "cogent_expression", "cogent_info"):
        assert (" T " + sym + "\n") in out, sym


def test_fp32_group_plan():
    rc, j = plan_json(os.path.join(PKG, "expressions", "fused_sd1_f32.in"), dtype="FLOAT")
    assert rc == 0 and j["dtype"] == "f32" and j["n_terms"] == 9 and j["sum_idx"] == ["h7"]
    assert int(np.prod(j["c_tile"])) * 4 <= 32768
    assert all(t["mapping"]["mfma"] == "v_mfma_f32_16x16x4_f32" for t in j["terms"])


def expected(terms, sizes, C, inputs, oracle, enabled=None):
    want = C.copy()
    for k, expr in enumerate(terms):
        if enabled is None or enabled[k]:
            want = oracle.contract(expr, sizes, want, inputs[2 * k], inputs[2 * k + 1])
    return want


TOL = {"f64": 1e-12, "f32": 1e-5}


def run_group(g, terms, sizes, tools, oracle, enabled=None, via="entry"):
    import torch
    from gpu_common import DeviceTensor
    dt = np.float64 if g.dtype == "f64" else np.float32
    rng_seed = 10
    inputs = []
    for expr in terms:
        _, nA, nB = helpers.tensor_sizes(expr, sizes)
        inputs.append(tools.fill_uniform(np.empty(nA, dt), rng_seed)); rng_seed += 1
        inputs.append(tools.fill_uniform(np.empty(nB, dt), rng_seed)); rng_seed += 1
    nC = helpers.tensor_sizes(terms[0], sizes)[0]
    C = tools.fill_uniform(np.empty(nC, dt), 3)
    dC = DeviceTensor(C)
    dI = [DeviceTensor(a) for a in inputs]
    ptrs = [d.ptr for d in dI]
    print("[gpu] group %s sizes=%s enabled=%s via=%s" % (os.path.basename(g.path), sizes, enabled, via), flush=True)
    rc = g.entry(sizes, dC.ptr, ptrs, enabled) if via == "entry" else g.run(sizes, dC.ptr, ptrs, enabled)
    torch.cuda.synchronize()
    assert rc == 0, g.last_error()
    assert dC.guards_intact(), "write outside C"
    for d, a in zip(dI, inputs):
        assert np.array_equal(d.host(), a), "an input was modified"
    return dC.host(), expected(terms, sizes, C, inputs, oracle, enabled)


def load_group(name):
    import cogent_mi355
    g = cogent_mi355.Group(name)
    return g, [helpers.parse_expression(t) for t in g.expressions]


@pytest.fixture(scope="module")
def group():
    return load_group("fused_sd2_f64")


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["fused_sd2_f64", "fused_sd1_f32", "var_fused_sd2_two_regions_f64", "var_fused_sd2_persistent_f64",
                                  "var_fused_sd1_per_term_pass_f32"])
@pytest.mark.parametrize("sizes", [[5, 3, 7, 6, 2, 9, 4], [16, 4, 4, 2, 2, 2, 16], [17, 5, 6, 3, 4, 3, 19], [1, 1, 1, 1, 1, 1, 1],
                                   [32, 8, 4, 4, 4, 2, 24], [16, 16, 16, 16, 8, 8, 16]])
def test_fused_group_matches_the_terms_applied_one_by_one(name, sizes, tools, oracle):
    g, terms = load_group(name)
    assert g.n_terms == 9 and g.n == 7
    got, want = run_group(g, terms, sizes, tools, oracle)
    assert helpers.rel_error(got, want) <= TOL[g.dtype]


@pytest.mark.gpu
def test_fused_group_term_flags_and_array_form(group, tools, oracle):
    g, terms = group
    sizes = [9, 5, 4, 3, 6, 2, 7]
    only = [1, 0, 0, 0, 1, 0, 0, 0, 1]
    got, want = run_group(g, terms, sizes, tools, oracle, enabled=only)
    assert helpers.rel_error(got, want) <= 1e-12
    got, want = run_group(g, terms, sizes, tools, oracle, enabled=only, via="run")
    assert helpers.rel_error(got, want) <= 1e-12
    none = [0] * 9
    got, want = run_group(g, terms, sizes, tools, oracle, enabled=none)
    assert np.array_equal(got, want)                                     # no term: C comes back bit for bit


@pytest.mark.gpu
def test_fused_group_full_size_and_status_codes(group, tools, oracle):
    import torch
    g, terms = group
    sizes = [16] * 7
    got, want = run_group(g, terms, sizes, tools, oracle)
    assert helpers.rel_error(got, want) <= 1e-12
    buf = torch.zeros(16, dtype=torch.float64, device="cuda")
    ptrs = [buf.data_ptr()] * 18
    assert g.entry([1, 1, 1, 1, 1, 1, -1], buf.data_ptr(), ptrs) == 2
    assert g.entry([1, 1, 1, 0, 1, 1, 1], buf.data_ptr(), ptrs) == 0      # empty: nothing to do
    assert g.entry([1] * 7, 0, ptrs) == 1 and "null" in g.last_error()
    assert g.run([1] * 6, buf.data_ptr(), ptrs) == 1


@pytest.mark.gpu
def test_fused_group_host_pointer_form(group, tools, oracle):
    """sd_t_d2_fusion_host_ of a group: the reference's calling convention (host buffers in, output copied back)."""
    g, terms = group
    sizes = [6, 5, 4, 3, 4, 2, 8]
    inputs, seed = [], 40
    for expr in terms:
        _, nA, nB = helpers.tensor_sizes(expr, sizes)
        inputs.append(tools.fill_uniform(np.empty(nA, np.float64), seed)); seed += 1
        inputs.append(tools.fill_uniform(np.empty(nB, np.float64), seed)); seed += 1
    C = tools.fill_uniform(np.empty(helpers.tensor_sizes(terms[0], sizes)[0], np.float64), 3)
    want = expected(terms, sizes, C, inputs, oracle)
    got = C.copy()
    print("[gpu] group host form sizes=%s" % sizes, flush=True)
    rc = g.entry_host(sizes, got.ctypes.data, [a.ctypes.data for a in inputs])
    assert rc == 0, g.last_error()
    assert helpers.rel_error(got, want) <= 1e-12
