"""GPU parity of the panel-resident streaming kernel (one persistent workgroup per run of output tiles).

An object emitted with `st=` in its mapping holds both kernels; the launcher takes the streaming one when the
extents give full tiles and the K-block count it was compiled for, and the per-tile kernel otherwise.  Both
paths are checked against the CPU oracle through the C-ABI entry points, and `cogent_last_kernel` tells which
one ran.  Tolerances as in test_gpu_parity.py: 1e-12 (fp64), 1e-5 (fp32).
"""
import numpy as np
import pytest

import helpers
from gpu_common import make_inputs, run_entry

pytestmark = pytest.mark.gpu

TOL = {"f64": 1e-12, "f32": 1e-5}
STREAMING = ["cfg2_f64", "var_cfg2_stream96_f64", "var_cfg4_stream_f32", "var_stream_2k_f64",
             "var_tccg11_stream_y_f64",      # the Y panel resident, its 72 rows padded to 80
             "var_tccg09_stream_pad_f64",    # the X panel resident, its 72 columns padded to 80
             "var_cfg4_stream_pad_f32",      # fp32, 128-bit C accesses, a Y tile of 24 rows padded to 32
             "var_cfg2_stream_cd2_f64",      # C read two tiles ahead (runs of 12 and 9 tiles: both parities end a run)
             "var_tccg11_stream_y_ov_f64"]   # Y panel loaded behind the first tile, interleaved runs


def _check(name, sizes, tools, oracle, variant=None, expect=None):
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    dtype = np.float64 if ex.dtype == "f64" else np.float32
    print("[gpu] %s sizes=%s variant=%s expect=%s" % (name, sizes, variant, expect), flush=True)
    C, A, B = make_inputs(tools, expr, sizes, dtype)
    got = run_entry(ex, sizes, C, A, B, variant)
    kind = ex.last_kernel()
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    err = helpers.rel_error(got, want)
    assert err <= TOL[ex.dtype], "%s %s: max rel err %.3g (%s kernel)" % (name, sizes, err, kind)
    if expect:
        assert kind == expect, "%s %s ran the %s kernel" % (name, sizes, kind)
    return ex


def _tiles(ex):
    return {n: t for side in ("x", "y", "k") for n, t in ex.info[side]}


@pytest.mark.parametrize("name", STREAMING)
def test_objects_carry_the_streaming_kernel(name):
    import cogent_mi355 as pkg
    info = pkg.Expression(name).info
    nkb, depth = info["stream"]
    assert nkb >= 2 and depth >= 1 and nkb % depth == 0
    assert info["stream_resident"] == ("y" if name.startswith("var_tccg11_stream_y") else "x")


@pytest.mark.parametrize("name", STREAMING)
def test_full_size_runs_of_several_tiles(name, tools, oracle):
    """The sizes the object was emitted for: every workgroup walks a run of output tiles."""
    import cogent_mi355 as pkg
    sizes = pkg.manifest_entry(name)["bench_sizes"]
    _check(name, sizes, tools, oracle, expect="stream")


@pytest.mark.parametrize("name", STREAMING)
def test_small_outputs_one_tile_per_workgroup(name, tools, oracle):
    """Contracted extents as emitted, external extents one or two tiles: runs of a single tile."""
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    rep = dict(zip(expr["all_idx"], pkg.manifest_entry(name)["bench_sizes"]))
    tiles = _tiles(ex)
    sizes = [rep[n] if n in expr["sum_idx"] else tiles[n] * (2 if j % 2 == 0 else 1) for j, n in enumerate(expr["all_idx"])]
    _check(name, sizes, tools, oracle, expect="stream")


@pytest.mark.parametrize("name", STREAMING)
def test_other_extents_fall_back_to_the_per_tile_kernel(name, tools, oracle):
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    rep = dict(zip(expr["all_idx"], pkg.manifest_entry(name)["bench_sizes"]))
    tiles = _tiles(ex)
    # ragged external extents, contracted extents as emitted
    ragged = [rep[n] if n in expr["sum_idx"] else tiles[n] + 1 + j for j, n in enumerate(expr["all_idx"])]
    _check(name, ragged, tools, oracle, expect="tiled")
    # full tiles, but another number of K blocks
    k0 = expr["sum_idx"][0]
    other_k = [tiles[n] if n not in expr["sum_idx"] else (tiles[n] * 2 if n == k0 and rep[n] != tiles[n] * 2 else tiles[n] * (4 if n == k0 else 1))
               for n in expr["all_idx"]]
    _check(name, other_k, tools, oracle, expect="tiled")


def test_explicit_variants_at_config_2(tools, oracle):
    """variant 2 asks for the per-tile kernel of the same object, variant 1 for the plain kernel."""
    sizes = [72, 72, 72, 72, 72]
    _check("cfg2_f64", sizes, tools, oracle, variant=2, expect="tiled")
    _check("cfg2_f64", [72, 4, 8, 8, 72], tools, oracle, variant=1, expect="plain")


def test_streaming_kernel_inside_a_captured_graph(tools, oracle):
    """After one eager call (which sizes the kernel's LDS once), calls on a caller's stream capture and replay."""
    import torch
    import cogent_mi355
    name, sizes = "cfg2_f64", [72, 8, 16, 16, 72]
    ex = cogent_mi355.Expression(name)
    expr = helpers.parse_expression(cogent_mi355.expression_text(name))
    C, A, B = make_inputs(tools, expr, sizes, np.float64)
    want1 = oracle.contract(expr, sizes, C.copy(), A, B)
    want2 = oracle.contract(expr, sizes, want1.copy(), A, B)
    dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
    dC0 = dC.clone()
    assert ex.run(sizes, dC.data_ptr(), dA.data_ptr(), dB.data_ptr(), None, 0) == 0 and ex.last_kernel() == "stream"
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    print("[gpu] graph capture of %s sizes=%s" % (name, sizes), flush=True)
    with torch.cuda.graph(g, stream=s):
        st = torch.cuda.current_stream().cuda_stream
        assert ex.run(sizes, dC.data_ptr(), dA.data_ptr(), dB.data_ptr(), st, 0) == 0
        assert ex.run(sizes, dC.data_ptr(), dA.data_ptr(), dB.data_ptr(), st, 0) == 0
    assert ex.last_kernel() == "stream"
    for replay in range(3):
        dC.copy_(dC0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert helpers.rel_error(dC.cpu().numpy(), want2) <= 1e-12, "replay %d" % replay


def test_first_call_of_a_streaming_object_inside_a_capture(tools, oracle, tmp_path):
    """The first call on a device sizes the kernel's dynamic LDS and reads the CU count; neither is a stream
    operation, so even a FIRST call may be captured.  A private copy of the object is loaded so that no earlier
    test of this process has made that first call."""
    import shutil
    import torch
    import cogent_mi355
    name, sizes = "cfg2_f64", [72, 8, 16, 16, 72]
    fresh = str(tmp_path / "cfg2_first_call.so")
    shutil.copy(cogent_mi355.Expression(name).path, fresh)
    ex = cogent_mi355.Expression(path=fresh)
    expr = helpers.parse_expression(cogent_mi355.expression_text(name))
    C, A, B = make_inputs(tools, expr, sizes, np.float64)
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
    dC0 = dC.clone()
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    print("[gpu] first call of a fresh copy of %s inside a capture, sizes=%s" % (name, sizes), flush=True)
    with torch.cuda.graph(g, stream=s):
        st = torch.cuda.current_stream().cuda_stream
        assert ex.run(sizes, dC.data_ptr(), dA.data_ptr(), dB.data_ptr(), st, 0) == 0, ex.last_error()
    assert ex.last_kernel() == "stream"
    for replay in range(3):
        dC.copy_(dC0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert helpers.rel_error(dC.cpu().numpy(), want) <= 1e-12, "replay %d" % replay


@pytest.mark.parametrize("name", ["var_cfg2_clds_f64", "var_cfg4_clds_f32"])
def test_c_through_lds_with_an_output_that_is_only_element_aligned(name, tools, oracle):
    """cl=1 objects move full C tiles as 16-byte vectors; C may still start at any ELEMENT of a larger buffer."""
    import torch
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    assert ex.info["c_through_lds"] == 1
    expr = helpers.parse_expression(pkg.expression_text(name))
    tiles = _tiles(ex)
    rep = dict(zip(expr["all_idx"], pkg.manifest_entry(name)["bench_sizes"]))
    sizes = [min(rep[n], tiles[n] * (2 if j == 0 else 1)) for j, n in enumerate(expr["all_idx"])]       # full tiles: the LDS path
    np_dtype = np.float64 if ex.dtype == "f64" else np.float32
    C, A, B = make_inputs(tools, expr, sizes, np_dtype)
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    for shift in (0, 1):
        buf = torch.full((C.size + 8,), 777.0, dtype=torch.float64 if ex.dtype == "f64" else torch.float32, device="cuda")
        buf[shift:shift + C.size] = torch.from_numpy(C).cuda()
        print("[gpu] %s sizes=%s C shifted by %d element(s)" % (name, sizes, shift), flush=True)
        rc = ex.run(sizes, buf.data_ptr() + buf.element_size() * shift, dA.data_ptr(), dB.data_ptr(), None, 2)
        torch.cuda.synchronize()
        assert rc == 0, ex.last_error()
        host = buf.cpu().numpy()
        assert np.all(host[:shift] == 777.0) and np.all(host[shift + C.size:] == 777.0), "write outside C"
        assert helpers.rel_error(host[shift:shift + C.size], want) <= TOL[ex.dtype]


@pytest.mark.parametrize("name,sizes,expect", [("var_cfg4_stream_f32", [24, 24, 8, 2, 2, 1, 24], "stream"),
                                               ("cfg4_16_f32", [16, 16, 16, 2, 2, 1, 16], "tiled")])
def test_output_not_16_byte_aligned_takes_the_column_layout(name, sizes, expect, tools, oracle):
    """fp32 objects read and write C with 128-bit accesses when C is 16-byte aligned; a C pointer that is only
    element-aligned must fall back to the column layout of the same kernel and give the same result."""
    import torch
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    assert ex.info["swapped_roles"] == 1
    expr = helpers.parse_expression(pkg.expression_text(name))
    C, A, B = make_inputs(tools, expr, sizes, np.float32)
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    for shift in (0, 1):                                       # elements: 0 = aligned, 1 = 4 bytes off
        buf = torch.full((C.size + 8,), 777.0, dtype=torch.float32, device="cuda")
        buf[shift:shift + C.size] = torch.from_numpy(C).cuda()
        print("[gpu] %s sizes=%s C shifted by %d element(s)" % (name, sizes, shift), flush=True)
        rc = ex.entry(sizes, buf.data_ptr() + 4 * shift, dA.data_ptr(), dB.data_ptr())
        torch.cuda.synchronize()
        assert rc == 0, ex.last_error()
        assert ex.last_kernel() == expect
        host = buf.cpu().numpy()
        assert np.all(host[:shift] == 777.0) and np.all(host[shift + C.size:] == 777.0), "write outside C"
        assert helpers.rel_error(host[shift:shift + C.size], want) <= TOL["f32"]
