"""Behaviour of the C-ABI entry points beyond the numbers: status codes, untouched outputs, the
host-pointer form with the reference's calling convention, streams."""
import ctypes

import numpy as np
import pytest

import helpers
from gpu_common import DeviceTensor, make_inputs

pytestmark = pytest.mark.gpu


def _setup(name, sizes, tools):
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    dtype = np.float64 if ex.dtype == "f64" else np.float32
    C, A, B = make_inputs(tools, expr, sizes, dtype)
    return ex, expr, C, A, B


def test_status_codes(tools):
    import torch
    ex, expr, C, A, B = _setup("cfg1_f64", [4, 5, 6, 7], tools)
    dC, dA, dB = DeviceTensor(C), DeviceTensor(A), DeviceTensor(B)
    print("[gpu] status codes", flush=True)
    assert ex.entry([4, 5, 6, 7], None, dA.ptr, dB.ptr) == 1 and "null" in ex.last_error()
    assert ex.entry([4, 5, 6, 7], dC.ptr, None, dB.ptr) == 1
    assert ex.entry([4, -5, 6, 7], dC.ptr, dA.ptr, dB.ptr) == 2 and "negative" in ex.last_error()
    assert ex.run([4, 5, 6, 7], dC.ptr, dA.ptr, dB.ptr, None, 9) == 5 and ex.run([4, 5, 6, 7], dC.ptr, dA.ptr, dB.ptr, None, -1) == 5
    assert ex.run([4, 5, 6], dC.ptr, dA.ptr, dB.ptr, None, 0) == 1          # wrong number of extents
    # 2^31 elements or more in a tensor: refused before anything is launched
    assert ex.entry([2048, 2048, 1024, 2], dC.ptr, dA.ptr, dB.ptr) == 3 and "2^31" in ex.last_error()
    # fewer than 2^31 elements, but a tile of the mapping would span more than 4 GB of C (32-bit byte offsets inside a tile)
    import cogent_mi355
    pinned = cogent_mi355.Expression("var_cfg1_nto_f64")                    # y = a:16,b:4 over C[c,b,a]
    assert pinned.entry([32, 1200000, 16, 1], dC.ptr, dA.ptr, dB.ptr) == 3 and "4 GB" in pinned.last_error()
    # an empty index range leaves C as it is and succeeds
    for sizes in ([0, 5, 6, 7], [4, 5, 6, 0]):
        assert ex.entry(sizes, dC.ptr, dA.ptr, dB.ptr) == 0
    torch.cuda.synchronize()
    assert np.array_equal(dC.host(), C) and dC.guards_intact()
    # and a good call still works afterwards, with an empty error message
    assert ex.entry([4, 5, 6, 7], dC.ptr, dA.ptr, dB.ptr) == 0 and ex.last_error() == ""
    torch.cuda.synchronize()


@pytest.mark.parametrize("name,sizes", [("tccg_01_f64", [9, 10, 5, 12]), ("cfg4_f32", [5, 4, 3, 6, 2, 3, 7])])
def test_host_pointer_entry_point(name, sizes, tools, oracle):
    """sd_t_d2_fusion_host_: host buffers in, result copied back, as the reference's drivers call it
    (cogent/drivers/tccg/code_main_tccg_01.c:69); C is accumulated into, not overwritten."""
    ex, expr, C, A, B = _setup(name, sizes, tools)
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    got = C.copy()
    print("[gpu] host entry %s %s" % (name, sizes), flush=True)
    rc = ex.entry_host(sizes, got.ctypes.data, A.ctypes.data, B.ctypes.data)
    assert rc == 0, ex.last_error()
    assert helpers.rel_error(got, want) <= (1e-12 if ex.dtype == "f64" else 1e-5)


def test_launch_on_a_caller_stream(tools, oracle):
    import torch
    sizes = [6, 5, 4, 3, 2, 3, 8]
    ex, expr, C, A, B = _setup("cfg5_2_f64", sizes, tools)
    dC, dA, dB = DeviceTensor(C), DeviceTensor(A), DeviceTensor(B)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    print("[gpu] caller stream", flush=True)
    rc = ex.run(sizes, dC.ptr, dA.ptr, dB.ptr, ctypes.c_void_p(stream.cuda_stream), 0)
    stream.synchronize()
    assert rc == 0
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    assert helpers.rel_error(dC.host(), want) <= 1e-12


def test_two_calls_accumulate(tools, oracle):
    """C <- C + sum twice equals C + 2 sum: the entry point really reads C."""
    import torch
    sizes = [8, 3, 5, 9]
    ex, expr, C, A, B = _setup("cfg1_f64", sizes, tools)
    dC, dA, dB = DeviceTensor(C), DeviceTensor(A), DeviceTensor(B)
    print("[gpu] two calls", flush=True)
    assert ex.entry(sizes, dC.ptr, dA.ptr, dB.ptr) == 0
    assert ex.entry(sizes, dC.ptr, dA.ptr, dB.ptr) == 0
    torch.cuda.synchronize()
    want = oracle.contract(expr, sizes, oracle.contract(expr, sizes, C.copy(), A, B), A, B)
    assert helpers.rel_error(dC.host(), want) <= 1e-12


@pytest.mark.gpu
def test_entry_point_inside_a_captured_graph(tools, oracle):
    """cogent_run on a caller's stream allocates nothing and does not synchronise, so a sequence of calls can be
    captured into a HIP graph and replayed: three replays, each checked against the eager result."""
    import torch
    import cogent_mi355
    ex = cogent_mi355.Expression("cfg5_1_f64")
    expr = helpers.parse_expression(cogent_mi355.expression_text("cfg5_1_f64"))
    sizes = [8, 6, 5, 7, 4, 6, 9]
    C, A, B = make_inputs(tools, expr, sizes, np.float64)
    want1 = oracle.contract(expr, sizes, C.copy(), A, B)
    want2 = oracle.contract(expr, sizes, want1.copy(), A, B)          # two launches per replay
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    dC = torch.from_numpy(C).cuda()
    dC0 = dC.clone()
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    print("[gpu] graph capture of cfg5_1_f64 sizes=%s" % sizes, flush=True)
    with torch.cuda.graph(g, stream=s):
        st = torch.cuda.current_stream().cuda_stream
        assert ex.run(sizes, dC.data_ptr(), dA.data_ptr(), dB.data_ptr(), st, 0) == 0
        assert ex.run(sizes, dC.data_ptr(), dA.data_ptr(), dB.data_ptr(), st, 0) == 0
    for replay in range(3):
        dC.copy_(dC0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = dC.cpu().numpy()
        assert helpers.rel_error(got, want2) <= 1e-12, "replay %d" % replay


@pytest.mark.parametrize("sizes", [[24, 16, 16, 24, 1, 5],      # whole output tiles, one K block that is not full
                                   [11, 9, 6, 10, 1, 5],        # ragged output tiles, the same
                                   [24, 16, 16, 24, 1, 8],      # one full K block, whole tiles: the one-K-block kernel serves it
                                   [11, 9, 6, 10, 1, 8],        # one full K block, ragged output tiles: the K loop again
                                   [48, 8, 8, 24, 3, 7]],       # three ragged K blocks: the K loop proper
                         ids=["full-tiles", "ragged-tiles", "full-block", "full-block-ragged-tiles", "k-loop"])
def test_ragged_single_k_block_through_the_k_loop_kernels(sizes, tools, oracle):
    """Mapping option ok=0: a call whose contracted extents fit one K block takes the K-loop kernels (one trip) unless
    all its tiles are whole, instead of the one-K-block kernels, whose variants for ragged tiles spill registers on
    this 192x192 tile.  Every element against the oracle."""
    import cogent_mi355 as pkg
    from gpu_common import make_inputs, run_entry
    name = "var_tccg20_ragged_k_loop_f64"
    ex = pkg.Expression(name)
    assert ex.info["one_block_ragged"] == 0 and ";ok=0" in ex.info["spec"]
    expr = helpers.parse_expression(pkg.expression_text(name))
    print("[gpu] %s sizes=%s" % (name, sizes), flush=True)
    C, A, B = make_inputs(tools, expr, sizes, np.float64)
    got = run_entry(ex, sizes, C, A, B)
    assert ex.last_kernel() == "tiled"
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    assert helpers.rel_error(got, want) <= 1e-12
