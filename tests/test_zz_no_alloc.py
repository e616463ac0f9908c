"""cogent_run_noalloc: the entry point for callers that cannot allocate.  On an object whose mapping repacks
both inputs (the one shipped kernel path with a scratch buffer) its output must equal, bit for bit, that of
cogent_run, which takes the buffer from the stream-ordered allocator: the kernels are the same, only the
home of the repacked copies differs.  Two calls in a row, the second on a smaller problem, so that what the
first call left in the static array is still there when the second one runs."""
import numpy as np
import pytest

import helpers
from gpu_common import DeviceTensor, make_inputs

pytestmark = pytest.mark.gpu

NAME = "var_cfg2_repack_f64"


def _both(ex, expr, sizes, tools, oracle, seeds):
    import torch
    C, A, B = make_inputs(tools, expr, sizes, np.float64, seeds=seeds)
    out = []
    for call in (ex.run, ex.run_noalloc):
        dC, dA, dB = DeviceTensor(C), DeviceTensor(A), DeviceTensor(B)
        rc = call(sizes, dC.ptr, dA.ptr, dB.ptr, None, 0)
        torch.cuda.synchronize()
        assert rc == 0, ex.last_error()
        assert dC.guards_intact() and np.array_equal(dA.host(), A) and np.array_equal(dB.host(), B)
        out.append(dC.host())
    assert np.array_equal(out[0], out[1]), "cogent_run_noalloc differs from cogent_run at sizes %s" % sizes
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    assert helpers.rel_error(out[1], want) <= 1e-12


def test_noalloc_entry_matches_allocating_entry(tools, oracle):
    import cogent_mi355 as pkg
    ex = pkg.Expression(NAME)
    assert ex.info["repack"] == [1, 1]
    expr = helpers.parse_expression(pkg.expression_text(NAME))
    print("[gpu] no-alloc entry %s: first call, full tiles" % NAME, flush=True)
    _both(ex, expr, [72, 8, 48, 6, 72], tools, oracle, (1, 2, 3))
    print("[gpu] no-alloc entry %s: second call, smaller and ragged" % NAME, flush=True)
    _both(ex, expr, [40, 3, 25, 5, 17], tools, oracle, (4, 5, 6))


def test_noalloc_entry_refuses_inputs_beyond_its_scratch(tools):
    """Both repacked inputs must fit the 16 MiB static array: a larger call is refused before any launch."""
    import torch
    import cogent_mi355 as pkg
    ex = pkg.Expression(NAME)
    sizes = [128, 128, 128, 128, 72]           # each input 128*72*128 doubles = 9.4 MB: 18.9 MB together
    buf = torch.zeros(1024, dtype=torch.float64, device="cuda")
    print("[gpu] no-alloc entry %s: oversize call" % NAME, flush=True)
    rc = ex.run_noalloc(sizes, buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), None, 0)
    assert rc == 3 and "scratch" in ex.last_error()
    torch.cuda.synchronize()
    assert float(buf.abs().max()) == 0.0


def test_noalloc_entry_on_an_object_without_scratch(tools, oracle):
    """A mapping that needs no scratch memory exports the same symbol; there it is cogent_run itself."""
    import cogent_mi355 as pkg
    from gpu_common import run_entry
    ex = pkg.Expression("cfg5_1_f64")
    expr = helpers.parse_expression(pkg.expression_text("cfg5_1_f64"))
    sizes = [6, 5, 4, 3, 2, 3, 8]
    C, A, B = make_inputs(tools, expr, sizes, np.float64)
    import torch
    dC, dA, dB = DeviceTensor(C), DeviceTensor(A), DeviceTensor(B)
    print("[gpu] no-alloc entry cfg5_1_f64", flush=True)
    assert ex.run_noalloc(sizes, dC.ptr, dA.ptr, dB.ptr, None, 0) == 0
    torch.cuda.synchronize()
    assert np.array_equal(dC.host(), run_entry(ex, sizes, C, A, B))
