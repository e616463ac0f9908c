"""The BASELINE configurations at their FULL sizes, through properties that need no CPU pass over
the whole tensor: a slab of the output against the CPU oracle, the whole output against the plain
kernel (which is bit-exact with the oracle at the sizes test_gpu_parity.py covers), closed forms and
linearity.  Tolerances: 1e-12 (fp64) / 1e-5 (fp32) on |gpu-ref| / max(|ref|, rms(ref))."""
import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu

TOL = {"f64": 1e-12, "f32": 1e-5}


def configs():
    import json
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "cgo2019-ae_amd", "expressions", "manifest.json")) as f:
        return [(e["name"], e["bench_sizes"], e.get("c_init") == "seeded") for e in json.load(f)["expressions"]
                if e["name"].startswith(("cfg", "smallk", "ext4"))]


@pytest.mark.parametrize("name,sizes,seeded", configs(), ids=[c[0] for c in configs()])
def test_full_size_against_plain_kernel_and_oracle_slab(name, sizes, seeded, tools, oracle):
    import torch
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    dtype = np.float64 if ex.dtype == "f64" else np.float32
    nC, nA, nB = helpers.tensor_sizes(expr, sizes)
    A = tools.fill_uniform(np.empty(nA, dtype), 1)
    B = tools.fill_uniform(np.empty(nB, dtype), 2)
    C = tools.fill_uniform(np.empty(nC, dtype), 3) if seeded else np.zeros(nC, dtype)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    d_tiled, d_plain = torch.from_numpy(C).cuda(), torch.from_numpy(C).cuda()
    print("[gpu] full size %s %s" % (name, sizes), flush=True)
    assert ex.entry(sizes, d_tiled.data_ptr(), dA.data_ptr(), dB.data_ptr()) == 0, ex.last_error()
    assert ex.run(sizes, d_plain.data_ptr(), dA.data_ptr(), dB.data_ptr(), None, 1) == 0, ex.last_error()
    torch.cuda.synchronize()
    # whole tensor on the device: tiled MFMA kernel vs plain kernel
    ref = d_plain.double()
    rms = torch.sqrt(torch.mean(ref * ref)).item() or 1.0
    err = (torch.abs(d_tiled.double() - ref) / torch.clamp(torch.abs(ref), min=rms)).max().item()
    assert err <= TOL[ex.dtype], "tiled vs plain: %.3g" % err
    # a slab of the slowest output index against the CPU oracle (a few hundred MFLOP at most)
    last = sizes[len(expr["out_idx"]) - 1]
    per_slice = 2.0 * np.prod(sizes, dtype=np.float64) / last
    n = int(max(1, min(last, 4e8 // per_slice)))
    want = oracle.contract(expr, sizes, C.copy(), A, B, last_range=(0, n))
    slab = (nC // last) * n
    got = d_tiled[:slab].cpu().numpy()
    assert helpers.rel_error(got, want[:slab]) <= TOL[ex.dtype]
    got_plain = d_plain[:slab].cpu().numpy()
    assert np.array_equal(got_plain, want[:slab]), "plain kernel is not bit-exact with the oracle"


@pytest.mark.parametrize("name", ["cfg2_f64", "cfg3_f64", "cfg4_16_f32", "cfg5_9_f64"])
def test_full_size_closed_form_and_linearity(name, tools):
    import torch
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    entry = pkg.manifest_entry(name)
    sizes = entry["bench_sizes"]
    expr = helpers.parse_expression(pkg.expression_text(name))
    tdtype = torch.float64 if ex.dtype == "f64" else torch.float32
    nC, nA, nB = helpers.tensor_sizes(expr, sizes)
    ksize = int(np.prod(sizes[len(expr["out_idx"]):]))
    print("[gpu] closed form %s" % name, flush=True)
    # all ones: every output element equals the product of the contracted extents, exactly
    ones_a = torch.ones(nA, dtype=tdtype, device="cuda")
    ones_b = torch.ones(nB, dtype=tdtype, device="cuda")
    c = torch.zeros(nC, dtype=tdtype, device="cuda")
    assert ex.entry(sizes, c.data_ptr(), ones_a.data_ptr(), ones_b.data_ptr()) == 0
    torch.cuda.synchronize()
    assert bool((c == float(ksize)).all())
    # linearity in A: scaling A by 2 scales the result by exactly 2 (power of two: no rounding)
    np_dtype = np.float64 if ex.dtype == "f64" else np.float32
    a = torch.from_numpy(tools.fill_uniform(np.empty(nA, np_dtype), 7)).cuda()
    b = torch.from_numpy(tools.fill_uniform(np.empty(nB, np_dtype), 8)).cuda()
    c1 = torch.zeros(nC, dtype=tdtype, device="cuda")
    c2 = torch.zeros(nC, dtype=tdtype, device="cuda")
    assert ex.entry(sizes, c1.data_ptr(), a.data_ptr(), b.data_ptr()) == 0
    a2 = a * 2
    assert ex.entry(sizes, c2.data_ptr(), a2.data_ptr(), b.data_ptr()) == 0
    torch.cuda.synchronize()
    if ex.info.get("split_k", 1) > 1:
        # the K shares of a tile are added with atomics in arrival order: equal up to rounding only
        rms = float(torch.sqrt(torch.mean(c1 * c1)))
        err = float((torch.abs(c2 - 2 * c1) / torch.clamp(torch.abs(2 * c1), min=2 * rms)).max())
        assert err <= TOL[ex.dtype]
    else:
        assert bool((c2 == 2 * c1).all())
    assert float(c1.abs().max()) > 0


@pytest.mark.parametrize("name", ["cfg5_1_f64", "cfg4_16_f32", "cfg2_f64", "smallk2_f64"])
@pytest.mark.parametrize("k", [1, 2, 3, 5, 7])
def test_contracted_extents_that_do_not_fill_a_matrix_step(name, k, tools, oracle):
    """Contracted extents below the 4-deep step of the fp64 / fp32 matrix instructions, and odd ones above it: the
    slices are zero-padded to the step in LDS (no separate small-K kernel: a padded step costs nothing next to the
    output traffic, see the measured small-K rows of the benchmark).  Every element against the oracle."""
    import cogent_mi355 as pkg
    from gpu_common import make_inputs, run_entry
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    tiles = {n: t for side in ("x", "y", "k") for n, t in ex.info[side]}
    sizes = [k if n in expr["sum_idx"] else min(2 * tiles[n], 24) for n in expr["all_idx"]]
    dtype = np.float64 if ex.dtype == "f64" else np.float32
    print("[gpu] small contracted extent %s sizes=%s" % (name, sizes), flush=True)
    C, A, B = make_inputs(tools, expr, sizes, dtype)
    got = run_entry(ex, sizes, C, A, B)
    want = oracle.contract(expr, sizes, C.copy(), A, B)
    assert helpers.rel_error(got, want) <= TOL[ex.dtype]
    if k == 1:
        # a single term per element: one product and one sum, the oracle's two roundings or the fused one
        assert helpers.rel_error(got, want) <= (3e-16 if ex.dtype == "f64" else 2e-7)


def _factor_tensor(torch, idx_list, ext, tdtype, skip=()):
    """Column-major tensor over idx_list whose value is the product of (i mod 3) + 1 over its indices not in `skip`
    (small integers: every product and sum below is exact in fp64 and fp32)."""
    shape = [ext[i] for i in reversed(idx_list)]                 # torch is row-major: slowest index first
    t = torch.ones(shape, dtype=tdtype, device="cuda")
    for pos, i in enumerate(reversed(idx_list)):
        if i in skip:
            continue
        view = [1] * len(shape)
        view[pos] = ext[i]
        t *= ((torch.arange(ext[i], device="cuda") % 3) + 1).to(tdtype).view(view)
    return t.reshape(-1)


# name, extents (output indices then contracted ones), the kernel expected to run
BEYOND_4_GIB = [
    ("tccg_12_f64", [24576, 24608, 16], "tiled"),                      # 2-D output, K loop: 4.84 GB
    ("cfg5_1_f64", [32, 32, 32, 32, 32, 18, 4], "tiled"),              # 6-D output, one K block, ragged: 4.83 GB
    ("cfg2_f64", [72, 72, 72, 1504, 72], "stream"),                   # the streaming kernel: 4.49 GB
    ("cfg4_16_f32", [16, 16, 16, 16, 16, 1040, 16], None),                      # fp32: 4.36 GB
]


@pytest.mark.parametrize("name,sizes,kernel", BEYOND_4_GIB, ids=[c[0] for c in BEYOND_4_GIB])
def test_output_beyond_4_gib(name, sizes, kernel, tools):
    """Outputs of more than 2^32 bytes: tile origins are 64-bit, offsets inside a tile 32-bit.  Inputs are products of
    per-index factors (i mod 3) + 1 over their external indices, so C[...] = (product of the contracted extents) x the
    product of the factors of ALL its indices: an origin that wrapped, a tile done twice or left out, or an index taken
    for another shows as a wrong integer somewhere.  Checked over every element, on the device, exactly."""
    import torch
    import cogent_mi355 as pkg
    ex = pkg.Expression(name)
    expr = helpers.parse_expression(pkg.expression_text(name))
    tdtype = torch.float64 if ex.dtype == "f64" else torch.float32
    ext = dict(zip(expr["all_idx"], sizes))
    nC, nA, nB = helpers.tensor_sizes(expr, sizes)
    assert nC * (8 if ex.dtype == "f64" else 4) > 2**32 and nC < 2**31
    print("[gpu] beyond 4 GiB %s %s" % (name, sizes), flush=True)
    a = _factor_tensor(torch, expr["a_idx"], ext, tdtype, skip=expr["sum_idx"])
    b = _factor_tensor(torch, expr["b_idx"], ext, tdtype, skip=expr["sum_idx"])
    assert a.numel() == nA and b.numel() == nB
    c = torch.zeros(nC, dtype=tdtype, device="cuda")
    assert ex.entry(sizes, c.data_ptr(), a.data_ptr(), b.data_ptr()) == 0, ex.last_error()
    torch.cuda.synchronize()
    if kernel:
        assert ex.last_kernel() == kernel, ex.last_kernel()
    # divide the factors out again, in place (exact: every value is a small integer multiple of them)
    shape = [ext[i] for i in reversed(expr["out_idx"])]
    cv = c.view(shape)
    for pos, i in enumerate(reversed(expr["out_idx"])):
        view = [1] * len(shape)
        view[pos] = ext[i]
        cv /= ((torch.arange(ext[i], device="cuda") % 3) + 1).to(tdtype).view(view)
    ksize = float(np.prod([ext[i] for i in expr["sum_idx"]]))
    sign = -1.0 if expr["op"] == "-=" else 1.0
    assert bool((c == sign * ksize).all())
    del c, cv, a, b
    torch.cuda.empty_cache()
