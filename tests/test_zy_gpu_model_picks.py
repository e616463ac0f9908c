"""The mapping pass on its own: every BASELINE configuration is also compiled from the pass's FIRST pick (no mapping
spec, no tuned table; lib/model_<name>.so) and must give the tuned object's result and come close to its time.

Bounds: every configuration within 15 % of its tuned object and at least 12 of the 14 within 5 % plus one point for
timing noise (1.06), measured side by side in one process (alternating, best of five rounds).  The margins are what the
spread between machines asks for: config 1's first pick (the per-tile kernel against the tuned object's streaming
kernel, 29 to 32 us) measured 1.04 on one box and 1.11 on another, two more configurations sit at 1.04 to 1.05.
Collected next to last on purpose: a timing bound that fails must not hide the parity tests.  Results are
compared with the tuned object's on the same inputs: 1e-12 (fp64) / 1e-5 (fp32) on |a-b| / max(|b|, rms(b))."""
import json
import os

import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"f64": 1e-12, "f32": 1e-5}


def configs():
    with open(os.path.join(ROOT, "cgo2019-ae_amd", "expressions", "manifest.json")) as f:
        return [e for e in json.load(f)["expressions"] if e["name"].startswith("cfg")]


def test_first_pick_of_the_mapping_pass_against_the_tuned_mappings(tools):
    import torch
    import cogent_mi355 as pkg
    driver = pkg.Driver()
    rows = []
    for e in configs():
        name, sizes = e["name"], e["bench_sizes"]
        tuned, model = pkg.Expression(name), pkg.Expression(path=os.path.join(pkg.LIB_DIR, "model_" + name + ".so"))
        assert model.info["spec"] and "spec" in tuned.info
        expr = helpers.parse_expression(pkg.expression_text(name))
        dtype = np.float64 if tuned.dtype == "f64" else np.float32
        nC, nA, nB = helpers.tensor_sizes(expr, sizes)
        dA = torch.from_numpy(tools.fill_uniform(np.empty(nA, dtype), 1)).cuda()
        dB = torch.from_numpy(tools.fill_uniform(np.empty(nB, dtype), 2)).cuda()
        print("[gpu] model pick %s %s: %s" % (name, sizes, model.info["spec"]), flush=True)
        # same result
        c_t, c_m = torch.zeros(nC, dtype=dA.dtype, device="cuda"), torch.zeros(nC, dtype=dA.dtype, device="cuda")
        assert tuned.run(sizes, c_t.data_ptr(), dA.data_ptr(), dB.data_ptr(), None, 0) == 0, tuned.last_error()
        assert model.run(sizes, c_m.data_ptr(), dA.data_ptr(), dB.data_ptr(), None, 0) == 0, model.last_error()
        torch.cuda.synchronize()
        rms = float(torch.sqrt(torch.mean(c_t * c_t)))
        err = float(torch.max(torch.abs(c_m - c_t) / torch.clamp(torch.abs(c_t), min=rms)))
        assert err <= TOL[tuned.dtype], (name, err)
        # time: rotate over enough copies of C that none of it stays in the 256 MB Infinity Cache between launches
        esize = 8 if tuned.dtype == "f64" else 4
        n_rot = max(2, min(8, int(1.2e9 // (nC * esize)) + 1))
        cs = [c_t, c_m] + [torch.zeros_like(c_t) for _ in range(n_rot - 2)]
        ptrs = [c.data_ptr() for c in cs]
        best = {"tuned": 1e30, "model": 1e30}
        for _ in range(5):
            for tag, ex in (("tuned", tuned), ("model", model)):
                st = driver.time(ex, sizes, ptrs, dA.data_ptr(), dB.data_ptr(), 30, 60)
                best[tag] = min(best[tag], st["mean_ms"] * 1e3)
        rows.append((name, best["tuned"], best["model"], best["model"] / best["tuned"], model.info["spec"]))
        print("      tuned %8.1f us   first pick %8.1f us   ratio %.3f" % rows[-1][1:4], flush=True)
        del cs, c_t, c_m, dA, dB
        torch.cuda.empty_cache()
    assert len(rows) == 14
    worst = max(rows, key=lambda r: r[3])
    assert worst[3] <= 1.15, worst
    assert sum(1 for r in rows if r[3] <= 1.06) >= 12, [(r[0], round(r[3], 3)) for r in rows if r[3] > 1.06]
