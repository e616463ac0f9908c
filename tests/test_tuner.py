"""The measured-mapping tuner (cogent_mi355/tuner.py): candidate selection, the cache file and its place in the
build's order of precedence run on the CPU; the measuring step runs on the GPU against candidates the build
compiled ahead of time.  The reference's counterpart is the rank override of its cost-model choice
(cogent/src/generators/configurations.py:285-289)."""
import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "cgo2019-ae_amd"))


def test_distinct_candidates_skip_repeats_of_one_tiling():
    from cogent_mi355 import tuner
    base = {"block_tile": [96, 96, 8], "waves": [2, 2], "x": [["d", 24]], "y": [["b", 24]], "k": [["e", 8]],
            "mfma": "v_mfma_f64_16x16x4_f64", "split_k": 1, "lds_layout": [0, 0]}
    cands = [dict(base, spec="a"), dict(base, spec="a2"), dict(base, waves=[4, 1], spec="b"), dict(base, split_k=2, spec="c")]
    assert [c["spec"] for c in tuner.distinct_candidates(cands, 5)] == ["a", "b", "c"]
    assert [c["spec"] for c in tuner.distinct_candidates(cands, 2)] == ["a", "b"]


def test_index_order_is_the_entry_points_size_order():
    from cogent_mi355 import tuner
    assert tuner.index_order("# note\nt3 [d,72,c,72,b,72,a,72] += sum(e,72) * t2 [b,e,a] * v2 [c,e,d];\n") == ["d", "c", "b", "a", "e"]
    assert tuner.index_order("t3 [a,48,b,48] -= sum(e,8,f,6) * t2 [a,e,f] * v2 [f,b,e];") == ["a", "b", "e", "f"]


def test_stream_shaped_candidates():
    """Shapes offered for the streaming kernel: whole rows of C on the X side, a whole small matrix on either side,
    both panels as the resident one; every one of them is either planned or refused with a message."""
    import cogent_mi355 as pkg
    from cogent_mi355 import tuner
    tools = pkg.HostTools()
    cand = {"x": [["d", 24], ["c", 4]], "y": [["b", 24], ["a", 4]], "k": [["e", 8]]}
    ext = dict(zip("dcbae", [72] * 5))
    specs = tuner.stream_shapes(cand, ext, "DOUBLE")
    assert "x=d:72,c:2;y=b:8,a:8;k=e:24;w=3x4;t=3x1;mi=0;st=3" in specs             # config 2's pinned mapping
    assert any(sp.endswith(";sy=1") for sp in specs) and len(specs) == len(set(specs)) <= 12
    text = pkg.expression_text("cfg2_f64")
    planned = 0
    for sp in specs:
        try:
            m = tools.plan(text, "DOUBLE", mapping_spec=sp).info["mapping"]
            assert m["stream"][0] == 3 and m["stream_resident"] == ("y" if sp.endswith("sy=1") else "x")
            planned += 1
        except pkg.CogentError as err:
            assert str(err)
    assert planned >= 4
    # one side a 72 x 72 matrix: the whole matrix becomes the panel, 72 padded to 80
    cand = {"x": [["a", 72]], "y": [["b", 8], ["c", 8], ["d", 1]], "k": [["e", 8]]}
    specs = tuner.stream_shapes(cand, dict(zip("abcde", [72] * 5)), "DOUBLE")
    assert any(sp.startswith("x=a:72;y=b:8,c:8,d:1;k=e:24;") for sp in specs)
    # nothing to offer when there is a single K block at every depth tried, or no summed index
    assert tuner.stream_shapes({"x": [["a", 64]], "y": [["b", 64]], "k": [["c", 4]]}, {"a": 64, "b": 64, "c": 4}, "FLOAT") == []


def test_prepared_set_of_the_build_is_complete():
    """build.py compiles the candidates of its TUNING_SETS; the index names one shared object per candidate."""
    import build
    for name, k in build.TUNING_SETS.items():
        d = os.path.join(ROOT, "cgo2019-ae_amd", "tuning", name)
        idx = json.load(open(os.path.join(d, "index.json")))
        assert idx["name"] == name and len(idx["candidates"]) >= k
        for c in idx["candidates"]:
            # a candidate is built, or was dropped because the kernel for the benchmark extents spills registers
            assert ("error" in c and "spills" in c["error"]) or os.path.exists(os.path.join(d, c["so"])), c
        assert sum(1 for c in idx["candidates"] if "so" in c) >= k
        assert len({c["spec"] for c in idx["candidates"]}) == len(idx["candidates"])


def test_build_prefers_pinned_then_tuned_then_model(tmp_path, monkeypatch):
    import build
    from cogent_mi355 import tuner
    entry = {"name": "x", "file": "cfg5_1_f64.in", "dtype": "DOUBLE", "bench_sizes": [16] * 7}
    monkeypatch.setattr(build, "EXPR", str(tmp_path))
    assert build.tuned_map(entry) is None                                   # no cache file
    key = tuner.cache_key(entry)
    assert key == "cfg5_1_f64.in|DOUBLE|16,16,16,16,16,16,16"
    (tmp_path / "tuned.json").write_text(json.dumps({key: {"map": "x=0:16;w=1x1", "mean_us": 1.0}}))
    assert build.tuned_map(entry) == "x=0:16;w=1x1"
    assert build.tuned_map(dict(entry, bench_sizes=[24] * 7)) is None       # other sizes: other key
    assert tuner.load_cache(str(tmp_path / "tuned.json"))[key]["map"] == "x=0:16;w=1x1"


@pytest.mark.gpu
def test_measure_times_verified_candidates_and_records_the_fastest(tmp_path):
    from cogent_mi355 import tuner
    cache = str(tmp_path / "tuned.json")
    print("[gpu] tuner.measure cfg5_1_f64", flush=True)
    rep = tuner.measure("cfg5_1_f64", warmup=2, iters=10, cache_path=cache)
    rows = rep["candidates"]
    dropped = [r for r in rows if "so" not in r]
    assert all("spills" in r["error"] for r in dropped), dropped               # the only reason a candidate may be missing
    rows = [r for r in rows if "so" in r]
    assert len(rows) >= 3 and all(r["ok"] for r in rows), rows
    assert all(r["max_rel_err"] <= 1e-12 for r in rows)
    best = min(rows, key=lambda r: r["mean_us"])
    assert rep["best"]["spec"] == best["spec"]
    assert 20.0 < best["mean_us"] < 500.0                                   # 269 MB of traffic: tens of microseconds
    saved = json.load(open(cache))
    assert saved["cfg5_1_f64.in|DOUBLE|16,16,16,16,16,16,16"]["map"] == best["spec"]


def test_every_cached_mapping_belongs_to_a_manifest_entry_and_still_plans():
    """expressions/tuned.json is keyed by file, element type and sizes: no stale keys, and every cached spec (and every
    spec pinned in manifest.json) is still accepted by the mapping pass for its expression."""
    import cogent_mi355 as pkg
    from cogent_mi355 import tuner
    tools = pkg.HostTools()
    entries = pkg.manifest()
    keys = {tuner.cache_key(e): e for e in entries}
    cache = tuner.load_cache()
    assert cache, "empty tuning cache"
    for key, rec in cache.items():
        assert key in keys, "stale cache key " + key
        e = keys[key]
        m = tools.plan(pkg.expression_text(e["name"]), e["dtype"], mapping_spec=rec["map"]).info["mapping"]
        assert m["threads"] <= 1024 and rec["mean_us"] > 0
    for e in entries:
        if e.get("map"):
            tools.plan(pkg.expression_text(e["name"]), e["dtype"], mapping_spec=e["map"])


def test_small_tile_shapes():
    """The 96x32 tile with the C tile through LDS for a 6-D shape at extents 24/16 (TCCG 34: X side a, d, f; Y side
    b, c, e; contracted g), both Y splits, each with and without non-temporal C; nothing for a long leading index."""
    from cogent_mi355 import tuner
    cand = {"x": [["a", 24], ["d", 4], ["f", 1]], "y": [["b", 16], ["c", 8], ["e", 1]], "k": [["g", 8]]}
    ext = dict(zip("abcdefg", [24, 16, 16, 24, 16, 16, 24]))
    specs = tuner.small_tile_shapes(cand, ext, "DOUBLE")
    assert specs == ["x=a:24,d:4,f:1;y=b:16,c:2,e:1;k=g:24;w=2x2;t=3x1;mi=0;cl=1",
                     "x=a:24,d:4,f:1;y=b:16,c:2,e:1;k=g:24;w=2x2;t=3x1;mi=0;cl=1;nt=3",
                     "x=a:24,d:4,f:1;y=b:8,c:4,e:1;k=g:24;w=2x2;t=3x1;mi=0;cl=1",
                     "x=a:24,d:4,f:1;y=b:8,c:4,e:1;k=g:24;w=2x2;t=3x1;mi=0;cl=1;nt=3",
                     # ... and the 192x32 tile on four wavefronts side by side
                     "x=a:24,d:8,f:1;y=b:8,c:4,e:1;k=g:24;w=4x1;t=3x2;mi=0;cl=1;to=1;vl=1",
                     "x=a:24,d:8,f:1;y=b:8,c:4,e:1;k=g:24;w=4x1;t=3x2;mi=0;cl=1;to=1;vl=1;nt=3"]
    assert tuner.small_tile_shapes({"x": [["a", 64], ["b", 1]], "y": [["c", 8], ["d", 8]], "k": [["e", 8]]},
                                   dict(zip("abcde", [72] * 5)), "DOUBLE") == []
