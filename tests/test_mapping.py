"""Invariants of the gfx950 index-to-tile mapping pass (the counterpart of the reference's
enumeration + cost model + selection; no equality with the reference's pick is claimed, its
mapping targets warp-32 CUDA).  Checked for every expression of the corpus in both element types."""
import glob
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXPR_DIR = os.path.join(ROOT, "cgo2019-ae_amd", "expressions")
FILES = sorted(p for p in glob.glob(os.path.join(EXPR_DIR, "*.in")) if not os.path.basename(p).startswith("fused_"))   # groups: tests/test_groups.py
MT = {"v_mfma_f64_16x16x4_f64": (16, 4), "v_mfma_f32_16x16x4_f32": (16, 4), "v_mfma_f32_32x32x2_f32": (32, 2)}


def check_mapping(info, m, dtype):
    ext = dict(zip(info["out_idx"] + info["sum_idx"], info["rep_sizes"]))
    x_op = info["a_idx"] if m["x_operand"] == info["a"] else info["b_idx"]
    y_op = info["b_idx"] if m["x_operand"] == info["a"] else info["a_idx"]
    xs, ys, ks = [n for n, _ in m["x"]], [n for n, _ in m["y"]], [n for n, _ in m["k"]]
    # every index mapped exactly once, on the right side
    assert sorted(xs + ys + ks) == sorted(ext)
    assert set(xs) == {i for i in x_op if i in info["out_idx"]}
    assert set(ys) == {i for i in y_op if i in info["out_idx"]}
    assert set(ks) == set(info["sum_idx"])
    # the X side is the input that holds the output's fastest index, and that index leads its tile list
    assert info["out_idx"][0] in x_op and xs[0] == info["out_idx"][0]
    mt, kstep = MT[m["mfma"]]
    assert (dtype == "DOUBLE") == m["mfma"].startswith("v_mfma_f64")
    prod = lambda side: eval("*".join(str(t) for _, t in side) or "1")
    bx, by, bk = m["block_tile"]
    assert (bx, by, bk) == (prod(m["x"]), prod(m["y"]), prod(m["k"]))
    for name, t in m["x"] + m["y"] + m["k"]:
        assert 1 <= t
    px, py, pk = m["padded"]
    wx, wy = m["waves"]
    tx, ty = m["mfma_tiles_per_wave"]
    assert px == wx * tx * mt >= bx and py == wy * ty * mt >= by and pk >= bk and pk % kstep == 0
    assert m["threads"] == 64 * wx * wy and 64 <= m["threads"] <= 1024
    assert m["lds_bytes"] <= 64 * 1024
    blocks = 1
    for name, t in m["x"] + m["y"]:
        blocks *= -(-ext[name] // t)
    assert m["model"]["blocks"] == blocks * m["split_k"]         # split K: that many workgroups per output tile
    ksteps = 1
    for name, t in m["k"]:
        ksteps *= -(-ext[name] // t)
    assert m["model"]["k_steps"] == -(-ksteps // m["split_k"])    # K blocks per workgroup
    assert m["model"]["cost_us"] > 0


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(p) for p in FILES])
@pytest.mark.parametrize("dtype", ["DOUBLE", "FLOAT"])
def test_chosen_mapping_invariants(path, dtype, tools):
    plan = tools.plan(open(path).read(), dtype)
    check_mapping(plan.info, plan.info["mapping"], dtype)


def test_candidates_are_sorted_and_admissible(tools):
    plan = tools.plan(open(os.path.join(EXPR_DIR, "cfg5_3_f64.in")).read(), "DOUBLE")
    cands = plan.candidates(200)
    assert len(cands) > 20
    costs = [c["model"]["cost_us"] for c in cands]
    assert costs == sorted(costs)
    for c in cands:
        check_mapping(plan.info, c, "DOUBLE")
    assert cands[0]["spec"] == plan.info["mapping"]["spec"]


def test_manual_rank_and_spec_round_trip(tools):
    text = open(os.path.join(EXPR_DIR, "cfg2_f64.in")).read()
    auto = tools.plan(text, "DOUBLE")
    cands = auto.candidates(5)
    third = tools.plan(text, "DOUBLE", config_rank=2)          # the reference's manual pick
    assert third.info["mapping"]["spec"] == cands[2]["spec"]
    same = tools.plan(text, "DOUBLE", mapping_spec=cands[2]["spec"])
    assert same.info["mapping"] == third.info["mapping"]
    named = tools.plan(text, "DOUBLE", mapping_spec="x=d:24,c:4;y=b:24,a:4;k=e:8;w=2x2;t=3x3")
    assert named.info["mapping"]["block_tile"] == [96, 96, 8] and named.info["mapping"]["threads"] == 256


def test_kernel_options_in_a_spec(tools):
    """pd= (K blocks requested ahead), nt= (non-temporal C: bit 0 loads, bit 1 stores), sw= (fp32: C's fastest
    index on the MFMA rows), lc=, mw=, sk= are carried into the plan and back out through its spec."""
    text = open(os.path.join(EXPR_DIR, "cfg2_f64.in")).read()
    base = "x=d:24,c:4;y=b:24,a:4;k=e:8;w=2x2;t=3x3"
    m = tools.plan(text, "DOUBLE", mapping_spec=base).info["mapping"]
    assert m["prefetch_depth"] == 1 and m["swapped_roles"] == 0 and m["nontemporal_c"] == 0   # 192-byte rows
    m = tools.plan(text, "DOUBLE", mapping_spec=base + ";pd=3;nt=2;mw=2;lc=1").info["mapping"]
    assert m["prefetch_depth"] == 3 and m["nontemporal_c"] == 2 and m["min_waves_per_simd"] == 2 and m["late_c"] == 1
    assert "pd=3" in m["spec"] and "nt=2" in m["spec"]
    again = tools.plan(text, "DOUBLE", mapping_spec=m["spec"]).info["mapping"]
    assert again == m
    # es=1: the first slices requested before the C tile is staged through LDS (an option of cl=1 mappings; off by default)
    small = "x=d:24,c:4;y=b:8,a:4;k=e:8;w=2x2;t=3x1"                      # a 24 KB tile: cl=1 needs at most 64 KB
    m = tools.plan(text, "DOUBLE", mapping_spec=small + ";cl=1").info["mapping"]
    assert m["c_through_lds"] == 1 and m["early_slices"] == 0 and "es=" not in m["spec"]
    m = tools.plan(text, "DOUBLE", mapping_spec=small + ";cl=1;es=1").info["mapping"]
    assert m["early_slices"] == 1 and m["spec"].endswith(";es=1")
    assert tools.plan(text, "DOUBLE", mapping_spec=m["spec"]).info["mapping"] == m
    # ok=0: single K blocks with ragged tiles through the K-loop kernels; not with split K
    m = tools.plan(text, "DOUBLE", mapping_spec=base + ";ok=0").info["mapping"]
    assert m["one_block_ragged"] == 0 and m["spec"].endswith(";ok=0")
    assert tools.plan(text, "DOUBLE", mapping_spec=base).info["mapping"]["one_block_ragged"] == 1
    with pytest.raises(Exception, match="exclude"):
        tools.plan(text, "DOUBLE", mapping_spec=base + ";sk=2;ok=0")
    # rx=/ry=: an input copied into tile order first; its slices then go to LDS K-major whatever its own order
    m = tools.plan(text, "DOUBLE", mapping_spec="x=d:72,c:2;y=b:24,a:2;k=e:12;w=3x1;t=3x3;rx=1;ry=1").info["mapping"]
    assert m["repack"] == [1, 1] and m["lds_layout"] == [0, 0] and "rx=1" in m["spec"] and "ry=1" in m["spec"]
    assert tools.plan(text, "DOUBLE").info["mapping"]["repack"] == [0, 0]      # never chosen automatically
    # no=: non-temporal loads of an input (bit 0 X side, bit 1 Y side), opt-in
    m = tools.plan(text, "DOUBLE", mapping_spec=base + ";no=2").info["mapping"]
    assert m["nontemporal_inputs"] == 2 and "no=2" in m["spec"]
    assert tools.plan(text, "DOUBLE", mapping_spec=base).info["mapping"]["nontemporal_inputs"] == 0
    # vl=1: slice loads of 8/16 bytes per lane along the operand's fastest index (opt-in)
    m = tools.plan(text, "DOUBLE", mapping_spec=base + ";vl=1").info["mapping"]
    assert m["vector_slice_loads"] == 1 and "vl=1" in m["spec"]
    assert tools.plan(text, "DOUBLE", mapping_spec=base).info["mapping"]["vector_slice_loads"] == 0
    # db=1: two LDS stages in dynamic LDS when together they exceed the 64 KB a static array may have
    text22 = open(os.path.join(EXPR_DIR, "tccg_22.in")).read()
    big = "x=0:24,2:8;y=1:72,3:2;k=5:8,4:2;w=4x3;t=3x3"
    m0 = tools.plan(text22, "DOUBLE", mapping_spec=big).info["mapping"]
    m1 = tools.plan(text22, "DOUBLE", mapping_spec=big + ";db=1").info["mapping"]
    assert m0["dynamic_lds_stages"] == 0 and m1["dynamic_lds_stages"] == 1 and "db=1" in m1["spec"]
    # so=1: with split K, the K shares as the outermost level of the grid (opt-in)
    text13 = open(os.path.join(EXPR_DIR, "tccg_13.in")).read()
    sk = "x=a:156;y=b:148;k=d:8,c:2;w=2x2;t=5x5;sk=64"
    m0 = tools.plan(text13, "DOUBLE", mapping_spec=sk).info["mapping"]
    m1 = tools.plan(text13, "DOUBLE", mapping_spec=sk + ";so=1").info["mapping"]
    assert m0["split_k_outermost"] == 0 and m1["split_k_outermost"] == 1 and "so=1" in m1["spec"] and "so=" not in m0["spec"]
    assert tools.plan(text13, "DOUBLE", mapping_spec=m1["spec"]).info["mapping"] == m1
    assert 32768 < m1["lds_bytes"] <= 65536                                    # one stage fits a static array, two do not
    # cl=1: the C tile passes through LDS in memory order (opt-in; refused silently when the tile is too large)
    m = tools.plan(text, "DOUBLE", mapping_spec="x=d:8,c:8;y=b:24,a:2;k=e:8;w=2x1;t=2x3;cl=1").info["mapping"]
    assert m["c_through_lds"] == 1 and "cl=1" in m["spec"]
    assert tools.plan(text, "DOUBLE", mapping_spec=base + ";cl=1").info["mapping"]["c_through_lds"] == 0   # 96x96x8 B > 64 KB
    # fp32 with a fastest tile that is a multiple of 4: swapped roles by default, sw=0 turns them off
    text4 = open(os.path.join(EXPR_DIR, "cfg4_16_f32.in")).read()
    auto = tools.plan(text4, "FLOAT", mapping_spec="x=0:16,2:16,4:1;y=1:16,3:2,5:1;k=6:16;w=4x1;t=4x2;mi=1").info["mapping"]
    assert auto["swapped_roles"] == 1 and auto["nontemporal_c"] == 0           # 64-byte rows: no whole lines per access
    # the pass's own pick for this shape (one K block, rows that are not whole lines): C through LDS in memory order,
    # whose tile is made of whole lines, tiles in C's memory order, 16-byte slice loads on the side whose runs reach 64
    # bytes (the Y input's 16 floats; the X input's runs are 8 floats here)
    pick = tools.plan(text4, "FLOAT").info["mapping"]
    assert pick["c_through_lds"] == 1 and pick["tile_order_c_memory"] == 1 and pick["vector_slice_loads"] == 3 and pick["stream"][0] == 0
    off = tools.plan(text4, "FLOAT", mapping_spec=auto["spec"] + ";sw=0").info["mapping"]
    assert off["swapped_roles"] == 0
    # fp64 rows of 16 elements are whole aligned lines: non-temporal loads and stores
    text5 = open(os.path.join(EXPR_DIR, "cfg5_1_f64.in")).read()
    assert tools.plan(text5, "DOUBLE").info["mapping"]["nontemporal_c"] == 3
    # a fastest tile that is not a multiple of 4 cannot use 128-bit accesses
    odd = tools.plan("t3 [a,30,b,64] += sum(c,64) * t2 [a,c] * v2 [c,b];", "FLOAT",
                     mapping_spec="x=a:30;y=b:32;k=c:8;w=1x1;t=2x2;mi=1").info["mapping"]
    assert odd["swapped_roles"] == 0


def test_streaming_kernel_option(tools, tmp_path):
    """st=<depth>: the object also gets the panel-resident streaming kernel, compiled for the K-block count of the
    representative extents; refused when tiles do not divide the extents, need padding, the depth does not divide
    the K-block count, there is a single K block, or the X panel does not fit the LDS of a CU."""
    text = open(os.path.join(EXPR_DIR, "cfg2_f64.in")).read()
    base = "x=d:24,c:4;y=b:24,a:4;k=e:8;w=2x2;t=3x3"
    assert tools.plan(text, "DOUBLE", mapping_spec=base).info["mapping"]["stream"] == [0, 1]
    m = tools.plan(text, "DOUBLE", mapping_spec=base + ";st=3").info["mapping"]
    assert m["stream"] == [9, 3] and "st=3" in m["spec"]
    assert tools.plan(text, "DOUBLE", mapping_spec=m["spec"]).info["mapping"] == m
    m = tools.plan(text, "DOUBLE", mapping_spec="x=d:72,c:2;y=b:8,a:8;k=e:24;w=3x4;t=3x1;st=1").info["mapping"]
    assert m["stream"] == [3, 1]
    assert m["stream_resident"] == "x"
    m = tools.plan(text, "DOUBLE", mapping_spec="x=d:72,c:2;y=b:8,a:8;k=e:24;w=3x4;t=3x1;st=3;sy=1").info["mapping"]
    assert m["stream_resident"] == "y" and "sy=1" in m["spec"]
    # the streaming kernel's own options round-trip through the spec: interleaved runs, the panel behind the first
    # tile, C read two tiles ahead; 16-byte slice loads per side
    m = tools.plan(text, "DOUBLE", mapping_spec="x=d:72,c:2;y=b:8,a:8;k=e:24;w=3x4;t=3x1;st=3;il=1;ov=1;cd=2;vl=2").info["mapping"]
    assert (m["stream_interleaved_runs"], m["stream_panel_overlap"], m["stream_c_distance"], m["vector_slice_loads"]) == (1, 1, 2, 2)
    assert all(k in m["spec"] for k in ("il=1", "ov=1", "cd=2", "vl=2"))
    assert tools.plan(text, "DOUBLE", mapping_spec=m["spec"]).info["mapping"] == m
    # tiles padded to the MFMA granularity are allowed (a 72-wide side runs as 80)
    text9 = open(os.path.join(EXPR_DIR, "tccg_09.in")).read()
    m = tools.plan(text9, "DOUBLE", mapping_spec="x=a:72;y=b:8,c:8,d:1;k=e:24;w=1x4;t=5x1;st=3").info["mapping"]
    assert m["stream"] == [3, 3] and m["padded"][0] == 80 and m["block_tile"][0] == 72
    out = os.path.join(str(tmp_path), "st.hip")
    tools.plan(text, "DOUBLE", mapping_spec=base + ";st=3").emit("st_test", out)
    src = open(out).read()
    assert "STREAM = 9, SPD = 3, SMW = 2" in src and "cogent_last_kernel" in src
    for bad, why in ((base + ";st=2", "divides"),                                             # 9 K blocks
                     ("x=d:24,c:4;y=b:24,a:4;k=e:36;w=2x2;t=3x3;st=3", "divides"),            # 2 K blocks
                     ("x=d:16,c:4;y=b:24,a:4;k=e:8;w=2x2;t=2x3;st=3", "divide"),              # 16 does not divide 72
                     ("x=d:72,c:4;y=b:8,a:4;k=e:8;w=6x2;t=3x1;st=3", "LDS"),                  # a 288 x 72 panel of doubles
                     (base + ";st=3;sk=2", "exclude"),                                         # K shares: every tile has ONE workgroup here
                     (base + ";sk=3;st=3", "exclude")):
        with pytest.raises(Exception) as err:
            tools.plan(text, "DOUBLE", mapping_spec=bad)
        assert why in str(err.value), (bad, str(err.value))
    text4 = open(os.path.join(EXPR_DIR, "cfg4_f32.in")).read()
    with pytest.raises(Exception) as err:                                                     # one K block
        tools.plan(text4, "FLOAT", mapping_spec="x=0:24,2:8,4:1;y=1:24,3:2,5:1;k=6:24;w=4x1;t=3x3;mi=1;st=1")
    assert "K blocks" in str(err.value)


BAD_SPECS = [
    "x=d:24;y=b:24,a:4;k=e:8;w=2x2;t=3x3",                # c unmapped
    "x=d:24,c:4,b:2;y=a:4;k=e:8;w=2x2;t=3x3",             # b on the wrong side
    "x=d:24,c:4;y=b:24,a:4;k=e:8;w=8x8;t=1x1",            # 4096 threads
    "x=d:72,c:8;y=b:72,a:8;k=e:72;w=4x4;t=9x9",           # LDS and registers
    "x=d:24,c:4;y=b:24,a:4;k=e:8;w=2x2;t=3x3;mi=1",       # fp32 instruction for fp64 data
    "x=d:24,c:4;y=b:24,a:4;k=e:8;w=1x1;t=1x1",            # wavefront tiling smaller than the block tile
]


def test_register_budget_of_specs_and_of_the_enumeration(tools):
    """The enumeration keeps the accumulators within half a wavefront's register share (at most 16 fp64 MFMA
    tiles); a spec may take all but 56 registers of the share: 5x5 tiles on four wavefronts (200 of 512) and
    3x4 on twelve (96 of 170) pass, 3x6 on twelve (144 of 170) and 6x6 on four (288 > 256) do not."""
    import cogent_mi355
    text13 = open(os.path.join(EXPR_DIR, "tccg_13.in")).read()
    plan = tools.plan(text13, "DOUBLE")
    for c in plan.candidates(300):
        tx, ty = c["mfma_tiles"] if "mfma_tiles" in c else [int(v) for v in c["spec"].split(";t=")[1].split(";")[0].split("x")]
        wx, wy = [int(v) for v in c["spec"].split(";w=")[1].split(";")[0].split("x")]
        share = min(512, 512 // -(-(wx * wy) // 4))
        assert tx * ty * 8 * 2 <= share, c["spec"]
    ok = tools.plan(text13, "DOUBLE", mapping_spec="x=a:156;y=b:148;k=d:8,c:2;w=2x2;t=5x5;sk=64").info["mapping"]
    assert "t=5x5" in ok["spec"]
    text22 = open(os.path.join(EXPR_DIR, "tccg_22.in")).read()
    tools.plan(text22, "DOUBLE", mapping_spec="x=a:24,c:8;y=b:24,d:8;k=f:8,e:1;w=4x3;t=3x4;pd=2")
    for text, bad in ((text22, "x=a:24,c:8;y=b:72,d:4;k=f:8,e:1;w=4x3;t=3x6"),          # 144 of 170
                      (text13, "x=a:156;y=b:148;k=d:8,c:2;w=2x2;t=6x6;sk=64")):          # 288 accumulator registers
        with pytest.raises(cogent_mi355.CogentError) as e:
            tools.plan(text, "DOUBLE", mapping_spec=bad)
        assert e.value.code == 3 and "register" in str(e.value)


@pytest.mark.parametrize("spec", BAD_SPECS)
def test_impossible_mappings_are_rejected(spec, tools):
    import cogent_mi355
    text = open(os.path.join(EXPR_DIR, "cfg2_f64.in")).read()
    with pytest.raises(cogent_mi355.CogentError) as e:
        tools.plan(text, "DOUBLE", mapping_spec=spec)
    assert e.value.code == 3


def _pick(tools, name, dtype="DOUBLE"):
    return tools.plan(open(os.path.join(EXPR_DIR, name)).read(), dtype).info["mapping"]


def test_first_picks_follow_the_measured_rules(tools):
    """What the pass decides on its own (no spec, no tuned table), pinned where a measurement stands behind it."""
    # config 2: whole aligned chunks of C (two full rows of d: 1152 bytes) and the streaming kernel at three K blocks
    m = _pick(tools, "cfg2_f64.in")
    assert m["x"] == [["d", 72], ["c", 2]] and m["k"] == [["e", 24]] and m["stream"] == [3, 3]
    assert m["nontemporal_c"] == 3 and m["stream_interleaved_runs"] == 1 and m["stream_panel_overlap"] == 1
    # the 6-D shapes keep a 24- or 16-deep contracted index in ONE K block; tiles then go out in C's memory order with
    # 16-byte slice loads, and C passes through LDS where its rows are not whole 128-byte lines (192 bytes here)
    m = _pick(tools, "tccg_31.in")
    assert m["k"] == [["g", 24]] and m["model"]["k_steps"] == 1 and m["stream"][0] == 0
    assert m["tile_order_c_memory"] == 1 and m["c_through_lds"] == 1 and m["nontemporal_c"] == 3
    # no 16-byte slice loads: one input has 32-byte runs, the other's 32x24 slice would fill two rounds of 256 lanes half
    assert m["vector_slice_loads"] == 0
    m = _pick(tools, "tccg_32.in")                    # its 48x24 slice with 192-byte runs: three 16-byte rounds against five
    assert m["vector_slice_loads"] == 2
    m = _pick(tools, "cfg5_1_f64.in")                                  # 128-byte rows: no LDS copy of C; 128-byte runs in both inputs
    assert m["model"]["k_steps"] == 1 and m["tile_order_c_memory"] == 1 and m["c_through_lds"] == 0 and m["vector_slice_loads"] == 1
    # a K loop with 192-byte rows of C: C through LDS there too; no tile-order option on a K loop
    m = _pick(tools, "tccg_03.in")
    assert m["model"]["k_steps"] > 1 and m["c_through_lds"] == 1 and m["tile_order_c_memory"] == 0
    # fp32 never gets the streaming kernel from the pass, nor does a shape with other than three K blocks
    assert _pick(tools, "cfg4_16_f32.in", "FLOAT")["stream"][0] == 0
    assert _pick(tools, "cfg1_f64.in")["stream"][0] == 0
    # a long MFMA-bound K loop with small slice shares: a second K block in flight
    m = _pick(tools, "tccg_20.in")
    assert m["prefetch_depth"] == 2 and m["split_k"] == 1
    # ... and where the pick has deep K blocks with one ahead, the same tile is emitted with 8-deep blocks and two ahead
    # (the ranked list itself is untouched: rank 0 asked for by number is the 24-deep mapping)
    m = _pick(tools, "cfg3_f64.in")
    assert m["k"] == [["e", 8], ["f", 1]] and m["prefetch_depth"] == 2 and m["split_k"] == 2
    ranked0 = tools.plan(open(os.path.join(EXPR_DIR, "cfg3_f64.in")).read(), "DOUBLE", config_rank=0).info["mapping"]
    assert ranked0["k"] == [["e", 24], ["f", 1]] and ranked0["prefetch_depth"] == 1
    assert (ranked0["x"], ranked0["y"], ranked0["waves"]) == (m["x"], m["y"], m["waves"])
    m = _pick(tools, "tccg_16.in")
    assert m["k"] == [["d", 8]] and m["prefetch_depth"] == 2
    # not where a second contracted index is an input's fastest one (its tile would drop to 1) ...
    m = _pick(tools, "tccg_30.in")
    assert m["prefetch_depth"] == 1 and dict(map(tuple, m["k"]))["e"] > 1
    # ... nor on a memory-bound shape
    m = _pick(tools, "tccg_05.in")
    assert m["k"] == [["e", 12]] and m["prefetch_depth"] == 1


BENCH_FILES = [p for p in FILES if os.path.basename(p).startswith(("cfg", "tccg_", "ccsd_"))]


@pytest.mark.parametrize("path", BENCH_FILES, ids=[os.path.basename(p) for p in BENCH_FILES])
def test_first_pick_has_whole_tiles(path, tools):
    """On the benchmark expressions whose extents are 16, 24, 32, 48, 72 or 256 every first pick divides the representative
    extents, so that calls at those extents take the kernel variants without predicates (312 and 296 have no divisor that
    is a multiple of the 16-wide matrix tile: there a ragged tile can be the better trade), and no workgroup has 6 or 9
    wavefronts (which load the four SIMDs unevenly: +40 % measured)."""
    text = open(path).read()
    for dtype in (("FLOAT",) if path.endswith("_f32.in") else ("DOUBLE",)):          # the data type the object is shipped in
        info = tools.plan(text, dtype).info
        m = info["mapping"]
        ext = dict(zip(info["out_idx"] + info["sum_idx"], info["rep_sizes"]))
        if not set(ext.values()) <= {16, 24, 32, 48, 72, 256}:
            return
        for name, tile in m["x"] + m["y"] + m["k"]:
            assert ext[name] % tile == 0, (name, tile, ext[name], m["spec"])
        assert m["threads"] // 64 not in (6, 9), m["spec"]
