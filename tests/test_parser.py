"""The C++ expression parser against the reference grammar (cogent/src/algs/bases/tc_gen_inputs.py:29-108).

Accept-fixtures: the 48 TCCG expressions, the BASELINE configs and the README example, each compared
with an independent positional reading in tests/helpers.py and, for a few, with hand-checked lists.
Reject-fixtures: the inputs on which the reference raises or silently mis-parses.
"""
import glob
import os

import pytest

import helpers

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXPR_DIR = os.path.join(ROOT, "cgo2019-ae_amd", "expressions")
FILES = sorted(p for p in glob.glob(os.path.join(EXPR_DIR, "*.in")) if not os.path.basename(p).startswith("fused_"))   # groups: tests/test_groups.py


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(p) for p in FILES])
def test_corpus_file_parses_like_the_positional_reading(path, tools):
    text = open(path).read()
    want = helpers.parse_expression(text)
    got = tools.plan(text, "DOUBLE").info
    assert got["out"] == want["out"] and got["a"] == want["a"] and got["b"] == want["b"]
    assert got["op"] == want["op"]
    assert got["out_idx"] == want["out_idx"] and got["sum_idx"] == want["sum_idx"]
    assert got["a_idx"] == want["a_idx"] and got["b_idx"] == want["b_idx"]
    assert got["rep_sizes"] == want["rep_sizes"]


def test_corpus_is_complete():
    names = {os.path.basename(p) for p in FILES}
    assert {"tccg_%02d.in" % n for n in range(1, 49)} <= names
    assert {"cfg1_f64.in", "cfg2_f64.in", "cfg3_f64.in", "cfg4_f32.in"} <= names
    assert {"cfg5_%d_f64.in" % n for n in range(1, 10)} <= names


def test_hand_checked_lists(tools):
    # the README's example line
    p = tools.plan("t3 [a,16,b,16,c,16,d,16] += sum(e,16,f,16) * t2 [a,e,b,f] * v2 [d,f,c,e];", "DOUBLE").info
    assert (p["out"], p["a"], p["b"], p["op"]) == ("t3", "t2", "v2", "+=")
    assert p["out_idx"] == ["a", "b", "c", "d"] and p["sum_idx"] == ["e", "f"]
    assert p["a_idx"] == ["a", "e", "b", "f"] and p["b_idx"] == ["d", "f", "c", "e"]
    assert p["rep_sizes"] == [16] * 6
    # TCCG-1 at its benchmark sizes, "-=" and multi-character index names
    p = tools.plan("t3 [a,312,b,312,c,24] -= sum(d,312) * t2 [b,d,a] * v2 [d,c];", "FLOAT").info
    assert p["op"] == "-=" and p["rep_sizes"] == [312, 312, 24, 312]
    p = tools.plan("t3 [h3,4,h2,5,p6,6] += sum(p7,7) * x1 [p7,h3] * y2 [h2,p7,p6];", "DOUBLE").info
    assert p["out_idx"] == ["h3", "h2", "p6"] and p["sum_idx"] == ["p7"] and p["b_idx"] == ["h2", "p7", "p6"]


def test_comment_lines_are_skipped(tools):
    text = "# abc-bda-dc\n# needs sizes\nt3 [a,8,b,8,c,8] += sum(d,8) * t2 [b,d,a] * v2 [d,c];\n"
    assert tools.plan(text, "DOUBLE").info["out_idx"] == ["a", "b", "c"]


REJECTS = [
    ("", "no expression"),
    ("# only a comment\n", "no expression"),
    ("\n", "empty expression line"),                                          # tc_gen_inputs.py:48 raises on a blank line
    ("t3 [a,8,b,8] += sum(c,8) * t2 [a,c]\n", "ten"),                         # fewer than ten fields
    ("t3 [a,b,c] += sum(d) * t2 [b,d,a] * v2 [d,c];", "representative"),      # the old size-less format (ccsd_t/*.in)
    ("t3 [a,8,b] += sum(c,8) * t2 [a,c] * v2 [c,b];", "representative"),      # odd idx/size list
    ("t3 [a,8,b,x] += sum(c,8) * t2 [a,c] * v2 [c,b];", "not an integer"),
    ("t3 [a,8,b,8] += sum(c,8.5) * t2 [a,c] * v2 [c,b];", "not an integer"),
    ("t3 [a,8,b,0] += sum(c,8) * t2 [a,c] * v2 [c,b];", "positive"),
    ("t3 [a,8,b,8] = sum(c,8) * t2 [a,c] * v2 [c,b];", "operator"),
    ("t3 [a,8,b,8] += sum(c,8) * t2 [a,q] * v2 [c,b];", "neither"),           # unknown input index
    ("t3 [a,8,b,8] += sum(c,8) * t2 [a,c] * v2 [c,a];", "exactly one input"), # b nowhere, a twice
    ("t3 [a,8,b,8] += sum(c,8) * t2 [a,c] * v2 [b];", "both inputs"),
    ("t3 [a,8,a,8] += sum(c,8) * t2 [a,c] * v2 [c,a];", "twice"),
    ("t3 [a, 8, b, 8] += sum(c,8) * t2 [a,c] * v2 [c,b];", ""),               # blanks inside a list shift the fields
]


@pytest.mark.parametrize("text,needle", REJECTS)
def test_rejected_inputs(text, needle, tools):
    import cogent_mi355
    with pytest.raises(cogent_mi355.CogentError) as e:
        tools.plan(text, "DOUBLE")
    assert e.value.code == 1
    assert needle in str(e.value)


def test_other_plan_errors(tools):
    import cogent_mi355
    good = "t3 [a,8,b,8] += sum(c,8) * t2 [a,c] * v2 [c,b];"
    with pytest.raises(cogent_mi355.CogentError) as e:
        tools.plan(good, "HALF")
    assert e.value.code == 2
    with pytest.raises(cogent_mi355.CogentError) as e:
        tools.plan(good + "\n" + good, "DOUBLE")
    assert e.value.code == 4
    with pytest.raises(cogent_mi355.CogentError) as e:
        tools.plan(good, "DOUBLE", mapping_spec="x=a:8;y=b:8;k=c:8;w=1x1;t=9x9")
    assert e.value.code == 3


def test_operation_and_byte_counts(tools):
    """Known answers: the operation counts printed in the reference's result files
    (cogent/expect_p100_cogent_tccg_results.txt:1, :9, :20, :31) = 2 * product of extents."""
    def plan(n):
        return tools.plan(open(os.path.join(EXPR_DIR, "tccg_%02d.in" % n)).read(), "DOUBLE")
    assert plan(1).flops([312, 312, 24, 312]) == 1457823744
    assert plan(9).flops([72] * 5) == 3869835264
    assert plan(20).flops([72] * 6) == 278628139008
    assert plan(31).flops([24, 16, 16, 24, 16, 16, 24]) == 1811939328
    # algorithmic bytes = sizeof(T) * (|A| + |B| + 2|C|)
    c1 = tools.plan(open(os.path.join(EXPR_DIR, "cfg1_f64.in")).read(), "DOUBLE")
    assert c1.bytes([32, 256, 256, 256]) == 167837696 and c1.flops([32, 256, 256, 256]) == 1073741824
    c4 = tools.plan(open(os.path.join(EXPR_DIR, "cfg4_f32.in")).read(), "FLOAT")
    assert c4.bytes([24] * 7) == 1531478016 and c4.bytes([16] * 7) == 134742016
