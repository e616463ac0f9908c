"""Host tools under AddressSanitizer + UndefinedBehaviorSanitizer (bin/cogent_gen_san, built by build.py): the parser,
the mapping pass, the spec reader and the emitter are run over the whole corpus and over malformed input; a sanitizer
report or a crash fails the test.  (The reference runs no sanitizer; its generator exits with a Python traceback on
such input, cogent/src/algs/bases/tc_gen_inputs.py:48-64.)"""
import glob
import os
import random
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "cgo2019-ae_amd")
GEN = os.path.join(PKG, "bin", "cogent_gen_san")
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:exitcode=99", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1:exitcode=98")


def gen(args, cwd):
    r = subprocess.run([GEN] + args, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=ENV, timeout=120)
    assert "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, (args, r.stderr[-2000:])
    assert r.returncode not in (98, 99) and r.returncode >= 0, (args, r.returncode, r.stderr[-500:])     # negative: killed by a signal
    return r


def test_corpus_through_the_sanitized_generator(tmp_path):
    files = sorted(glob.glob(os.path.join(PKG, "expressions", "*.in")))
    assert len(files) > 80
    # (the enumeration of a large expression takes seconds under the sanitizers: every BASELINE, random, small-K and
    # fused file, every fourth TCCG one; the candidate listing on three)
    files = [f for f in files if not os.path.basename(f).startswith("tccg_") or int(os.path.basename(f)[5:7]) % 4 == 1]
    for k, f in enumerate(files):
        dtype = "FLOAT" if "f32" in f else "DOUBLE"
        r = gen(["7", f, "-1", "-1", dtype, "-o", str(tmp_path / "o.hip"), "--json"] + (["--list", "5"] if k < 3 else []), tmp_path)
        assert r.returncode == 0, (f, r.stderr)
    # every mapping the build ships (pinned or tuned) through the spec reader
    import json
    m = json.load(open(os.path.join(PKG, "expressions", "manifest.json")))
    tuned = json.load(open(os.path.join(PKG, "expressions", "tuned.json")))
    specs = [(e["file"], e["dtype"], e["map"]) for e in m["expressions"] if e.get("map")]
    specs += [(k.split("|")[0], k.split("|")[1], v["map"]) for k, v in tuned.items()]
    for f, dtype, spec in specs:                 # (a given spec is not enumerated: milliseconds each)
        r = gen(["7", os.path.join(PKG, "expressions", f), "-1", "-1", dtype, "-o", str(tmp_path / "o.hip"), "--map", spec], tmp_path)
        assert r.returncode == 0, (f, spec, r.stderr)


MALFORMED = [
    "", "\n\n", "#only a comment\n", "t3", "t3 [a,16", "t3 [a,16] += sum() * t2 [a] * v2 [];",
    "t3 [a,16,b,16] += sum(c,16) * t2 [a,c] * v2 [c,b] extra tokens here;",
    "t3 [a,16,b,16] *= sum(c,16) * t2 [a,c] * v2 [c,b];",
    "t3 [a,-4,b,16] += sum(c,16) * t2 [a,c] * v2 [c,b];",
    "t3 [a,99999999999999999999,b,16] += sum(c,16) * t2 [a,c] * v2 [c,b];",
    "t3 [a,16,a,16] += sum(c,16) * t2 [a,c] * v2 [c,a];",
    "t3 [a,16,b,16] += sum(c,16) * t2 [a,z] * v2 [c,b];",
    "t3 [a,16,b,16] += sum(c,0) * t2 [a,c] * v2 [c,b];",
    "t3 [" + ",".join("i%d,2" % i for i in range(40)) + "] += sum(k,2) * t2 [i0,k] * v2 [k,i1];",
    "t3 [a,16,b,16] += sum(c,16) * t2 [a,c] * v2 [c,b];\nt3 [a,16,b,16] += sum(c,8) * t2 [a,c] * v2 [c,b];",
    "t3 [a,16,b,16] += sum(c,16) * t2 [a,c] * v2 [c,b];" + "x" * 100000,
    "\x00\x01\x02 [a,16] += sum(c,4) * \xff [a,c] * v2 [c];",
]


@pytest.mark.parametrize("k", range(len(MALFORMED)))
def test_malformed_expressions_are_refused_cleanly(k, tmp_path):
    f = tmp_path / "bad.in"
    f.write_text(MALFORMED[k], errors="surrogateescape") if "\xff" not in MALFORMED[k] else f.write_bytes(MALFORMED[k].encode("latin-1"))
    for dtype in ("DOUBLE", "HALF"):
        gen(["1", str(f), "-1", "-1", dtype, "-o", str(tmp_path / "o.hip")], tmp_path)
    gen(["1", str(f), "3", "-1", "FLOAT", "-o", str(tmp_path / "o.hip"), "--list", "3"], tmp_path)


def test_malformed_mapping_specs_are_refused_cleanly(tmp_path):
    src = os.path.join(PKG, "expressions", "cfg2_f64.in")
    rng = random.Random(7)
    good = "x=d:72,c:2;y=b:8,a:8;k=e:24;w=3x4;t=3x1;st=3;nt=3;il=1;ov=1"
    specs = ["", ";", "x=", "x=d", "x=d:", "x=:4", "x=d:0;y=b:8,a:8;k=e:24;w=3x4;t=3x1", "x=d:-8;y=b:8;k=e:4;w=1x1;t=1x1",
             "x=d:72,c:2;y=b:8,a:8;k=e:24;w=0x4;t=3x1", "x=d:72,c:2;y=b:8,a:8;k=e:24;w=3x4;t=999999x999999",
             "x=d:72,c:2;y=b:8,a:8;k=e:24;w=3x4;t=3x1;st=-5", "x=d:2147483647,c:2147483647;y=b:2147483647;k=e:2147483647;w=16x16;t=64x64",
             "x=zz:4;y=b:8;k=e:4", "w=3x4", "x=d:72,c:2;y=b:8,a:8;k=e:24;w=3x4;t=3x1;mw=99;pd=99;sk=99999;cd=9;vl=9", good * 50]
    for _ in range(60):                      # mutations of a good spec: one character replaced, dropped or doubled
        s = list(good)
        i = rng.randrange(len(s))
        op = rng.choice("rdx")
        if op == "r":
            s[i] = rng.choice("0123456789:;,=xyk-")
        elif op == "d":
            del s[i]
        else:
            s.insert(i, s[i])
        specs.append("".join(s))
    for spec in specs:
        gen(["1", src, "-1", "-1", "DOUBLE", "-o", str(tmp_path / "o.hip"), "--map", spec], tmp_path)


def test_fused_group_files_through_the_sanitized_generator(tmp_path):
    for f in sorted(glob.glob(os.path.join(PKG, "expressions", "fused_*.in"))):
        r = gen(["9", f, "-1", "-1", "DOUBLE" if "f64" in f else "FLOAT", "-o", str(tmp_path / "g.hip"), "--json"], tmp_path)
        assert r.returncode == 0, r.stderr
        gen(["9", f, "-1", "-1", "DOUBLE", "-o", str(tmp_path / "g.hip"), "--map", "ct=1,1,1,1,1,1"], tmp_path)
        gen(["9", f, "-1", "-1", "DOUBLE", "-o", str(tmp_path / "g.hip"), "--map", "ct=99999,0,-3"], tmp_path)
