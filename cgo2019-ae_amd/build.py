"""Build everything the engine ships as native code, in-tree.

  lib/libcogent_mi355.so   host tools: parser, gfx950 mapping pass, emitter, seeded fill  (g++)
  bin/cogent_gen           command-line generator with the reference's five arguments     (g++)
  generated/<name>.hip     one emitted translation unit per expression in expressions/manifest.json
  lib/<name>.so            the same, compiled for gfx950                                   (hipcc)
  lib/libcogent_driver.so  timing driver (HIP events around batches of launches)           (hipcc)
  tuning/<name>/cand_NN.so candidate mappings of the entries listed in TUNING_SETS, for the on-GPU tuner

A mapping comes from, in this order: the entry's "map" in manifest.json (pinned by hand), the tuner's
cache expressions/tuned.json (measured), the mapping pass's cost model.

hipcc cross-compiles for gfx950 without a GPU, so this runs on a CPU-only machine.
"""
import concurrent.futures
import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
BIN = os.path.join(HERE, "bin")
GEN = os.path.join(HERE, "generated")
EXPR = os.path.join(HERE, "expressions")

HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC",
               # keep hipcc from forming packed-fp32 instructions
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument",
               "-I" + os.path.join(CSRC, "kernels")]


def run(cmd, **kw):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), r.stdout))
    return r.stdout


def manifest():
    with open(os.path.join(EXPR, "manifest.json")) as f:
        return json.load(f)["expressions"]


def group_manifest():
    """Files that hold several expressions with one output: each becomes one fused-group object."""
    with open(os.path.join(EXPR, "manifest.json")) as f:
        return json.load(f).get("groups", [])


def build_host_tools():
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(BIN, exist_ok=True)
    srcs = [os.path.join(CSRC, f) for f in ("tc_parse.cpp", "tc_mapping.cpp", "tc_emit.cpp", "tc_group.cpp", "tc_capi.cpp")]
    run(["g++", "-O2", "-std=c++17", "-fopenmp", "-shared", "-fPIC", "-Wall",
         "-o", os.path.join(LIB, "libcogent_mi355.so")] + srcs)
    run(["g++", "-O2", "-std=c++17", "-Wall", "-o", os.path.join(BIN, "cogent_gen"),
         os.path.join(CSRC, "tc_cli.cpp"), "-L" + LIB, "-lcogent_mi355", "-Wl,-rpath,$ORIGIN/../lib"])


# manifest entries whose top candidates are compiled ahead of time so that the tuner's measuring step
# (cogent_mi355/tuner.py) has something to time on a GPU machine without compiling there
TUNING_SETS = {"cfg5_1_f64": 3}


def tuned_map(entry):
    path = os.path.join(EXPR, "tuned.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        hit = json.load(f).get("%s|%s|%s" % (entry["file"], entry["dtype"], ",".join(str(s) for s in entry["bench_sizes"])))
    return hit["map"] if hit else None


def emit_and_compile(entry):
    name = entry["name"]
    hip = os.path.join(GEN, name + ".hip")
    cmd = [os.path.join(BIN, "cogent_gen"), name, os.path.join(EXPR, entry["file"]),
           str(entry.get("config", -1)), "-1", entry["dtype"], "-o", hip, "--name", name]
    spec = entry.get("map") or tuned_map(entry)
    if spec:
        cmd += ["--map", spec]
    run(cmd)
    run(["hipcc"] + HIPCC_FLAGS + ["-o", os.path.join(LIB, name + ".so"), hip])
    return name


def build_driver():
    run(["hipcc"] + HIPCC_FLAGS + ["-o", os.path.join(LIB, "libcogent_driver.so"),
                                   os.path.join(CSRC, "tc_driver.cpp"), "-ldl"])


def build_all(jobs=8, only=None):
    build_host_tools()
    os.makedirs(GEN, exist_ok=True)
    entries = [e for e in manifest() + group_manifest() if only is None or e["name"] in only]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        futs = [ex.submit(emit_and_compile, e) for e in entries]
        futs.append(ex.submit(build_driver))
        for f in futs:
            f.result()
    if only is None:
        sys.path.insert(0, HERE)
        from cogent_mi355 import tuner
        for name, k in TUNING_SETS.items():
            bad = [c for c in tuner.prepare(name, k, jobs=jobs) if "so" not in c]
            if bad:
                raise RuntimeError("tuning candidate failed to build: %r" % bad[0])
    return [e["name"] for e in entries]


if __name__ == "__main__":
    names = build_all(only=set(sys.argv[1:]) or None)
    print("built", len(names), "expression objects:", " ".join(names))
