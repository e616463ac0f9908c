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
import re
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
    # the same generator with AddressSanitizer and UndefinedBehaviorSanitizer (host code only; the runtimes linked
    # statically so that nothing has to be preloaded): parser, spec reader and emitter take untrusted text, and the
    # CPU tests push the corpus and malformed input through this binary
    run(["g++", "-O1", "-g", "-std=c++17", "-fopenmp", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
         "-fno-omit-frame-pointer", "-static-libasan", "-static-libubsan", "-o", os.path.join(BIN, "cogent_gen_san"),
         os.path.join(CSRC, "tc_cli.cpp")] + srcs)


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


RESOURCE_FLAG = "-Rpass-analysis=kernel-resource-usage"


def kernel_resources(remarks):
    """hipcc's per-kernel resource remarks (the counterpart of the reference's `nvcc -Xptxas -v`,
    cogent/Makefile:16) as {kernel: {"vgprs", "agprs", "scratch_bytes", "occupancy", "lds_bytes"}}; kernel names
    are shortened to the template and its boolean arguments."""
    import re
    out, cur = {}, None
    keys = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes",
            "Occupancy [waves/SIMD]": "occupancy", "LDS Size [bytes/block]": "lds_bytes", "VGPRs Spill": "vgpr_spills"}
    for line in remarks.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            sym = m.group(1)
            base = re.search(r"(tc_\w+?_kernel|cogent_\w+_kernel)", sym)
            flags = re.findall(r"Lb([01])", sym)
            cur = (base.group(1) if base else sym) + ("<" + ",".join(flags) + ">" if flags else "")
            if "IdE" in sym and not flags: cur += "<f64>"
            if "IfE" in sym and not flags: cur += "<f32>"
            out[cur] = {}
            continue
        m = re.search(r"remark:\s+([A-Za-z \[\]/]+): (\d+)", line)
        if m and cur is not None and m.group(1).strip() in keys:
            out[cur][keys[m.group(1).strip()]] = int(m.group(2))
    return out


def hot_kernel(info, sizes):
    """The kernel instantiation the launcher picks for these extents (tc_launch.hpp: streaming kernel when the object
    has one and the extents give full tiles and its K-block count; else the per-tile kernel's variant by divisibility)."""
    m = info["mapping"]
    ext = dict(zip(info["out_idx"] + info["sum_idx"], sizes))
    div = lambda side: all(ext[n] % t == 0 for n, t in m[side])
    nkb = 1
    for n, t in m["k"]:
        nkb *= -(-ext[n] // t)
    swp = int(bool(m["swapped_roles"]) and ext[info["out_idx"][0]] % 4 == 0)
    if m["stream"][0] > 0 and div("x") and div("y") and div("k") and nkb == m["stream"][0]:
        return "tc_stream_kernel<%d>" % swp
    bx, by, bk = m["block_tile"]
    px, py, pk = m["padded"]
    ext_full = int(div("x") and div("y") and bx == px and by == py)
    int_full = int(div("k") and bk == pk)
    return "tc_mfma_kernel<%d,%d,%d,%d>" % (ext_full, int_full, int(nkb == 1), swp)


def emit_and_compile(entry):
    """Emits and compiles one expression.  The compiler's resource report of every kernel in the object goes to
    lib/<name>.resources.json ("hot" names the instantiation that runs at the entry's benchmark extents).  If THAT
    kernel spills registers to scratch memory the build fails (such kernels ran 15 to 20 times slower when they were
    measured) unless the entry says "allow_scratch"; spills in the variants for other extents are recorded, and where
    they are the one-K-block kernels for ragged tiles the object is emitted again so that it no longer uses them."""
    name = entry["name"]
    hip = os.path.join(GEN, name + ".hip")
    cmd = [os.path.join(BIN, "cogent_gen"), name, os.path.join(EXPR, entry["file"]),
           str(entry.get("config", -1)), "-1", entry["dtype"], "-o", hip, "--name", name, "--json"]
    spec = entry.get("map") or tuned_map(entry)
    if spec:
        cmd += ["--map", spec]
    plan = json.loads(run(cmd))
    remarks = run(["hipcc"] + HIPCC_FLAGS + [RESOURCE_FLAG, "-o", os.path.join(LIB, name + ".so"), hip])
    res = kernel_resources(remarks)
    is_spilling = lambda r: sorted(k for k, v in r.items() if v.get("scratch_bytes", 0) > 0 and k.startswith(("tc_mfma", "tc_stream", "tc_group")))
    spilling = is_spilling(res)
    # A one-K-block kernel for calls with ragged tiles (tc_mfma_kernel<E,I,1,*> other than E = I = 1) that spills: emit
    # the object again with ok=0, which sends those calls through the K-loop kernels (a loop of one trip) instead.  Only
    # for mappings without split K (the generator refuses the combination).  The spilling kernels stay in the object,
    # unused; "rerouted" names them.
    m = plan.get("mapping", {})
    ragged = lambda names: [k for k in names if re.match(r"tc_mfma_kernel<[01],[01],1,[01]>$", k) and not k.startswith("tc_mfma_kernel<1,1,")]
    if ragged(spilling) and m.get("split_k", 1) == 1 and m.get("one_block_ragged", 1) == 1:
        cmd2 = [c for c in cmd]
        if "--map" in cmd2:
            cmd2[cmd2.index("--map") + 1] += ";ok=0"
        else:
            cmd2 += ["--map", m["spec"] + ";ok=0"]
        plan = json.loads(run(cmd2))
        m = plan.get("mapping", {})
        remarks = run(["hipcc"] + HIPCC_FLAGS + [RESOURCE_FLAG, "-o", os.path.join(LIB, name + ".so"), hip])
        res = kernel_resources(remarks)
        spilling = is_spilling(res)
    rerouted = ragged(spilling) if m.get("one_block_ragged", 1) == 0 else []
    hot = hot_kernel(plan, entry["bench_sizes"]) if "mapping" in plan else None      # (a fused group has one kernel of its own)
    with open(os.path.join(LIB, name + ".resources.json"), "w") as f:
        json.dump({"hot": hot, "spilling": spilling, "rerouted": rerouted, "kernels": res}, f, indent=1, sort_keys=True)
    bad = [k for k in spilling if hot is None or k == hot]
    if bad and not entry.get("allow_scratch"):
        raise RuntimeError("%s: the kernel for its benchmark extents spills registers to scratch memory: %s (mapping %s)"
                           % (name, ", ".join(bad), spec or "by the model"))
    return name


def model_name(name):
    return "model_" + name


def emit_and_compile_model_pick(entry):
    """The same expression compiled from the mapping pass's FIRST pick: no mapping spec, no tuned table.  These
    objects (lib/model_<name>.so, benchmark configurations only) exist to measure the mapping pass on its own against
    the tuned objects."""
    name = model_name(entry["name"])
    hip = os.path.join(GEN, name + ".hip")
    run([os.path.join(BIN, "cogent_gen"), name, os.path.join(EXPR, entry["file"]), "-1", "-1", entry["dtype"],
         "-o", hip, "--name", name, "--json"])
    run(["hipcc"] + HIPCC_FLAGS + ["-o", os.path.join(LIB, name + ".so"), hip])
    return name


def benchmark_configs():
    return [e for e in manifest() if e["name"].startswith("cfg")]


def build_driver():
    run(["hipcc"] + HIPCC_FLAGS + ["-o", os.path.join(LIB, "libcogent_driver.so"),
                                   os.path.join(CSRC, "tc_driver.cpp"), "-ldl"])


def build_all(jobs=8, only=None):
    build_host_tools()
    os.makedirs(GEN, exist_ok=True)
    entries = [e for e in manifest() + group_manifest() if only is None or e["name"] in only]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        futs = [ex.submit(emit_and_compile, e) for e in entries]
        futs += [ex.submit(emit_and_compile_model_pick, e) for e in benchmark_configs() if only is None or model_name(e["name"]) in only]
        futs.append(ex.submit(build_driver))
        for f in futs:
            f.result()
    if only is None:
        sys.path.insert(0, HERE)
        from cogent_mi355 import tuner
        for name, k in TUNING_SETS.items():
            # (a candidate whose kernel spills registers is dropped by the tuner on purpose: not a build failure)
            bad = [c for c in tuner.prepare(name, k, jobs=jobs) if "so" not in c and "spills" not in c.get("error", "")]
            if bad:
                raise RuntimeError("tuning candidate failed to build: %r" % bad[0])
    return [e["name"] for e in entries]


if __name__ == "__main__":
    names = build_all(only=set(sys.argv[1:]) or None)
    print("built", len(names), "expression objects:", " ".join(names))
