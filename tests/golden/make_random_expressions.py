"""Writes rand_NN.in: seeded random contractions in the reference's grammar, beyond the shapes of its corpus
(odd extents, contracted extents that are not multiples of the matrix instruction's depth, one to three
summed indices, inputs with a single external index, outputs of rank 1 to 6, both operators).  The files and
their manifest entries are committed; this script only documents how they were made and can remake them."""
import json
import os
import random

# the files are written into the package's expression corpus
HERE = os.path.join(os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))), "cgo2019-ae_amd", "expressions")
LETTERS = "abcdefghijkl"


def one(rng, k):
    n_out = rng.choice([1, 2, 2, 3, 3, 4, 4, 5, 6])
    n_sum = rng.choice([1, 1, 1, 2, 2, 3])
    out = list(LETTERS[:n_out])
    summed = list(LETTERS[n_out:n_out + n_sum])
    ext = {}
    budget = 2.0e6                                   # elements of C at the representative sizes
    for i in out:
        ext[i] = rng.choice([2, 3, 5, 7, 8, 9, 12, 16, 17, 24, 30, 32, 40])
    while True:
        vol = 1
        for i in out:
            vol *= ext[i]
        if vol <= budget:
            break
        big = max(out, key=lambda i: ext[i])
        ext[big] = max(2, ext[big] // 2)
    for i in summed:
        ext[i] = rng.choice([1, 2, 3, 5, 6, 8, 10, 13, 16, 24])
    # split the output indices between the inputs: each input gets at least one unless the output has rank 1
    rng_out = out[:]
    rng.shuffle(rng_out)
    cut = rng.randint(1, max(1, n_out - 1)) if n_out > 1 else 1
    a_ext, b_ext = rng_out[:cut], rng_out[cut:]
    a = a_ext + summed
    b = b_ext + summed
    rng.shuffle(a)
    rng.shuffle(b)
    rng.shuffle(out)                                  # output order independent of the inputs'
    op = rng.choice(["+=", "+=", "-="])
    sizes = lambda names: ",".join("%s,%d" % (i, ext[i]) for i in names)
    text = "t3 [%s] %s sum(%s) * t2 [%s] * v2 [%s];" % (sizes(out), op, sizes(summed), ",".join(a), ",".join(b))
    dtype = rng.choice(["DOUBLE", "DOUBLE", "FLOAT"])
    return text, dtype, [ext[i] for i in out + summed]


def main(n=12, seed=20190216):
    rng = random.Random(seed)
    entries = []
    for k in range(n):
        text, dtype, sizes = one(rng, k)
        name = "rand_%02d_%s" % (k, "f64" if dtype == "DOUBLE" else "f32")
        fn = "rand_%02d.in" % k
        with open(os.path.join(HERE, fn), "w") as f:
            f.write("# seeded random contraction %d (tests/golden/make_random_expressions.py, seed %d)\n%s\n" % (k, seed, text))
        entries.append({"name": name, "file": fn, "dtype": dtype, "bench_sizes": sizes, "config_id": "random %d" % k})
    path = os.path.join(HERE, "manifest.json")
    m = json.load(open(path))
    m["expressions"] = [e for e in m["expressions"] if not e["name"].startswith("rand_")] + entries
    json.dump(m, open(path, "w"), indent=1)
    for e in entries:
        print(e["name"], open(os.path.join(HERE, e["file"])).read().splitlines()[1])


if __name__ == "__main__":
    main()
