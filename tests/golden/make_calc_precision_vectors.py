"""Write tests/golden/calc_precision_vectors.json from the reference's own calc_precision.cc.

The reference file is compiled unmodified into oracle/_ref by `make -C oracle ref` (it is host-only
C++ against torch headers, which this image ships).  This script feeds it seeded inputs - random,
tied and near-tied after the float narrowing of the heap keys - and records inputs and outputs.
Only data is committed; run it again where the reference checkout is present to regenerate.

    python tests/golden/make_calc_precision_vectors.py
"""
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402


def main():
    oracle.build_ref()
    ref = oracle.load_ref_calc_precision()
    if ref is None:
        sys.exit("oracle/_ref is not built (needs the reference checkout)")
    rng = np.random.default_rng(20240607)
    cases = []

    def add(name, C, w, init, target):
        C = np.asarray(C, np.float32)
        w = np.asarray(w, np.int64)
        b = torch.full((C.size,), int(init), dtype=torch.int32)
        out = ref.calc_precision(b, torch.from_numpy(C.copy()), torch.from_numpy(w.copy()), float(target))
        cases.append({"name": name, "C_bits": [int(v) for v in C.view(np.uint32)], "w": [int(v) for v in w],
                      "init": int(init), "target": float(target), "bits": [int(v) for v in out.tolist()]})

    # hand cases: equal sensitivities and sizes step down highest index first
    add("equal-3", [1, 1, 1], [256] * 3, 8, 2.0 * 768)
    add("equal-3-budget-3", [1, 1, 1], [256] * 3, 8, 3.0 * 768)
    add("equal-5-from-32", [2, 2, 2, 2, 2], [1024] * 5, 32, 4.0 * 5120)
    add("already-within-budget", [1, 5, 9], [256, 512, 1024], 8, 8.0 * 1792)
    add("single", [3.5], [4096], 32, 2.0 * 4096)
    # random, Swin-like sizes
    shapes = [128 * 3136 * 96, 128 * 784 * 192, 128 * 196 * 384, 128 * 49 * 768]
    for t in range(24):
        L = int(rng.integers(2, 140))
        C = np.exp(rng.normal(0, 2, L)).astype(np.float32)
        w = np.array([shapes[i] for i in rng.integers(0, 4, L)], np.int64)
        init = int(rng.choice([8, 32]))
        avg = float(rng.choice([1.0, 1.5, 2.0, 2.5, 3.0, 4.0, 6.0]))
        add("random-%d" % t, C, w, init, avg * float(w.sum()))
    # near ties: sensitivities one float ulp apart, equal sizes -> keys that collide or order by a hair after
    # the double -> float narrowing
    for t in range(12):
        L = int(rng.integers(4, 40))
        base = np.float32(np.exp(rng.normal(0, 1)))
        C = np.full(L, base, np.float32)
        ulps = rng.integers(-2, 3, L)
        C = (C.view(np.int32) + ulps.astype(np.int32)).view(np.float32)
        w = np.full(L, int(rng.choice([256, 4096, 65536])), np.int64)
        if t % 3 == 0:
            w[rng.integers(0, L)] *= 2
        add("near-tie-%d" % t, C, w, int(rng.choice([8, 32])), float(rng.choice([1.5, 2.0, 3.0])) * float(w.sum()))
    # sensitivity capped at 1e10 (gact/gact/autoprec.py:124-125) and tiny ones
    add("capped", [1e10, 1e-12, 1.0, 1e10, 3e-7], [4096, 256, 1024, 256, 65536], 32, 2.0 * (4096 + 256 + 1024 + 256 + 65536))

    path = os.path.join(ROOT, "tests", "golden", "calc_precision_vectors.json")
    with open(path, "w") as f:
        json.dump({"source": "gact/gact/cpp_extension/calc_precision.cc:66-118 compiled unmodified (oracle/_ref)",
                   "cases": cases}, f)
    print("wrote %d cases to %s" % (len(cases), path))


if __name__ == "__main__":
    main()
