"""Greedy bit allocation: the oracle and the library's host entry point against (a) vectors written by
the reference's own calc_precision.cc (tests/golden/calc_precision_vectors.json), (b) that same compiled
reference live, where oracle/_ref is built, (c) properties the algorithm fixes."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from gact.cpp_extension import calc_precision as ext

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "calc_precision_vectors.json")


def load_cases():
    with open(GOLDEN) as f:
        return json.load(f)["cases"]


def run_oracle(C, w, init, target):
    return oracle.calc_precision(np.full(C.size, init, np.int32), C, w, target)


def run_lib(C, w, init, target):
    b = torch.full((C.size,), init, dtype=torch.int32)
    out = ext.calc_precision(b, torch.from_numpy(C.copy()), torch.from_numpy(w.copy()), target)
    assert out.data_ptr() == b.data_ptr()          # mutated in place and returned, like the reference
    return out.numpy()


@pytest.mark.parametrize("case", load_cases(), ids=lambda c: c["name"])
def test_golden_vectors(case):
    C = np.array(case["C_bits"], np.uint32).view(np.float32)
    w = np.array(case["w"], np.int64)
    want = np.array(case["bits"], np.int32)
    np.testing.assert_array_equal(run_oracle(C, w, case["init"], case["target"]), want)
    np.testing.assert_array_equal(run_lib(C, w, case["init"], case["target"]), want)


def test_against_the_compiled_reference_live():
    ref = oracle.load_ref_calc_precision()
    if ref is None:
        pytest.skip("oracle/_ref is not built here (needs the reference checkout)")
    rng = np.random.default_rng(0)
    for t in range(300):
        L = int(rng.integers(1, 60))
        C = np.exp(rng.normal(0, 2, L)).astype(np.float32)
        if t % 4 == 0:                               # ties and near ties
            C[:] = C[0]
            C = (C.view(np.int32) + rng.integers(-1, 2, L).astype(np.int32)).view(np.float32)
        w = (rng.integers(1, 500, L) * 256).astype(np.int64)
        if t % 5 == 0:
            w[:] = w[0]
        init = int(rng.choice([8, 32]))
        target = float(rng.choice([1.0, 1.5, 2.0, 3.0, 4.0, 8.0])) * float(w.sum())
        want = ref.calc_precision(torch.full((L,), init, dtype=torch.int32), torch.from_numpy(C.copy()),
                                  torch.from_numpy(w.copy()), target).numpy()
        np.testing.assert_array_equal(run_oracle(C, w, init, target), want)
        np.testing.assert_array_equal(run_lib(C, w, init, target), want)


def test_hand_cases():
    C = np.ones(3, np.float32)
    w = np.full(3, 256, np.int64)
    # budget 2 bits/element from 8: every tensor goes 8 -> 4 -> 2
    np.testing.assert_array_equal(run_lib(C, w, 8, 2.0 * 768), [2, 2, 2])
    # 3 bits/element (2304 bits): 6144 -> three 8->4 steps -> 3072, then 4->2 on index 2 (2560, still over)
    # and on index 1 (2048): ties pop the highest index first
    np.testing.assert_array_equal(run_lib(C, w, 8, 3.0 * 768), [4, 2, 2])
    # a more sensitive tensor keeps more bits
    C2 = np.array([100.0, 1.0, 1.0], np.float32)
    out = run_lib(C2, w, 8, 3.0 * 768)
    assert out[0] >= out[1] and out[0] >= out[2]


def test_properties():
    rng = np.random.default_rng(4)
    for _ in range(50):
        L = int(rng.integers(2, 80))
        C = np.exp(rng.normal(0, 2, L)).astype(np.float32)
        w = (rng.integers(1, 300, L) * 256).astype(np.int64)
        prev = None
        for avg in (8.0, 6.0, 4.0, 3.0, 2.0, 1.5, 1.0):
            out = run_lib(C, w, 8, avg * float(w.sum()))
            assert set(out.tolist()) <= {1, 2, 4, 8}
            assert float((out.astype(np.int64) * w).sum()) <= avg * float(w.sum())
            if prev is not None:
                assert (out <= prev).all()           # monotone in the budget
            prev = out
    # from the default max_bit = 32 the result may keep 32 only if the budget allows it
    out = run_lib(np.ones(4, np.float32), np.full(4, 256, np.int64), 32, 32.0 * 1024)
    assert out.tolist() == [32] * 4


def test_unreachable_budget_is_an_error_not_undefined_behaviour():
    # the reference pops an empty queue here; the library reports it
    b = torch.full((4,), 8, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="budget"):
        ext.calc_precision(b, torch.ones(4), torch.full((4,), 256, dtype=torch.int64), 10.0)
    with pytest.raises(RuntimeError):
        oracle.calc_precision(np.full(4, 8, np.int32), np.ones(4, np.float32), np.full(4, 256, np.int64), 10.0)


def test_argument_checks():
    b = torch.full((4,), 8, dtype=torch.int32)
    C = torch.ones(4)
    w = torch.full((4,), 256, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.calc_precision(torch.full((8,), 8, dtype=torch.int32)[::2], C, w, 1e9)
    with pytest.raises(RuntimeError):
        ext.calc_precision(b.to(torch.int64), C, w, 1e9)
    with pytest.raises(RuntimeError):
        ext.calc_precision(torch.full((4,), 3, dtype=torch.int32), C, w, 1.0)   # 3 is not a width the descent knows
