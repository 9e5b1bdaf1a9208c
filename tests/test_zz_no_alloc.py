"""The batched quantize that brings its own workspace (gact_quantize_batched_static) against the entry points it
stands for (gact_batch_plan + gact_quantize_batched on caller memory), through the C ABI: packed arena, scale
and min arenas and the planned offsets must be identical, bit for bit, on two calls in a row, the second on a
smaller table (the library's array still holds the first call's lists)."""
import numpy as np
import pytest
import torch

from gact.batched import BatchedQuantizer
from gact.cpp_extension import _abi

pytestmark = pytest.mark.gpu


def _run_both(shapes, dtypes, widths, stream, seed0):
    lib = _abi.lib()
    g = torch.Generator().manual_seed(seed0)
    tensors = [torch.randn(s, generator=g).to(d).cuda() for s, d in zip(shapes, dtypes)]
    L = len(tensors)
    bq = BatchedQuantizer([t.numel() for t in tensors], dtypes, "cuda")
    bits = torch.tensor(widths, dtype=torch.int32, device="cuda")
    seeds = [seed0 + i for i in range(L)]
    mode = _abi.NOISE_MODES[stream]
    st = torch.cuda.current_stream().cuda_stream
    results = []
    for static in (False, True):
        table = bq._table(tensors, seeds)
        # arenas start from the same known bytes, so that every byte the kernels leave alone compares equal too
        packed = torch.full((bq.arena_bytes_worst_case(),), 0xA5, dtype=torch.uint8, device="cuda")
        scale = torch.full((bq.total_groups * 4,), 0x5A, dtype=torch.uint8, device="cuda")
        mn = torch.full((bq.total_groups * 4,), 0x3C, dtype=torch.uint8, device="cuda")
        if static:
            verdict = torch.full((2,), -7, dtype=torch.int64, device="cuda")
            _abi.check(lib.gact_quantize_batched_static(table.data_ptr(), bits.data_ptr(), L, bq.total_blocks,
                                                        packed.numel(), mode, bq.dtype_mask, packed.data_ptr(),
                                                        scale.data_ptr(), mn.data_ptr(), verdict.data_ptr(), st))
        else:
            ws = bq.new_workspace()
            _abi.check(lib.gact_batch_plan(table.data_ptr(), bits.data_ptr(), L, bq.total_blocks, packed.numel(),
                                           ws.data_ptr(), st))
            _abi.check(lib.gact_quantize_batched(table.data_ptr(), bits.data_ptr(), L, bq.total_blocks, mode,
                                                 bq.dtype_mask, ws.data_ptr(), packed.data_ptr(), scale.data_ptr(),
                                                 mn.data_ptr(), st))
            assert bq.plan_ok(ws)
        torch.cuda.synchronize()
        if static:      # the verdict the caller gets equals the header the caller-workspace path reads
            assert verdict.tolist() == [need, 1]
        else:
            need = int(ws[:8].view(torch.int64).item())
        results.append((table.cpu().numpy().copy(), packed.cpu().numpy(), scale.cpu().numpy(), mn.cpu().numpy()))
    (t0, p0, s0, m0), (t1, p1, s1, m1) = results
    offsets0 = t0.view(np.int64).reshape(-1, 7)[:, 5]
    offsets1 = t1.view(np.int64).reshape(-1, 7)[:, 5]
    assert np.array_equal(offsets0, offsets1), "planned offsets differ"
    assert (p0 != 0xA5).any(), "the reference launch wrote nothing"
    assert np.array_equal(p0, p1), "packed arena differs"
    assert np.array_equal(s0, s1), "scale arena differs"
    assert np.array_equal(m0, m1), "min arena differs"


def test_static_workspace_matches_caller_workspace_twice_in_a_row():
    rng = np.random.default_rng(11)
    # first call: 40 tensors of mixed types and widths, a few thousand blocks
    shapes = [(int(rng.integers(1, 300)), int(rng.integers(1, 40)), int(rng.choice([96, 192, 384, 77]))) for _ in range(40)]
    dtypes = [(torch.float32, torch.float16, torch.bfloat16)[i % 3] for i in range(40)]
    widths = [int(rng.choice([1, 2, 4, 8])) for _ in range(40)]
    _run_both(shapes, dtypes, widths, "fast", 100)
    # second call, smaller: 7 half tensors; whatever the first call left in the library's array must not matter
    shapes = [(int(rng.integers(1, 50)), 33, 64) for _ in range(7)]
    widths = [2, 2, 1, 8, 4, 1, 2]
    _run_both(shapes, [torch.float16] * 7, widths, "deterministic", 7)


def _static_call(tensors, widths, capacity_of):
    """One call of the static entry point on arenas pre-filled with known bytes -> (verdict, arenas untouched?)."""
    lib = _abi.lib()
    L = len(tensors)
    bq = BatchedQuantizer([t.numel() for t in tensors], [t.dtype for t in tensors], "cuda")
    bits = torch.tensor(widths, dtype=torch.int32, device="cuda")
    table = bq._table(tensors, list(range(L)))
    packed = torch.full((capacity_of(bq),), 0xA5, dtype=torch.uint8, device="cuda")
    scale = torch.full((bq.total_groups * 4,), 0x5A, dtype=torch.uint8, device="cuda")
    mn = torch.full((bq.total_groups * 4,), 0x3C, dtype=torch.uint8, device="cuda")
    verdict = torch.full((2,), -7, dtype=torch.int64, device="cuda")
    _abi.check(lib.gact_quantize_batched_static(table.data_ptr(), bits.data_ptr(), L, bq.total_blocks, packed.numel(),
                                                _abi.NOISE_CONST, bq.dtype_mask, packed.data_ptr(), scale.data_ptr(),
                                                mn.data_ptr(), verdict.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    untouched = bool((packed == 0xA5).all() and (scale == 0x5A).all() and (mn == 0x3C).all())
    return verdict.tolist(), untouched


def test_static_workspace_void_plans_are_reported_and_do_not_leak_into_the_next_call():
    """A width the kernels cannot pack (calc_precision can leave 32) or an arena that is too short voids the launch:
    the caller's verdict words say so, the arenas stay as they were, and the verdict the library's array keeps from
    a void call does not survive into the next, valid, call - nor a valid one into the next void call."""
    g = torch.Generator().manual_seed(3)
    tensors = [torch.randn(s, generator=g).half().cuda() for s in ((40, 33, 64), (7, 300), (129, 256))]
    worst = lambda bq: bq.arena_bytes_worst_case()
    verdict, untouched = _static_call(tensors, [4, 32, 2], worst)           # void: a width of 32
    assert verdict[1] == 0 and untouched
    _run_both([(40, 33, 64), (7, 300), (129, 256)], [torch.float16] * 3, [4, 8, 2], "deterministic", 3)   # valid, checked bit for bit
    verdict, untouched = _static_call(tensors, [8, 8, 8], lambda bq: 4096)  # void: the arena is too short
    assert verdict[1] == 0 and verdict[0] > 4096 and untouched
    verdict, untouched = _static_call(tensors, [4, 8, 2], worst)            # valid again
    assert verdict[1] == 1 and 0 < verdict[0] <= sum(t.numel() for t in tensors) + 768 * 3 + 256 and not untouched
    verdict, untouched = _static_call(tensors, [0, 1, 1], worst)            # void: a width of 0
    assert verdict[1] == 0 and untouched


def test_static_workspace_limits():
    lib = _abi.lib()
    # beyond the array: refused before anything is launched (the pointers are never touched)
    assert lib.gact_quantize_batched_static(16, 16, 10, 262145, 1 << 20, 3, 0, 16, 16, 16, None, None) == -6
    assert lib.gact_quantize_batched_static(16, 16, 10, (1 << 29) - 1, 1 << 20, 3, 0, 16, 16, 16, None, None) == -6
    assert lib.gact_quantize_batched_static(16, 16, 10, 100, 1 << 20, 3, 0, 16, 16, 16, 4, None) == -2      # verdict not 8-byte aligned
    assert b"limit" in lib.gact_strerror(-6)
