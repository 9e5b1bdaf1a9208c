"""Helpers next to the path: tensor-key sampling (tests/test_sample.py of the reference), byte counting,
the JSON-lines recorder."""
import json

import torch

from gact.utils import (GlobalExpRecorder, compute_tensor_bytes, empty_cache, random_sample, sampled_key_with_sum,
                        uniform_sample, uniform_sample_ref)


def sample_by_loop(t, cnt, add_dataptr=True):
    step = max(t.numel() // cnt, 1)
    key = [t.data_ptr()] if add_dataptr else []
    for i in range(min(cnt, t.numel())):
        key.append(t.view(-1)[i * step].item())
    return key


def test_uniform_sample_matches_a_plain_loop():
    torch.manual_seed(0)
    for shape, cnt in (((1000,), 100), ((37, 11), 100), ((5,), 100), ((4, 4, 4), 7), ((256, 256), 1)):
        t = torch.randn(shape)
        assert uniform_sample(t, cnt) == sample_by_loop(t, cnt)
        assert uniform_sample(t, cnt, add_dataptr=False) == sample_by_loop(t, cnt, add_dataptr=False)
        assert uniform_sample(t, cnt) == uniform_sample_ref(t, cnt)
    assert uniform_sample(torch.empty(0), 10, add_dataptr=False) == []


def test_key_with_sum_equals_the_two_step_key():
    # the duplicate-detection key of gact/gact/quantizer.py:85-93: address, strided sample, sum
    for dtype in (torch.float32, torch.float16):
        for n in (1, 7, 100, 1000, 4097):
            t = torch.randn(n).to(dtype)
            assert sampled_key_with_sum(t, 100) == uniform_sample(t, min(100, n)) + [t.sum().item()]


def test_random_sample_is_reproducible_and_leaves_the_global_stream_alone():
    t = torch.arange(1000.0).reshape(10, 100)
    torch.manual_seed(5)
    before = torch.rand(3)
    torch.manual_seed(5)
    key = random_sample(t, 20)
    after = torch.rand(3)
    assert torch.equal(before, after)
    assert key[0] == t.data_ptr() and len(key) == 21
    assert key == random_sample(t, 20) and all(0 <= v < 1000 for v in key[1:])
    g = torch.Generator().manual_seed(t.dim())          # the positions come from a generator seeded by the rank
    assert key[1:] == t.reshape(-1)[torch.randint(0, 1000, (20,), generator=g)].tolist()
    empty_cache(None)                                    # no ratio: nothing to do, no GPU needed


def test_compute_tensor_bytes():
    ts = [torch.zeros(3, 4), torch.zeros(5, dtype=torch.float16), torch.zeros(7, dtype=torch.int8),
          torch.zeros(2, dtype=torch.long), 4]
    assert compute_tensor_bytes(ts) == 48 + 10 + 7 + 16 + 4
    assert compute_tensor_bytes(torch.zeros(10, dtype=torch.uint8)) == 10


def test_recorder_appends_json_lines(tmp_path):
    rec = GlobalExpRecorder()
    rec.record("iter", 3)
    rec.record("value", 0.123456789)
    path = tmp_path / "log.jsonl"
    rec.dump(str(path))
    rec.record("iter", 4)
    rec.dump(str(path))
    lines = [json.loads(l) for l in path.read_text().splitlines()]
    assert [l["iter"] for l in lines] == [3, 4] and lines[0]["value"] == 0.123457
