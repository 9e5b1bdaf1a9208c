"""The callers of the operators (Quantizer, Controller, AutoPrecision.refresh_bits) as state machines,
on the CPU, with the operators replaced by recording stand-ins: what the hooks hand to autograd, the
tid / bits / dims / seeds tables, reference counting, and the inputs handed to calc_precision."""
import numpy as np
import pytest
import torch

import gact.autoprec as autoprec_mod
import gact.quantizer as quantizer_mod
from gact.conf import config
from gact.controller import Controller


class Recorder:
    def __init__(self):
        self.calls = []

    def op_quantize(self, x, bit, seed):
        self.calls.append(("q", tuple(x.shape), bit, seed))
        return [x.detach().clone(), bit, None, None]

    def op_dequantize(self, q, shape):
        self.calls.append(("dq", tuple(shape), q[1]))
        return q[0].reshape(shape)


@pytest.fixture
def rec(monkeypatch):
    r = Recorder()
    monkeypatch.setattr(quantizer_mod, "op_quantize", r.op_quantize)
    monkeypatch.setattr(quantizer_mod, "op_dequantize", r.op_dequantize)
    saved = dict(vars(config))
    yield r
    vars(config).update(saved)


def act(shape, requires_grad=True):
    return torch.randn(shape, requires_grad=requires_grad)


def test_filter_rules(rec):
    q = quantizer_mod.Quantizer(default_bit=4, swap=False, prefetch=False)
    p = torch.nn.Parameter(torch.randn(4, 4))
    q.filter_tensors([("w", p)])
    assert q.check_quantize(p) == (False, False)                       # parameters
    assert q.check_quantize(act((4, 4))) == (True, False)
    assert q.check_quantize(act((4, 4), requires_grad=False)) == (False, False)   # e.g. running statistics
    assert q.check_quantize(torch.randn(8).requires_grad_()) == (False, False)    # 1-D
    assert q.check_quantize(torch.randn(2, 2, 2, 2, 2).requires_grad_()) == (False, False)
    assert q.check_quantize(torch.randn(4, 4).double().requires_grad_()) == (False, False)
    assert q.check_quantize(torch.tensor([0, 1, 1, 0], dtype=torch.uint8)) == (True, True)   # dropout mask
    assert q.check_quantize(torch.tensor([0, 2, 1, 0], dtype=torch.uint8)) == (False, False)
    assert q.check_quantize(torch.zeros(4, dtype=torch.uint8)) == (False, False)
    assert q.check_quantize(torch.ones(8192, dtype=torch.bool)) == (False, False)   # bool masks: only on the GPU
    # bfloat16 (not in the reference) exists in the group-256 kernels only; with another group size it is left alone
    bf = torch.randn(4, 4).bfloat16().requires_grad_()
    assert q.check_quantize(bf) == (True, False)
    config.group_size = 128
    assert q.check_quantize(bf) == (False, False)
    assert q.check_quantize(act((4, 4))) == (True, False)
    config.group_size = 256


def test_tuple_protocol_tids_seeds_and_tables(rec):
    q = quantizer_mod.Quantizer(default_bit=4, swap=False, prefetch=False)
    passthrough = torch.randn(3)
    assert q.quantize(passthrough)[0] is False and q.quantize(passthrough)[1] is passthrough
    a, b = act((4, 8)), act((2, 3, 5))
    ha, hb = q.quantize(a), q.quantize(b)
    assert ha == (True, False, 0, a.shape, 0) and hb == (True, False, 1, b.shape, 1)
    assert q.bits == {0: 4, 1: 4} and q.dims == {0: 32, 1: 30} and q.seeds == {0: 0, 1: 1}
    assert rec.calls == [("q", (4, 8), 4, 0), ("q", (2, 3, 5), 4, 1)]
    # backward visits in reverse; every entry is released when its last reference is consumed
    assert torch.equal(q.dequantize(hb), b) and torch.equal(q.dequantize(ha), a)
    assert q.ptr_qtensor_map == {}
    assert torch.equal(q.dequantize((False, passthrough)), passthrough)

    # next iteration: tid restarts, widths come from the table, seeds add the iteration
    q.iterate()
    q.seed_iter = 1
    q.bits = {0: 2, 1: 8}
    rec.calls.clear()
    q.quantize(a), q.quantize(b)
    assert rec.calls == [("q", (4, 8), 2, 1), ("q", (2, 3, 5), 8, 2)]
    assert q.tid == 2 and q.iter == 1


def test_duplicate_saves_share_one_compressed_copy(rec):
    config.check_dup = True
    q = quantizer_mod.Quantizer(default_bit=4, swap=False, prefetch=False)
    a = act((16, 16))
    h1, h2 = q.quantize(a), q.quantize(a)
    assert len(rec.calls) == 1 and h1[2] == h2[2]
    assert list(q.ptr_qtensor_map.values())[0][1] == 2
    q.dequantize(h2)
    assert len(q.ptr_qtensor_map) == 1
    q.dequantize(h1)
    assert q.ptr_qtensor_map == {}
    with pytest.raises(KeyError):
        q.dequantize(h1)                    # a third unpack has nothing left to read


def test_controller_hooks_and_iteration_order(rec, monkeypatch):
    config.auto_prec = False
    config.bit = 3                          # level L2.1's average -> default width 4
    model = torch.nn.Sequential(torch.nn.Linear(8, 8), torch.nn.ReLU(), torch.nn.Linear(8, 2))
    ctl = Controller(model)
    assert ctl.quantizer.default_bit == 4
    ctl.install_hook()
    try:
        x = torch.randn(4, 8, requires_grad=True)
        loss = model(x).sum()
        n_saved = len([c for c in rec.calls if c[0] == "q"])
        assert n_saved >= 2                 # activations were packed, parameters were not
        assert all(c[2] == 4 for c in rec.calls)
        loss.backward()
        assert len([c for c in rec.calls if c[0] == "dq"]) == n_saved
    finally:
        ctl.uninstall_hook()
    assert model[0].weight.grad is not None
    ctl.iterate(lambda: None)
    assert ctl.iter == 1 and ctl.quantizer.seed_iter == 1 and ctl.quantizer.tid == 0 and ctl.quantizer.iter == 1
    # without hooks nothing is recorded
    rec.calls.clear()
    model(x).sum().backward()
    assert rec.calls == []


def test_refresh_bits_feeds_calc_precision_like_the_reference(rec, monkeypatch):
    q = quantizer_mod.Quantizer(default_bit=4, swap=False, prefetch=False)
    for shape in ((128, 96), (64, 192), (32, 384)):
        q.quantize(act(shape))
    ap = autoprec_mod.AutoPrecision(None, q, bits=2, max_bits=32, work_dir="./log/", adapt_interval=1000,
                                    log_interval=-1)
    ap.init_from_dims()
    assert ap.total_bits == 2 * (128 * 96 + 64 * 192 + 32 * 384)
    ap.C = {0: 10.0, 1: 1.0, 2: 0.1}
    seen = {}

    def fake_calc(b, C, w, target):
        seen.update(b=b.clone(), C=C.clone(), w=w.clone(), target=target)
        b[:] = torch.tensor([8, 2, 1], dtype=torch.int32)
        return b

    monkeypatch.setattr(autoprec_mod.ext_calc_precision, "calc_precision", fake_calc)
    ap.refresh_bits()
    assert seen["b"].dtype == torch.int32 and seen["b"].tolist() == [32, 32, 32]
    assert seen["C"].dtype == torch.float32 and seen["w"].dtype == torch.int64
    assert seen["w"].tolist() == [128 * 96, 64 * 192, 32 * 384] and seen["target"] == ap.total_bits
    assert ap.bits == {0: 8, 1: 2, 2: 1} and q.bits == ap.bits and q.bits is not ap.bits


def test_refresh_bits_end_to_end_on_the_library():
    q = quantizer_mod.Quantizer(default_bit=4, swap=False, prefetch=False)
    q.dims = {i: n for i, n in enumerate([128 * 96, 64 * 192, 32 * 384, 4096])}
    q.bits = {i: 4 for i in q.dims}
    ap = autoprec_mod.AutoPrecision(None, q, bits=2, max_bits=32, work_dir="./log/", adapt_interval=1000,
                                    log_interval=-1)
    ap.init_from_dims()
    ap.C = {0: 50.0, 1: 1.0, 2: 0.02, 3: 7.0}
    ap.refresh_bits()
    import oracle
    want = oracle.calc_precision(np.full(4, 32, np.int32), np.array([50.0, 1.0, 0.02, 7.0], np.float32),
                                 np.array(list(q.dims.values()), np.int64), float(ap.total_bits))
    assert [q.bits[i] for i in range(4)] == want.tolist()
