"""The hook layer end to end on the GPU: a small network trained under Controller hooks, as the
reference's integration tests do (tests/test_controller_auto_precision.py, tests/test_bert.py)."""
import copy

import pytest
import torch
import torch.nn as nn

import gact
from gact.conf import config
from gact.controller import Controller

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def restore_config():
    saved = dict(vars(config))
    yield
    vars(config).update(saved)


def make_net():
    torch.manual_seed(0)
    return nn.Sequential(
        nn.Conv2d(3, 16, 3, padding=1), nn.BatchNorm2d(16), nn.ReLU(),
        nn.Conv2d(16, 32, 3, padding=1), nn.ReLU(), nn.Dropout(0.1), nn.AdaptiveAvgPool2d(4),
        nn.Flatten(), nn.Linear(512, 64), nn.ReLU(), nn.Linear(64, 10)).cuda()


def grads_under_hooks(level, x, y, net):
    gact.set_optimization_level(level)
    ctl = Controller(net)
    ctl.install_hook()
    try:
        torch.manual_seed(1)
        loss = nn.functional.cross_entropy(net(x), y)
        loss.backward()
    finally:
        ctl.uninstall_hook()
    return loss.item(), torch.cat([p.grad.ravel() for p in net.parameters()])


def test_gradients_under_compression_approach_the_exact_ones():
    torch.manual_seed(7)
    x = torch.randn(16, 3, 32, 32, device="cuda")
    y = torch.randint(0, 10, (16,), device="cuda")
    net = make_net()
    torch.manual_seed(1)
    loss0 = nn.functional.cross_entropy(net(x), y)
    loss0.backward()
    exact = torch.cat([p.grad.ravel() for p in net.parameters()])
    errs = {}
    for level in ("L1.2", "L1", "L1.1"):          # fixed 2, 4, 8 bit
        n2 = copy.deepcopy(net)
        n2.zero_grad()
        loss, g = grads_under_hooks(level, x, y, n2)
        assert abs(loss - loss0.item()) < 1e-5    # the forward pass is untouched
        errs[level] = ((g - exact).norm() / exact.norm()).item()
    # every saved float activation is compressed, the 160-element log-softmax of the loss included, so
    # even 8 bits leave a few percent; what must hold is the ordering and a sane magnitude
    assert errs["L1.1"] < 0.2 and errs["L1.1"] < errs["L1"] < errs["L1.2"] < 1.5, errs


def test_hooks_on_hip_kernels_equal_hooks_on_the_cpu_oracle(monkeypatch):
    """The same forward/backward twice: once with the HIP operators, once with the operators replaced by
    the CPU oracle (same widths, seeds and noise stream).  Every tensor handed back to autograd must be
    bit-identical, hence the gradients agree."""
    import numpy as np

    import gact.quantizer as quantizer_mod
    import oracle

    torch.manual_seed(8)
    x = torch.randn(8, 3, 32, 32, device="cuda")
    y = torch.randint(0, 10, (8,), device="cuda")
    net = make_net()
    net.eval()
    for level, stream in (("L1.2", "fast"), ("L1", "reference"), ("L1.1", "deterministic")):
        config.rng_stream = stream
        mode = {"fast": oracle.NOISE_FAST, "reference": oracle.NOISE_REF, "deterministic": oracle.NOISE_CONST}[stream]
        seen = {"hip": [], "cpu": []}
        real_q, real_dq = quantizer_mod.op_quantize, quantizer_mod.op_dequantize

        def hip_dq(q, shape):
            out = real_dq(q, shape)
            seen["hip"].append(out.detach().cpu())
            return out

        def cpu_q(t, bit, seed):
            ref = oracle.op_quantize(t.detach().cpu().numpy(), bit, mode, seed)
            return [ref, bit, None, None]

        def cpu_dq(q, shape):
            out = torch.from_numpy(oracle.op_dequantize(q[0], tuple(shape)))
            seen["cpu"].append(out)
            return out.cuda()

        n_hip, n_cpu = copy.deepcopy(net), copy.deepcopy(net)
        monkeypatch.setattr(quantizer_mod, "op_dequantize", hip_dq)
        _, g_hip = grads_under_hooks(level, x, y, n_hip)
        monkeypatch.setattr(quantizer_mod, "op_quantize", cpu_q)
        monkeypatch.setattr(quantizer_mod, "op_dequantize", cpu_dq)
        config.rng_stream = stream
        _, g_cpu = grads_under_hooks(level, x, y, n_cpu)
        monkeypatch.setattr(quantizer_mod, "op_quantize", real_q)
        monkeypatch.setattr(quantizer_mod, "op_dequantize", real_dq)
        assert len(seen["hip"]) == len(seen["cpu"]) >= 5
        for a, b in zip(seen["hip"], seen["cpu"]):
            assert a.shape == b.shape and np.array_equal(a.numpy(), b.numpy())
        assert torch.allclose(g_hip, g_cpu, rtol=1e-4, atol=1e-7)


def train(swap, steps=6, adapt_interval=4, max_bit=32, bit=4):
    vars(config).update(dict(compress_activation=True, auto_prec=True, bit=bit, swap=swap, prefetch=swap,
                             adapt_interval=adapt_interval, max_bit=max_bit, log_interval=-1))
    net = make_net()
    net.eval()      # no dropout / batch statistics: the run must be reproducible bit for bit
    opt = torch.optim.SGD(net.parameters(), lr=0.05)
    ctl = Controller(net)
    ctl.install_hook()
    torch.manual_seed(3)
    data = [(torch.randn(8, 3, 32, 32, device="cuda"), torch.randint(0, 10, (8,), device="cuda")) for _ in range(steps)]
    losses = []
    try:
        for x, y in data:
            def backprop():
                net.zero_grad()
                nn.functional.cross_entropy(net(x), y).backward()
            opt.zero_grad()
            loss = nn.functional.cross_entropy(net(x), y)
            loss.backward()
            opt.step()
            losses.append(loss.item())
            ctl.iterate(backprop)
    finally:
        ctl.uninstall_hook()
    return losses, dict(ctl.quantizer.bits)


def test_auto_precision_training_is_identical_with_and_without_swap():
    # tests/test_controller_auto_precision.py:145 of the reference: the losses agree exactly
    base, bits = train(swap=False)
    swapped, bits_s = train(swap=True)
    # the compressed tensors are identical either way; the convolution backward kernels accumulate with
    # atomics, so the losses may differ in the last float digits from run to run
    assert len(base) == len(swapped) and all(abs(a - b) <= 2e-6 * abs(a) for a, b in zip(base, swapped))
    assert bits == bits_s
    assert set(bits.values()) <= {1, 2, 4, 8, 32} and len(bits) >= 4
    assert all(l == l for l in base)              # no NaN


class MaskedScale(torch.autograd.Function):
    """Dropout as the torch versions the reference targets saved it: a uint8 0/1 mask kept for backward."""

    @staticmethod
    def forward(ctx, x, mask):
        ctx.save_for_backward(mask)
        return x * mask

    @staticmethod
    def backward(ctx, g):
        (mask,) = ctx.saved_tensors
        return g * mask, None


def test_saved_uint8_mask_takes_the_one_bit_mask_kernels(monkeypatch):
    """quantizer.py:52-55,102-104 of the reference: a saved uint8 tensor holding only 0 and 1 is packed to one
    bit per element; the backward pass must get the very same mask back."""
    import gact.quantizer as quantizer_mod

    calls = {"pack": 0, "unpack": 0, "words": 0}
    real_qm, real_dm = quantizer_mod.op_quantize_mask, quantizer_mod.op_dequantize_mask

    def qm(t):
        q = real_qm(t)
        calls["pack"] += 1
        calls["words"] = q[0].numel()
        assert q[0].dtype == torch.int32
        return q

    def dm(q):
        calls["unpack"] += 1
        return real_dm(q)

    monkeypatch.setattr(quantizer_mod, "op_quantize_mask", qm)
    monkeypatch.setattr(quantizer_mod, "op_dequantize_mask", dm)
    torch.manual_seed(11)
    lin = nn.Linear(300, 77).cuda()
    x = torch.randn(100, 300, device="cuda")
    mask = (torch.rand(100, 77, device="cuda") < 0.7).to(torch.uint8)       # 7700 elements: a ragged last word
    out = MaskedScale.apply(lin(x), mask)
    out.sum().backward()
    exact = lin.weight.grad.clone()
    lin.zero_grad()

    gact.set_optimization_level("L1.1")
    ctl = Controller(lin)
    ctl.install_hook()
    try:
        out = MaskedScale.apply(lin(x), mask)
        out.sum().backward()
    finally:
        ctl.uninstall_hook()
    assert calls == {"pack": 1, "unpack": 1, "words": (7700 + 31) // 32}
    # the mask comes back exactly; the only lossy tensor is the 8-bit input of the linear layer
    assert torch.equal(lin.bias.grad, mask.float().sum(0))
    assert ((lin.weight.grad - exact).norm() / exact.norm()).item() < 0.02


def test_saved_bool_masks_are_packed_to_one_bit_losslessly(monkeypatch):
    """Not in the reference: dropout in current PyTorch saves a bool mask, which the uint8 rule never sees.
    With config.compress_bool_masks it goes through the mask kernels (no values inspected, nothing
    synchronised) and comes back as the same bool tensor, so a dropout layer's gradient is exact."""
    import gact.quantizer as quantizer_mod

    packed_words = []
    real_qm = quantizer_mod.op_quantize_mask

    def qm(t):
        assert t.dtype == torch.uint8
        q = real_qm(t)
        packed_words.append(q[0].numel())
        return q

    monkeypatch.setattr(quantizer_mod, "op_quantize_mask", qm)
    drop = nn.Dropout(0.3).cuda().train()
    x = torch.randn(64, 1000, device="cuda", requires_grad=True)
    upstream = torch.randn(64, 1000, device="cuda")

    def run(hooked):
        torch.manual_seed(5)
        torch.cuda.manual_seed_all(5)
        x.grad = None
        gact.set_optimization_level("L1")
        ctl = Controller(drop)
        if hooked:
            ctl.install_hook()
        try:
            drop(x).backward(upstream)
        finally:
            ctl.uninstall_hook()
        return x.grad.clone()

    exact = run(False)
    assert packed_words == []
    assert torch.equal(run(True), exact)
    assert packed_words == [(64000 + 31) // 32]

    # the tuple protocol: a fourth entry carries the dtype; strided and small tensors
    q = quantizer_mod.Quantizer(default_bit=4, swap=False, prefetch=False)
    m = torch.rand(300, 130, device="cuda") < 0.5
    for t in (m, m.t().contiguous(), m[::2, 1::3].repeat(3, 5), m.reshape(3, 100, 130)):
        h = q.quantize(t)
        assert h[:2] == (True, True) and h[3] == torch.bool
        back = q.dequantize(h)
        assert back.dtype == torch.bool and back.shape == t.shape and torch.equal(back, t)
    # views that are not contiguous are left alone: a broadcast mask occupies less than it looks
    for t in (m.t(), m[:1].expand(300, 130), m[::2]):
        assert q.quantize(t)[0] is False
    small = torch.rand(10, 10, device="cuda") < 0.5
    assert q.quantize(small) == (False, small) or q.quantize(small)[1] is small
    config.compress_bool_masks = False
    assert q.quantize(m)[0] is False


class TwoReaders(nn.Module):
    """One activation saved for backward by two operators: both linear layers keep `h` as their input."""

    def __init__(self):
        super().__init__()
        torch.manual_seed(0)
        self.stem = nn.Linear(64, 128)
        self.left, self.right = nn.Linear(128, 32), nn.Linear(128, 32)

    def forward(self, x):
        h = torch.relu(self.stem(x))
        return self.left(h) + self.right(h)


def test_check_dup_compresses_a_twice_saved_activation_once(monkeypatch):
    """quantizer.py:85-93,106-112,138-141 of the reference: with config.check_dup the key of a saved tensor is its
    address, a strided sample and its sum, a second save under the same key adds a consumer instead of new
    codes, and the codes are dropped when the last consumer has read them."""
    import gact.quantizer as quantizer_mod

    real_q = quantizer_mod.op_quantize
    launches = []

    def counting_q(t, *a, **k):
        launches.append((t.data_ptr(), tuple(t.shape)))
        return real_q(t, *a, **k)

    monkeypatch.setattr(quantizer_mod, "op_quantize", counting_q)
    torch.manual_seed(5)
    x = torch.randn(48, 4, 64, device="cuda")       # rank 3: the input is compressed too
    target = torch.randn(48, 4, 32, device="cuda")
    results = {}
    for dup in (False, True):
        vars(config).update(dict(compress_activation=True, auto_prec=False, bit=4, swap=False, prefetch=False,
                                 check_dup=dup, rng_stream="deterministic"))
        net = TwoReaders().cuda()
        ctl = Controller(net)
        launches.clear()
        with ctl:
            loss = nn.functional.mse_loss(net(x), target)
            held = {k: v[1] for k, v in ctl.quantizer.ptr_qtensor_map.items()}
            saves = ctl.quantizer.tid
            loss.backward()
        results[dup] = (list(launches), held, saves, dict(ctl.quantizer.ptr_qtensor_map),
                        torch.cat([p.grad.ravel() for p in net.parameters()]))
    plain, deduped = results[False], results[True]
    assert plain[2] == deduped[2] >= 3                  # the hooks saw the same saves either way
    assert len(plain[0]) == plain[2]                    # one launch per save without check_dup
    # the key is the address, a strided sample and the sum, not the shape: h is saved by relu as [48,4,128] and by
    # both readers as [192,128], three saves of one buffer
    addresses = [p for p, _ in plain[0]]
    shared = [p for p in set(addresses) if addresses.count(p) > 1]
    assert len(shared) == 1 and addresses.count(shared[0]) == 3
    # with check_dup: one launch per distinct buffer, the shared one held for all of its consumers
    assert len(deduped[0]) == len(set(addresses)) == deduped[2] - 2
    assert sorted(deduped[1].values()) == [1] * (len(set(addresses)) - 1) + [3]
    assert plain[3] == {} and deduped[3] == {}          # every compressed copy was released by the backward pass
    assert torch.equal(plain[4], deduped[4])            # deterministic rounding: the very same gradients


def test_device_calc_precision_gives_the_host_tables(monkeypatch):
    """config.device_calc_precision: the sensitivities stay on the GPU, the greedy of calc_precision.cc:66-118 runs
    there, and the tables (autoprec.py:188-209 of the reference) equal the host routine's on the same
    sensitivities, adaptation after adaptation, from max_bit 32 and from 8."""
    from gact.autoprec import AutoPrecision

    seen = []
    on_device = AutoPrecision.refresh_bits_on_device

    def both(self, C_dev):
        on_device(self, C_dev)
        device_bits, device_C = dict(self.bits), dict(self.C)
        assert self.quantizer.bits == device_bits
        self.refresh_bits()                     # the host routine on the sensitivities that came back
        assert self.C == device_C
        seen.append((device_bits, dict(self.bits)))

    monkeypatch.setattr(AutoPrecision, "refresh_bits_on_device", both)
    for max_bit, avg in ((32, 4), (8, 2), (32, 3)):
        before = len(seen)
        vars(config).update(dict(device_calc_precision=True))
        losses, bits = train(swap=False, steps=6, adapt_interval=2, max_bit=max_bit, bit=avg)
        assert len(seen) - before == 3          # adaptations at iterations 0, 2, 4
        for device_bits, host_bits in seen[before:]:
            assert device_bits == host_bits and len(device_bits) >= 4
            assert set(device_bits.values()) <= {1, 2, 4, 8, 32}
        assert bits == seen[-1][0]
        assert all(l == l for l in losses)


def test_device_calc_precision_on_ties_zero_and_capped_sensitivities():
    from gact.autoprec import AutoPrecision, SENSITIVITY_CAP

    class Tables:
        bits = {}

    dims = {i: n for i, n in enumerate([4096, 4096, 4096, 100, 100, 65536, 65536, 7, 300000, 300000])}
    cases = [[1.0] * 10, [0.0] * 10, [SENSITIVITY_CAP] * 5 + [0.0] * 5,
             [3.0, 3.0, 3.0, 1e-30, 1e-30, 7.5, 7.5, 1e10, 0.5, 0.5], [float(i % 3) for i in range(10)]]
    for max_bit, avg in ((32, 4), (8, 2), (8, 1), (32, 8)):
        for C in cases:
            tables = []
            for device in (False, True):
                ap = AutoPrecision(None, Tables(), avg, max_bit, "/tmp", 1, -1)
                ap.quantizer.dims = dict(dims)
                ap.init_from_dims()
                if device:
                    ap.refresh_bits_on_device(torch.tensor(C, dtype=torch.float32, device="cuda"))
                    assert [ap.C[l] for l in dims] == [float(torch.tensor(c, dtype=torch.float32)) for c in C]
                else:
                    ap.C = {l: c for l, c in zip(dims, C)}
                    ap.refresh_bits()
                tables.append(dict(ap.bits))
                assert ap.quantizer.bits == ap.bits
            assert tables[0] == tables[1], (max_bit, avg, C, tables)
