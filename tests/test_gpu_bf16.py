"""bfloat16 activations (an addition: the reference knows float and half).

The rule: a bfloat16 tensor is quantized exactly as the float path quantizes the float values it holds -
same codes, same float scale, same minimum (which is one of the inputs, so it goes back to bfloat16
unchanged) - and dequantize rounds float(code) / scale + min to bfloat16 once, to nearest even.  So the
checker is the float oracle on the widened tensor, followed by torch's float -> bfloat16 conversion (an
independent round-to-nearest-even), and a second check runs the float kernels on the widened tensor.
"""
import copy

import numpy as np
import pytest
import torch

import oracle
from gact import ops
from gact.batched import BatchedQuantizer
from gact.conf import config
from gact.cpp_extension import calc_precision as ext_calc_precision

pytestmark = pytest.mark.gpu

MODES = {"deterministic": oracle.NOISE_CONST, "reference": oracle.NOISE_REF, "fast": oracle.NOISE_FAST}


@pytest.fixture(autouse=True)
def _restore_config():
    saved = copy.copy(config.__dict__)
    yield
    config.__dict__.update(saved)


def u32(a):
    return np.ascontiguousarray(a).view(np.uint32)


def check(x_bf16, bits, stream, seed):
    """x_bf16: CPU bfloat16 tensor of any shape."""
    wide = x_bf16.float()
    want = oracle.op_quantize(wide.numpy(), bits, MODES[stream], seed)
    q = ops.op_quantize(x_bf16.cuda(), bits, seed, rng_stream=stream)
    N = -(-x_bf16.numel() // 256)
    assert q[2].dtype == torch.float32 and q[3].dtype == torch.bfloat16
    assert q[2].shape == (N, 1, 1) and q[3].shape == (N, 1, 1)
    tag = "%s bits=%d %s" % (tuple(x_bf16.shape), bits, stream)
    np.testing.assert_array_equal(q[0].cpu().numpy().view(np.uint8)[:want[0].size], want[0], err_msg=tag)
    np.testing.assert_array_equal(u32(q[2].cpu().numpy().ravel()), u32(want[2].ravel()), err_msg=tag)
    got_min = q[3].float().cpu().numpy().ravel()
    m = ~np.isnan(want[3].ravel())
    np.testing.assert_array_equal(got_min[m], want[3].ravel()[m], err_msg=tag)

    # the float kernels on the widened tensor give the same bytes and the same scale
    qf = ops.op_quantize(wide.cuda(), bits, seed, rng_stream=stream)
    assert torch.equal(qf[0][:-1], q[0][:-1])            # the last byte is allocated and never written
    assert torch.equal(qf[2].view(torch.int32), q[2].view(torch.int32))

    out = ops.op_dequantize(q, x_bf16.shape)
    assert out.dtype == torch.bfloat16 and out.shape == x_bf16.shape
    ref = torch.from_numpy(oracle.op_dequantize(want, tuple(x_bf16.shape))).to(torch.bfloat16)
    got = out.cpu()
    nan = torch.isnan(ref)
    assert torch.equal(torch.isnan(got), nan), tag
    assert torch.equal(got[~nan].view(torch.int16), ref[~nan].view(torch.int16)), tag
    return q, out


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("stream", ["deterministic", "fast", "reference"])
def test_bf16_equals_the_float_path_on_the_widened_values(bits, stream):
    g = torch.Generator().manual_seed(bits)
    for shape in ((64, 256), (37, 101), (3, 5, 7, 11), (1,), (255,), (257,), (300, 1000)):
        x = (torch.randn(shape, generator=g) * 3).to(torch.bfloat16)
        check(x, bits, stream, 17 + bits)


def test_bf16_edge_groups():
    rows = [torch.zeros(256), torch.full((256,), 1.5), torch.linspace(-1e-30, 1e-30, 256),
            torch.linspace(-3e38, 3e38, 256), torch.cat([torch.zeros(255), torch.ones(1)]),
            torch.relu(torch.randn(256, generator=torch.Generator().manual_seed(1))),
            torch.randn(256, generator=torch.Generator().manual_seed(2)) * 1e-3 + 100.0]
    x = torch.stack(rows).to(torch.bfloat16)
    for bits in (1, 2, 4, 8):
        for stream in ("deterministic", "fast"):
            check(x, bits, stream, 5)


def test_bf16_random_cases():
    rng = np.random.default_rng(77)
    for case in range(150):
        numel = int(rng.integers(1, 30000))
        scale = float(rng.choice([1e-4, 1.0, 300.0]))
        x = (torch.randn(numel, generator=torch.Generator().manual_seed(case)) * scale).to(torch.bfloat16)
        if rng.random() < 0.5:
            x = torch.relu(x)
        check(x, int(rng.choice([1, 2, 4, 8])), str(rng.choice(list(MODES))), int(rng.integers(0, 2 ** 31 - 1)))


def test_bf16_large_tensor_with_capped_occupancy():
    x = torch.randn((196608 + 5, 256), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    for bits in (8, 2):
        check(x, bits, "fast", 99)


def test_bf16_error_is_that_of_the_width():
    x = torch.rand((512, 256), generator=torch.Generator().manual_seed(4)).to(torch.bfloat16)
    for bits, bound in ((8, 1.0 / 255 + 2 ** -8), (4, 1.0 / 15 + 2 ** -8)):
        q = ops.op_quantize(x.cuda(), bits, 1)
        out = ops.op_dequantize(q, x.shape).float().cpu()
        assert (out - x.float()).abs().max().item() <= bound      # one code step plus the final rounding
        assert abs((out - x.float()).mean().item()) < 2e-3          # stochastic rounding stays unbiased


def test_bf16_batched_equals_tensor_by_tensor():
    rng = np.random.default_rng(5)
    shapes = [(8, 3136, 96), (8, 784, 192), (8, 196, 384), (8, 49, 768), (3, 100)]
    dtypes = [torch.bfloat16, torch.float16, torch.bfloat16, torch.float32, torch.bfloat16]
    tensors = [torch.randn(s, generator=torch.Generator().manual_seed(i)).to(d).cuda()
               for i, (s, d) in enumerate(zip(shapes, dtypes))]
    L = len(tensors)
    bits = torch.tensor([1, 2, 4, 8, 2], dtype=torch.int32, device="cuda")
    seeds = [int(s) for s in rng.integers(0, 2 ** 31 - 1, L)]
    bq = BatchedQuantizer([t.numel() for t in tensors], dtypes, "cuda")
    assert bq.dtype_mask == 7
    packed = bq.quantize(tensors, bits, seeds)
    ok, need = packed.ok()
    assert ok and need <= packed.packed.numel()
    outs = bq.dequantize(packed)
    for i, t in enumerate(tensors):
        q = ops.op_quantize(t, int(bits[i]), seeds[i])
        pk, b, sc, mn = packed.per_tensor(i)
        assert b == int(bits[i]) and sc.dtype == q[2].dtype and mn.dtype == q[3].dtype
        assert torch.equal(pk, q[0][:pk.numel()]), i
        assert torch.equal(sc.contiguous().view(torch.uint8), q[2].view(torch.uint8)), i
        assert torch.equal(mn.contiguous().view(torch.uint8), q[3].view(torch.uint8)), i
        one = ops.op_dequantize(q, t.shape)
        assert outs[i].dtype == t.dtype and torch.equal(outs[i].view(torch.uint8), one.view(torch.uint8)), i


def test_bf16_autocast_training_under_the_hooks():
    import gact
    from gact.controller import Controller
    torch.manual_seed(0)
    net = torch.nn.Sequential(torch.nn.Linear(256, 512), torch.nn.GELU(), torch.nn.Linear(512, 512), torch.nn.ReLU(),
                              torch.nn.Linear(512, 10)).cuda()
    x = torch.randn(64, 256, device="cuda")
    y = torch.randint(0, 10, (64,), device="cuda")

    def grads(level):
        net.zero_grad(set_to_none=True)
        ctl = None
        if level:
            gact.set_optimization_level(level)
            ctl = Controller(net)
            ctl.install_hook()
        try:
            with torch.autocast("cuda", dtype=torch.bfloat16):
                loss = torch.nn.functional.cross_entropy(net(x), y)
            loss.backward()
        finally:
            if ctl:
                ctl.uninstall_hook()
        seen = set(ctl.quantizer.dims) if ctl else set()
        return torch.cat([p.grad.ravel() for p in net.parameters()]), len(seen)

    exact, _ = grads(None)
    approx, n = grads("L1.1")
    assert n >= 4                                   # bfloat16 activations went through the hooks
    rel = ((approx - exact).norm() / exact.norm()).item()
    assert rel < 0.1, rel                           # 8 bit codes of the activations and of the cast weights
