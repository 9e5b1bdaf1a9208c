"""The five benchmark workloads (config 1-5 of bench.py) at their full sizes.

Each is checked three ways: against the CPU oracle on the same seeded input (bit-exact packed bytes,
scale, min and dequantized values - the C oracle finishes these sizes in seconds), through size-independent
properties (codes in range, |x_hat - x| within one quantisation step, unbiased rounding), and by running
two different kernel paths against each other (fused quantize vs minimax + pack with caller-supplied
min/max; fused dequantize vs the general-shape unpack kernel; batched launch vs tensor by tensor).
"""
import numpy as np
import pytest
import torch

import oracle
from gact import ops
from gact.batched import BatchedQuantizer
from gact.cpp_extension import _abi
from gact.cpp_extension import calc_precision as ext_calc_precision
from gact.cpp_extension import minimax as ext_minimax
from gact.cpp_extension import quantization as ext_quantization

pytestmark = pytest.mark.gpu

MODES = {"deterministic": oracle.NOISE_CONST, "reference": oracle.NOISE_REF, "fast": oracle.NOISE_FAST}


def gen(shape, dtype, kind, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32)
    if kind == "relu":
        x = torch.relu(x)
    elif kind == "relu60":
        x = torch.relu(x - 0.2533)
    elif kind == "softmax":
        x = torch.softmax(x, dim=-1)
    return x.to(dtype).contiguous()


def bits_of(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


def check_against_oracle(x, bits, stream, seed):
    q = ops.op_quantize(x, bits, seed, rng_stream=stream)
    out = ops.op_dequantize(q, x.shape)
    torch.cuda.synchronize()
    ref = oracle.op_quantize(x.cpu().numpy(), bits, MODES[stream], seed)
    n = ref[0].size
    got = q[0].cpu().numpy().view(np.uint8)[:n]
    assert np.array_equal(got, ref[0]), "packed bytes differ at %d positions" % int((got != ref[0]).sum())
    assert np.array_equal(bits_of(q[2].cpu().numpy()), bits_of(ref[2]))
    assert np.array_equal(q[3].cpu().numpy(), ref[3])
    want = oracle.op_dequantize(ref, tuple(x.shape))
    assert np.array_equal(bits_of(out.cpu().numpy().reshape(-1)), bits_of(want.reshape(-1)))
    return q, out


def check_properties(x, q, out, bits, stochastic):
    N = q[3].numel()
    mn = q[3].reshape(N).float()
    sc = q[2].reshape(N).float()
    pad = N * 256 - x.numel()
    xf = x.reshape(-1).float()
    if pad:
        xf = torch.cat([xf, torch.zeros(pad, device=x.device)])
    xg = xf.reshape(N, 256)
    og = out.reshape(-1).float()
    if pad:
        og = torch.cat([og, torch.zeros(pad, device=x.device)])
    og = og.reshape(N, 256)
    assert torch.equal(mn, xg.min(dim=1).values)
    step = (xg.max(dim=1).values - mn) / (2 ** bits - 1)
    err = (og - xg)[: N - 1 if pad else N]          # the padded last group also holds implicit zeros
    st = step[: N - 1 if pad else N]
    if x.dtype == torch.float32:
        assert bool((err.abs() <= st[:, None] * 1.001 + 1e-6).all())
        if stochastic:
            # unbiased rounding: mean error within 1e-3 of the typical range
            assert abs(err.mean().item()) < 1e-3 * st.mean().item() * (2 ** bits - 1)


def cross_check_kernel_paths(x, q, bits, stream, seed):
    """fused quantize == minimax + pack(GIVEN min/max); fused dequantize == general-shape unpack kernel."""
    if x.numel() % 256:
        return
    N = x.numel() // 256
    groups = x.reshape(N, 256)
    mn, mx = ext_minimax.minimax(groups)
    packed, scale = ext_quantization.pack_single_precision(groups.view(N, 1, 256), mn.view(N, 1, 1), mx.view(N, 1, 1),
                                                           bits, True, seed, rng_stream=stream)
    assert torch.equal(packed[:-1], q[0][:-1]) and torch.equal(scale.view(-1), q[2].view(-1))
    assert torch.equal(mn, q[3].view(-1))
    # general-shape kernel: the same bytes viewed as [N/2, 2, 128] do not keep the byte layout, so use a
    # sample of whole byte rows as their own small tensors through the (N,2,128)-shaped entry point instead
    wpt = 8 // bits
    rows = min(64, N // wpt)
    sub = groups[: rows * wpt].contiguous()
    smn, smx = ext_minimax.minimax(sub.view(rows * wpt * 2, 128))
    pk2, sc2 = ext_quantization.pack_single_precision(sub.view(rows * wpt, 2, 128), smn.view(-1, 2, 1), smx.view(-1, 2, 1),
                                                      bits, True, seed, rng_stream="deterministic")
    un2 = ext_quantization.unpack_single_precision(pk2, bits, sc2, smn.view(-1, 2, 1), rows * wpt, 2, 128)
    ref = oracle.unpack(pk2.cpu().numpy().view(np.uint8)[:-1], bits, sc2.cpu().numpy().reshape(-1),
                        smn.cpu().numpy().reshape(-1), rows * wpt, 2, 128)
    assert np.array_equal(bits_of(un2.cpu().numpy().reshape(-1)), bits_of(ref.reshape(-1)))


def test_config1_fp32_2bit_deterministic():
    torch.manual_seed(0)
    x = torch.randn(4096, 1024).cuda()
    q, out = check_against_oracle(x, 2, "deterministic", 0)
    check_properties(x, q, out, 2, stochastic=False)
    cross_check_kernel_paths(x, q, 2, "deterministic", 0)


@pytest.mark.parametrize("stream", ["fast", "reference"])
def test_config2_resnet_activation_fp32_4bit(stream):
    x = gen((128, 256, 56, 56), torch.float32, "relu", 0)
    q, out = check_against_oracle(x, 4, stream, 42)
    check_properties(x, q, out, 4, stochastic=True)
    cross_check_kernel_paths(x, q, 4, stream, 42)


@pytest.mark.parametrize("name,shape,kind,bits", [
    ("hidden", (32 * 512, 1024), "randn", 8),
    ("gelu-input", (32 * 512, 4096), "randn", 4),
    ("attention-probs", (32, 16, 512, 512), "softmax", 2),
    ("hidden-2bit", (32 * 512, 1024), "randn", 2),
])
def test_config3_bert_large_fp16(name, shape, kind, bits):
    x = gen(shape, torch.float16, kind, 3)
    q, out = check_against_oracle(x, bits, "fast", 7)
    check_properties(x, q, out, bits, stochastic=True)
    cross_check_kernel_paths(x, q, bits, "fast", 7)


@pytest.mark.parametrize("groups", [32768 + 3, 100000 + 3, 196608 + 3, 262144 + 3])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_large_tensor_launches(dtype, bits, groups):
    """Large tensors take their own dequantize geometry (from 73 728, 98 304 or 131 072 groups on) and some kernels are
    launched with fewer resident waves per CU (a request for dynamic LDS that they never touch; the last of those
    sizes is 262 144 groups), quantize changes how its rows are worked through at 32 768 groups, and 1 bit leaves the
    wave-per-super-group kernel at 40 960 (half) and 262 144 groups (float): every type and width just past the first,
    the middle and the last of those sizes, with a partial last super-group."""
    x = gen((groups, 256), dtype, "relu", 5)
    q, out = check_against_oracle(x, bits, "fast", 13)
    check_properties(x, q, out, bits, stochastic=True)


def test_config4_gcn_features_fp32_1bit():
    x = gen((169343, 256), torch.float32, "relu60", 4)
    zeros = (x == 0).float().mean().item()
    assert 0.55 < zeros < 0.65
    assert (169343 % 8) == 7                        # partial last byte row: the boundary-check path
    q, out = check_against_oracle(x, 1, "fast", 11)
    check_properties(x, q, out, 1, stochastic=True)
    cross_check_kernel_paths(x, q, 1, "fast", 11)
    # the same features with half the width: numel is then not a multiple of 256 (zero-padded last group)
    x2 = x[:, :128].contiguous()
    assert x2.numel() % 256 == 128
    check_against_oracle(x2, 1, "fast", 11)


def test_config5_adaptive_step_batched():
    shapes = [(128, 3136, 96)] * 20 + [(128, 784, 192)] * 20 + [(128, 196, 384)] * 60 + [(128, 49, 768)] * 20
    g = torch.Generator(device="cuda").manual_seed(5)
    xs = [torch.randn(s, generator=g, device="cuda", dtype=torch.float16) for s in shapes]
    L = len(xs)
    assert sum(x.numel() for x in xs) == 1830420480
    rng = np.random.default_rng(5)
    C = np.exp(rng.normal(0.0, 2.0, L)).astype(np.float32)
    w = np.array([x.numel() for x in xs], dtype=np.int64)
    target = 2.0 * float(w.sum())

    # bit allocation: device == host == oracle, widths in {1,2,4,8}, budget met
    want_bits = oracle.calc_precision(np.full(L, 8, np.int32), C, w, target)
    bits = ext_calc_precision.calc_precision_device(torch.full((L,), 8, dtype=torch.int32, device="cuda"),
                                                    torch.from_numpy(C).cuda(), torch.from_numpy(w).cuda(), target)
    host_bits = bits.cpu().numpy()
    assert np.array_equal(host_bits, want_bits)
    assert set(host_bits.tolist()) <= {1, 2, 4, 8} and float((host_bits * w).sum()) <= target

    seeds = [100 + i for i in range(L)]
    bq = BatchedQuantizer([x.numel() for x in xs], [torch.float16] * L, "cuda")
    q = bq.quantize(xs, bits, seeds, arena_bytes=bq.arena_bytes_for_budget(target), rng_stream="fast")
    ok, need = q.ok()
    assert ok and need <= q.packed.numel()
    outs = bq.dequantize(q)
    torch.cuda.synchronize()

    # every tensor: batched == single-tensor kernels; a sample of tensors (one per shape and width) == oracle
    sampled = {}
    for i, x in enumerate(xs):
        b = int(host_bits[i])
        single = ops.op_quantize(x, b, seeds[i], rng_stream="fast")
        pk, bb, sc, mn = q.per_tensor(i)
        assert bb == b
        assert torch.equal(pk, single[0][: pk.numel()]), "tensor %d: packed bytes" % i
        assert torch.equal(sc.view(torch.int16), single[2].view(torch.int16)) and torch.equal(mn, single[3])
        assert torch.equal(outs[i], ops.op_dequantize(single, x.shape)), "tensor %d: dequantized" % i
        sampled.setdefault((tuple(x.shape), b), i)
    for (shape, b), i in sampled.items():
        ref = oracle.op_quantize(xs[i].cpu().numpy(), b, oracle.NOISE_FAST, seeds[i])
        pk, _, sc, mn = q.per_tensor(i)
        assert np.array_equal(pk.cpu().numpy().view(np.uint8), ref[0])
        want = oracle.op_dequantize(ref, shape)
        assert np.array_equal(bits_of(outs[i].cpu().numpy().reshape(-1)), bits_of(want.reshape(-1)))
