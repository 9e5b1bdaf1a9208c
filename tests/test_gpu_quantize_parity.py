"""HIP kernels against the CPU oracle on the same seeded inputs, through the C ABI.

Bars: packed bytes, scale and the bit allocation bit-exact; min equal by value; dequantized values
bit-exact (the stated tolerance is 1 ulp; the kernels use an IEEE division, so 0 ulp is asserted).
The reference's trailing, never-written packed byte is excluded from every comparison.
"""
import numpy as np
import pytest
import torch

import oracle
from gact import ops
from gact.conf import config
from gact.cpp_extension import _abi

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16]
BITS = [1, 2, 4, 8]
MODES = {"deterministic": oracle.NOISE_CONST, "reference": oracle.NOISE_REF, "fast": oracle.NOISE_FAST}


def make_input(kind, shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "randn":
        x = torch.randn(shape, generator=g)
    elif kind == "relu":
        x = torch.relu(torch.randn(shape, generator=g))
    elif kind == "uniform":
        x = torch.rand(shape, generator=g)
    elif kind == "wide":
        x = torch.randn(shape, generator=g) * 100.0
    else:
        raise ValueError(kind)
    return x.to(dtype)


def check_quantize(x_cpu, bits, mode_name, seed, noise=None):
    x = x_cpu.cuda()
    if noise is not None:
        q = ops.op_quantize(x, bits, seed, noise=noise.cuda())
        ref = oracle.op_quantize(x_cpu.numpy(), bits, oracle.NOISE_INJECT, seed, noise.numpy())
    else:
        q = ops.op_quantize(x, bits, seed, rng_stream=mode_name)
        ref = oracle.op_quantize(x_cpu.numpy(), bits, MODES[mode_name], seed)
    torch.cuda.synchronize()
    pk, b, sc, mn = q
    assert b == bits
    n_written = ref[0].size
    assert pk.dtype == torch.int8 and pk.numel() == n_written + 1
    assert sc.shape == ref[2].shape and mn.shape == ref[3].shape
    got_mn = mn.cpu().numpy()
    got_sc = sc.cpu().numpy()
    np.testing.assert_array_equal(got_mn, ref[3])  # by value (+0 == -0)
    np.testing.assert_array_equal(got_sc.view(np.uint16 if got_sc.dtype == np.float16 else np.uint32),
                                  ref[2].view(np.uint16 if got_sc.dtype == np.float16 else np.uint32))
    got_pk = pk.cpu().numpy().view(np.uint8)[:n_written]
    bad = np.nonzero(got_pk != ref[0])[0]
    assert bad.size == 0, "packed bytes differ at %d of %d positions, first %s: got %s want %s" % (
        bad.size, n_written, bad[:5], got_pk[bad[:5]], ref[0][bad[:5]])
    return q, ref


def check_dequantize(q, ref, shape):
    out = ops.op_dequantize(q, shape)
    torch.cuda.synchronize()
    want = oracle.op_dequantize(ref, shape)
    got = out.cpu().numpy()
    assert got.shape == tuple(shape) and got.dtype == want.dtype
    it = np.uint16 if got.dtype == np.float16 else np.uint32
    bad = np.nonzero(got.view(it).ravel() != want.view(it).ravel())[0]
    assert bad.size == 0, "dequantized values differ at %d positions, first %s: got %s want %s" % (
        bad.size, bad[:5], got.ravel()[bad[:5]], want.ravel()[bad[:5]])


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("bits", BITS)
@pytest.mark.parametrize("mode", list(MODES))
def test_quantize_dequantize_matches_oracle(dtype, bits, mode):
    # 1100 groups: not a multiple of 8 groups per row nor of 128 per block, N % wpt != 0 for bits 1
    shape = (1100, 256) if bits != 1 else (1099, 256)
    x = make_input("randn", shape, dtype, seed=bits)
    q, ref = check_quantize(x, bits, mode, seed=42)
    check_dequantize(q, ref, shape)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("bits", BITS)
def test_injected_noise_matches_oracle(dtype, bits):
    shape = (515, 256)
    x = make_input("relu", shape, dtype, seed=10 + bits)
    g = torch.Generator().manual_seed(99)
    noise = torch.rand(shape, generator=g)
    noise[0, :8] = torch.tensor([0.0, 1.0, 0.5, 0.25, 0.75, 1e-7, 0.9999999, 0.5])
    q, ref = check_quantize(x, bits, None, seed=0, noise=noise)
    check_dequantize(q, ref, shape)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("bits", BITS)
@pytest.mark.parametrize("shape", [(100, 77), (1, 1), (3, 5, 7), (257,), (2, 3, 4, 129), (169343 // 97, 256)])
def test_ragged_shapes(dtype, bits, shape):
    # numel not a multiple of 256 (zero-padded last group), N % (8/bits) != 0 (partial last byte fields)
    x = make_input("relu", shape, dtype, seed=5)
    q, ref = check_quantize(x, bits, "fast", seed=7)
    check_dequantize(q, ref, shape)
    q, ref = check_quantize(x, bits, "deterministic", seed=7)
    check_dequantize(q, ref, shape)


@pytest.mark.parametrize("kind", ["uniform", "wide"])
@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("bits", BITS)
def test_other_distributions(kind, dtype, bits):
    shape = (640, 256)
    x = make_input(kind, shape, dtype, seed=3)
    for mode in ("deterministic", "fast"):
        q, ref = check_quantize(x, bits, mode, seed=123456)
        check_dequantize(q, ref, shape)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("bits", BITS)
def test_edge_groups(dtype, bits):
    # constant groups (range 0), tiny ranges (half scale overflows to inf), NaN elements, huge values
    x = torch.zeros((64, 256), dtype=torch.float32)
    x[0] = 3.0
    x[1] = -7.5
    x[2] = torch.linspace(1.0, 1.0 + 1e-4, 256)
    x[3] = torch.linspace(-1e-6, 1e-6, 256)
    x[4] = torch.randn(256)
    x[4, 17] = float("nan")
    x[5] = torch.randn(256) * 3e4
    x[6, 0] = 1.0
    x[7] = torch.rand(256) * 6e-5      # subnormal halves
    x[8:] = torch.randn(56, 256)
    x = x.to(dtype)
    for mode in ("deterministic", "reference", "fast"):
        q, ref = check_quantize(x, bits, mode, seed=1)
        out = ops.op_dequantize(q, x.shape).cpu().numpy()
        want = oracle.op_dequantize(ref, x.shape)
        np.testing.assert_array_equal(np.isnan(out), np.isnan(want))
        m = ~np.isnan(want)
        np.testing.assert_array_equal(out[m], want[m])


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_nan_payloads_give_code_zero_like_the_reference(bits):
    """quantization_cuda_kernel.cu:66: fmax(NaN, 0) is 0 whatever the NaN's bits.  float NaNs other than the one
    arithmetic generates (0x7fc00000) keep their payload through the kernel's arithmetic; their low byte must
    not leak into the code, nor into the neighbouring groups' fields of the same byte."""
    torch.manual_seed(9)
    x = torch.randn(32, 256)
    raw = x.view(torch.int32)
    patterns = [0x7fc00001, 0x7fffffff, 0x7fc000ff, 0x7fe0a5c3, -0x003fff01]   # the last: 0xffc000ff, a negative NaN
    for g in range(0, 32, 3):
        for k, pat in enumerate(patterns):
            raw[g, (37 * g + 50 * k) % 256] = pat
    assert torch.isnan(x).sum() == 11 * len(patterns)
    noise = torch.rand(x.shape)
    for mode in ("deterministic", "reference", "fast"):
        q, ref = check_quantize(x, bits, mode, seed=4)
        out = ops.op_dequantize(q, x.shape).cpu().numpy()
        want = oracle.op_dequantize(ref, x.shape)
        np.testing.assert_array_equal(out, want)       # code 0 dequantizes to the group's min: no NaN comes back
    check_quantize(x, bits, "inject", seed=0, noise=noise)


def test_config1_full_size_deterministic():
    # benchmark workload config 1: fp32 [4096,1024] ~ N(0,1), seed 0, 2 bit, deterministic rounding
    torch.manual_seed(0)
    x = torch.randn(4096, 1024)
    q, ref = check_quantize(x, 2, "deterministic", seed=0)
    check_dequantize(q, ref, x.shape)


def test_one_hot_round_trips_at_one_bit():
    # tests/test_act_quantized_ops.py:23-38 of the reference: 0/1 data survives 1-bit quantisation exactly
    config.rng_stream = "fast"
    for inp in (torch.nn.functional.one_hot(torch.arange(1000), 1000),
                torch.nn.functional.one_hot(torch.arange(0, 100) % 77)):
        x = inp.to(torch.float32).cuda()
        for seed in (0, 1, 2):
            d = ops.op_dequantize(ops.op_quantize(x, 1, seed), x.shape)
            assert torch.equal(d.to(torch.uint8), inp.to(torch.uint8).cuda())
            for stream in ("reference", "deterministic"):
                d = ops.op_dequantize(ops.op_quantize(x, 1, seed, rng_stream=stream), x.shape)
                assert torch.equal(d.to(torch.uint8), inp.to(torch.uint8).cuda())


def test_big_min_matches_torch_min():
    # tests/test_act_quantized_ops.py:62-70: (655350, 256) at 4 bit, q_min == torch.min(dim=1)
    x = torch.rand((65535 * 10, 256), device="cuda")
    q_input, q_bit, q_scale, q_min = ops.op_quantize(x, 4, 0)
    assert torch.equal(q_min.reshape(-1), torch.min(x, dim=1).values)
    rng = torch.max(x, dim=1).values - torch.min(x, dim=1).values  # a float subtraction, then double
    ref_scale = (15.0 / (rng.double() + 2e-6)).float()
    assert torch.equal(q_scale.reshape(-1), ref_scale)


def test_32bit_passthrough():
    # tests/test_act_quantized_ops.py:73-91
    x = torch.rand((2048, 256), device="cuda")
    q = ops.op_quantize(x, 32, 0)
    q_input, q_bit, q_scale, q_min = q
    assert torch.equal(q_min.reshape(-1), torch.min(x, dim=1).values)
    assert torch.equal(q_scale.reshape(-1), torch.max(x, dim=1).values - torch.min(x, dim=1).values)
    assert torch.equal(ops.op_dequantize(q, x.shape), x)


def test_empty_tensor():
    x = torch.empty((0, 256), device="cuda")
    q = ops.op_quantize(x, 4, 0)
    assert q[0].numel() == 1 and q[2].shape == (0, 1, 1) and q[3].shape == (0, 1, 1)
    assert ops.op_dequantize(q, x.shape).shape == (0, 256)


@pytest.mark.parametrize("bits", [1, 8])
def test_more_than_2_to_31_elements(bits):
    # indices beyond 32 bits: element offsets, byte offsets and Philox block numbers are 64-bit
    numel = (1 << 31) + 256 * 24 + 100
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.empty(numel, dtype=torch.float16, device="cuda")
    x.normal_(generator=g)
    q = ops.op_quantize(x, bits, 9, rng_stream="deterministic")
    out = ops.op_dequantize(q, x.shape)
    torch.cuda.synchronize()
    N = (numel + 255) // 256
    wpt = 8 // bits
    # oracle on the first and the last 4096 groups (whole byte rows, so the slices are self-contained)
    for g0 in (0, (N - 4096) // 8 * 8):
        g1 = min(g0 + 4096, N)
        xs = x[g0 * 256: min(g1 * 256, numel)].cpu().numpy()
        ref = oracle.op_quantize(xs, bits, oracle.NOISE_CONST)
        nb = ref[0].size
        b0 = (g0 // wpt) * 256
        got = q[0][b0: b0 + nb].cpu().numpy().view(np.uint8)
        assert np.array_equal(got, ref[0])
        assert np.array_equal(q[2][g0:g1].cpu().numpy(), ref[2]) and np.array_equal(q[3][g0:g1].cpu().numpy(), ref[3])
        want = oracle.op_dequantize(ref, xs.shape)
        assert np.array_equal(out[g0 * 256: g0 * 256 + xs.size].cpu().numpy(), want)
    # and the fast stream reaches the far end too: block numbers differ from their 32-bit truncation
    qf = ops.op_quantize(x, bits, 9, rng_stream="fast")
    g0 = (N - 4096) // 8 * 8
    tail = x[g0 * 256:].cpu().numpy()
    Nt = (tail.size + 255) // 256
    # the oracle numbers elements from 0, so feed it the absolute indices through an injected noise tensor
    idx = (np.arange(Nt * 256, dtype=np.uint64) + np.uint64(g0 * 256))
    # element E draws block (E/512)*16 + (E%128)/8, byte ((E/256)%2)*8 + E%8, c = (2h - 255)/512, negated in the
    # upper half of every 256; injected as the uniform c + 1/2 (for half data the reference form's two additions
    # are exact, so it gives the same codes)
    blk = (idx >> np.uint64(9)) * np.uint64(16) + ((idx & np.uint64(127)) >> np.uint64(3))
    uu = np.empty(Nt * 256, np.float32)
    cache = {}
    for b in np.unique(blk[:512]):                      # the blocks of the first two groups are enough to pin the indexing
        cache[int(b)] = oracle.philox4x32([0, 0, int(b) & 0xFFFFFFFF, int(b) >> 32], [9, 0], oracle.FAST_ROUNDS)
    sel = np.arange(512)
    for e in sel:
        E = int(idx[e])
        byte = ((E // 256) % 2) * 8 + E % 8
        h = (int(cache[int(blk[e])][byte // 4]) >> (8 * (byte % 4))) & 0xFF
        c = (2 * h - 255) / 512.0
        uu[e] = (-c if E % 256 >= 128 else c) + 0.5
    first = int(sel.max()) + 1                          # the selected elements are the first 512 of the tail
    assert first == 512
    ref = oracle.op_quantize(tail[:512], bits, oracle.NOISE_INJECT, 0, uu[:512])
    # 512 elements = 2 groups; compare their codes field by field
    pk = qf[0].cpu().numpy().view(np.uint8)
    for n_local in range(2):
        n = g0 + n_local
        row, ni = divmod(n, wpt)
        got = (pk[row * 256: row * 256 + 256] >> (ni * bits)) & (2 ** bits - 1)
        rrow, rni = divmod(n_local, wpt)
        want = (ref[0][rrow * 256: rrow * 256 + 256] >> (rni * bits)) & (2 ** bits - 1)
        assert np.array_equal(got, want)


def random_case(rng):
    dtype = DTYPES[rng.integers(2)]
    bits = BITS[rng.integers(4)]
    mode = list(MODES)[rng.integers(3)]
    numel = int(rng.choice([rng.integers(1, 600), rng.integers(600, 40000), 256 * rng.integers(1, 70)]))
    magnitude = 10.0 ** rng.uniform(-6, 4 if dtype == torch.float32 else 3)
    offset = rng.choice([0.0, 1.0, -3.0, 100.0]) * magnitude
    x = rng.standard_normal(numel) * magnitude + offset
    kind = rng.integers(6)
    if kind == 0:
        x = np.maximum(x - offset, 0.0)                    # post-ReLU: many exact zeros, -0.0 never
    elif kind == 1:
        x = np.round(x / magnitude) * magnitude            # few distinct values, many ties
    elif kind == 2:
        x[rng.random(numel) < 0.05] = np.nan               # scattered NaN
    elif kind == 3 and numel >= 512:
        g = rng.integers(numel // 256)
        x[g * 256:(g + 1) * 256] = np.nan                  # a whole group of NaN
        x[(g ^ 1) * 256 + 8 * 3:(g ^ 1) * 256 + 8 * 3 + 8] = np.nan   # and all of one lane's first chunk
    elif kind == 4:
        x = -np.abs(x)                                     # negative only, -0.0 possible after the cast
    return torch.from_numpy(x).to(dtype), bits, mode


def test_random_cases_against_the_oracle():
    rng = np.random.default_rng(2024)
    for case in range(150):
        x, bits, mode = random_case(rng)
        seed = int(rng.integers(0, 2 ** 31 - 1))
        try:
            q, ref = check_quantize(x, bits, mode, seed)
            out = ops.op_dequantize(q, x.shape).cpu().numpy()
            want = oracle.op_dequantize(ref, tuple(x.shape))
            np.testing.assert_array_equal(np.isnan(out), np.isnan(want))
            m = ~np.isnan(want)
            it = np.uint16 if out.dtype == np.float16 else np.uint32
            np.testing.assert_array_equal(out[m].view(it), want[m].view(it))
        except AssertionError as e:
            raise AssertionError("case %d: dtype %s bits %d stream %s numel %d seed %d: %s"
                                 % (case, x.dtype, bits, mode, x.numel(), seed, e))


@pytest.mark.parametrize("group", [64, 128, 512])
@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
def test_other_group_sizes_take_the_extension_sequence(group, dtype):
    """config.group_size other than 256 (gact/gact/conf.py:50 makes it a setting): zero-pad, minimax, pack,
    unpack, slice - the reference's own sequence on the general-shape kernels."""
    saved = config.group_size
    config.group_size = group
    try:
        g = torch.Generator().manual_seed(group)
        x_cpu = torch.randn((37, 101), generator=g).to(dtype)           # 3737 elements: a padded last group
        N = -(-x_cpu.numel() // group)
        flat = np.zeros(N * group, dtype=x_cpu.numpy().dtype)
        flat[: x_cpu.numel()] = x_cpu.numpy().ravel()
        groups = flat.reshape(N, group)
        mn, mx = oracle.minimax(groups)
        for bits in BITS:
            sc = oracle.scale(mn, mx, bits)
            for stream in ("deterministic", "fast", "reference"):
                want = oracle.pack(groups.reshape(N, 1, group), mn, sc, bits, MODES[stream], 9)
                q = ops.op_quantize(x_cpu.cuda(), bits, 9, rng_stream=stream)
                assert q[0].numel() == want.size + 1 and q[2].shape == (N, 1, 1) and q[3].shape == (N, 1, 1)
                np.testing.assert_array_equal(q[0].cpu().numpy().view(np.uint8)[: want.size], want)
                np.testing.assert_array_equal(q[3].cpu().numpy().ravel(), mn)
                out = ops.op_dequantize(q, x_cpu.shape)
                ref = oracle.unpack(want, bits, sc, mn, N, 1, group).ravel()[: x_cpu.numel()].reshape(x_cpu.shape)
                it = np.uint16 if ref.dtype == np.float16 else np.uint32
                np.testing.assert_array_equal(out.cpu().numpy().view(it), ref.view(it))
    finally:
        config.group_size = saved


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
def test_seed_offset_in_device_memory_equals_the_sum_on_the_host(dtype):
    x = torch.randn((50, 300), generator=torch.Generator().manual_seed(8)).to(dtype).cuda()
    offset = torch.tensor([12345], dtype=torch.int64, device="cuda")
    for bits in BITS:
        for stream in ("fast", "reference"):
            a = ops.op_quantize(x, bits, 7 + 12345, rng_stream=stream)
            b = ops.op_quantize(x, bits, 7, rng_stream=stream, seed_offset=offset)
            assert torch.equal(a[0][:-1], b[0][:-1]) and torch.equal(a[2], b[2]) and torch.equal(a[3], b[3])
    with pytest.raises(RuntimeError):
        ops.op_quantize(x, 4, 7, seed_offset=offset.int())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_stochastic_rounding_statistics_of_both_streams_on_the_gpu(dtype, bits):
    """What the task asks of the stochastic streams: mean error within 1e-3 of the range, and the variance of
    stochastic rounding, step^2 * f (1 - f), for the library's own stream exactly as for the reference's.  Per element
    over 2048 seeds' worth of draws (the same group at 2048 positions), and over a 4 M-element tensor."""
    qmax = 2 ** bits - 1
    # (a) one group repeated: every position draws its own noise, so a column is 2048 draws for one value
    torch.manual_seed(21)
    group = torch.rand(256)
    group[0], group[1] = 0.0, 1.0
    x = group.repeat(2048, 1).to(dtype).cuda()
    xf = x.float()
    stats = {}
    for stream in ("reference", "fast"):
        out = ops.op_dequantize(ops.op_quantize(x, bits, 77, rng_stream=stream), x.shape).float()
        err = out - xf
        stats[stream] = (err.mean(dim=0), err.var(dim=0))
        step = 1.0 / qmax
        # per value: the mean over 2048 draws within 4 sigma of zero (+ the half-precision grid), overall within 1e-3
        assert float(err.mean().abs()) < 1e-3, (stream, float(err.mean()))
        assert float(err.mean(dim=0).abs().max()) < 4 * 0.5 * step / 2048 ** 0.5 + 2e-3
    if dtype == torch.float32:
        f = (group.double() * qmax) % 1.0
        want = ((1.0 / qmax) ** 2 * f * (1 - f)).sum().item()
        for stream in stats:
            assert abs(stats[stream][1].double().sum().item() / want - 1) < 0.05, stream
    # half at 8 bit: the group's maximum can code 2^8, which the reference's uint8 accumulator wraps to 0 (an error of the
    # whole range, reproduced bit for bit and rare): keep that one column out of the comparison of the variances
    keep = torch.ones(256, dtype=torch.bool, device="cuda")
    if dtype == torch.float16 and bits == 8:
        keep[1] = False
    ratio = stats["fast"][1][keep].double().sum().item() / stats["reference"][1][keep].double().sum().item()
    assert abs(ratio - 1) < 0.05, ratio
    # (b) a whole tensor: mean error and mean squared error of the two streams agree
    y = torch.rand(16384, 256, generator=torch.Generator().manual_seed(5)).to(dtype).cuda()
    yf = y.float()
    mse = {}
    for stream in ("reference", "fast"):
        out = ops.op_dequantize(ops.op_quantize(y, bits, 3, rng_stream=stream), y.shape).float()
        e = out - yf
        assert float(e.mean().abs()) < 1e-3                      # range is 1
        # (half at 8 bit: without the rare wrapped maxima, whose count differs between any two streams)
        mse[stream] = float((e.double() ** 2)[e.abs() < 0.5].mean())
    assert abs(mse["fast"] / mse["reference"] - 1) < 0.02, mse
