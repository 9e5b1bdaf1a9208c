"""The extension-style entry points (minimax, pack/unpack_single_precision, dropout masks,
calc_precision on the device, the batched launch) against the CPU oracle, through the C ABI."""
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

DTYPES = [torch.float32, torch.float16]


def bits_view(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("shape", [(1000, 256), (37, 64), (5, 1024), (129, 96), (3, 4096)])
def test_minimax(dtype, shape):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(shape, generator=g).to(dtype)
    mn, mx = ext_minimax.minimax(x.cuda())
    rmn, rmx = oracle.minimax(x.numpy())
    np.testing.assert_array_equal(mn.cpu().numpy(), rmn)
    np.testing.assert_array_equal(mx.cpu().numpy(), rmx)
    # the library routine the reference's own tests compare with (tests/test_act_quantized_ops.py:67-70)
    assert torch.equal(mn.cpu(), x.min(dim=1).values) and torch.equal(mx.cpu(), x.max(dim=1).values)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("shape", [(41, 64), (7, 256), (6, 1024), (11, 160)])
def test_minimax_on_a_base_address_that_is_not_16_byte_aligned(dtype, shape):
    # a contiguous view one element into a buffer: the element-by-element variant of the kernel
    N, D = shape
    g = torch.Generator().manual_seed(2)
    buf = torch.randn(N * D + 1, generator=g).to(dtype).cuda()
    x = buf[1:].view(N, D)
    assert x.is_contiguous() and x.data_ptr() % 16 != 0
    mn, mx = ext_minimax.minimax(x)
    assert torch.equal(mn, x.min(dim=1).values) and torch.equal(mx, x.max(dim=1).values)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("ngd", [(203, 1, 256), (21, 3, 64), (10, 2, 256), (9, 1, 128), (33, 1, 64), (5, 1, 1024),
                                 (12, 1, 96), (7, 1, 72), (6, 1, 100)])
@pytest.mark.parametrize("stream", ["deterministic", "reference", "fast"])
def test_pack_unpack_entry_points(dtype, bits, ngd, stream):
    N, G, D = ngd
    g = torch.Generator().manual_seed(bits)
    x = torch.randn((N, G, D), generator=g).to(dtype)
    mn_np, mx_np = oracle.minimax(x.reshape(N * G, D).numpy())
    mode = {"deterministic": 0, "reference": 2, "fast": 3}[stream]
    sc_np = oracle.scale(mn_np, mx_np, bits)
    want = oracle.pack(x.numpy(), mn_np, sc_np, bits, mode, 17)

    xd = x.cuda()
    mn = torch.from_numpy(mn_np).reshape(N, G, 1).cuda()
    mx = torch.from_numpy(mx_np).reshape(N, G, 1).cuda()
    packed, scale = ext_quantization.pack_single_precision(xd, mn, mx, bits, True, 17, rng_stream=stream)
    assert packed.dtype == torch.int8 and packed.numel() == want.size + 1
    assert scale.shape == (N, G, 1) and scale.dtype == dtype
    np.testing.assert_array_equal(bits_view(scale.cpu().numpy().reshape(-1)), bits_view(sc_np))
    np.testing.assert_array_equal(packed.cpu().numpy().view(np.uint8)[:want.size], want)

    out = ext_quantization.unpack_single_precision(packed, bits, scale, mn, N, G, D)
    assert out.shape == (N, G, D) and out.dtype == dtype
    ref = oracle.unpack(want, bits, sc_np, mn_np, N, G, D)
    np.testing.assert_array_equal(bits_view(out.cpu().numpy().reshape(-1)), bits_view(ref.reshape(-1)))


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f16"])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("ngd", [(67, 1, 256), (13, 2, 96)])
def test_pack_with_min_max_narrower_than_the_data(dtype, bits, ngd):
    """Caller-supplied min / max that do not bracket the data: elements below min give negative products
    (code 0), elements above max give codes beyond 2^bits - 1 whose shifted bits spill into the neighbouring
    fields or fall off the byte (quantization_cuda_kernel.cu:66-67).  All of it must match the restatement."""
    N, G, D = ngd
    g = torch.Generator().manual_seed(100 + bits)
    x = torch.randn((N, G, D), generator=g).to(dtype)
    mn_np = np.full(N * G, -0.5, dtype=x.numpy().dtype) + (np.arange(N * G) % 5).astype(x.numpy().dtype) * 0.1
    mx_np = mn_np + np.asarray(0.7, dtype=mn_np.dtype)
    sc_np = oracle.scale(mn_np, mx_np, bits)
    xd = x.cuda()
    mn = torch.from_numpy(mn_np).reshape(N, G, 1).cuda()
    mx = torch.from_numpy(mx_np).reshape(N, G, 1).cuda()
    for stream, mode in (("deterministic", 0), ("reference", 2), ("fast", 3)):
        want = oracle.pack(x.numpy(), mn_np, sc_np, bits, mode, 23)
        packed, scale = ext_quantization.pack_single_precision(xd, mn, mx, bits, True, 23, rng_stream=stream)
        np.testing.assert_array_equal(bits_view(scale.cpu().numpy().reshape(-1)), bits_view(sc_np))
        np.testing.assert_array_equal(packed.cpu().numpy().view(np.uint8)[:want.size], want)
        out = ext_quantization.unpack_single_precision(packed, bits, scale, mn, N, G, D)
        ref = oracle.unpack(want, bits, sc_np, mn_np, N, G, D)
        np.testing.assert_array_equal(bits_view(out.cpu().numpy().reshape(-1)), bits_view(ref.reshape(-1)))


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("ngd", [(67, 1, 256), (13, 2, 96), (21, 1, 128)])
def test_pack_codes_past_two_to_the_31_saturate_like_the_signed_conversion(bits, ngd):
    """float32 with caller-supplied min = max = 0: scale = (2^bits - 1) / 2e-6, so data up to 1e5 gives codes from 0
    to beyond 2^33.  The reference converts with __float2int_rn, which saturates at 0x7fffffff: from 2^31 on the
    low byte of a code is 0xff, not the low byte of the value (quantization_cuda_kernel.cu:66-67).  Every
    kernel behind gact_pack (the row kernel at D = 256, 8 columns per thread, one thread per byte)."""
    N, G, D = ngd
    g = torch.Generator().manual_seed(7 + bits)
    mag = torch.pow(10.0, torch.rand((N, G, D), generator=g) * 8.0 - 3.0)       # 1e-3 .. 1e5
    x = (mag * (torch.rand((N, G, D), generator=g) < 0.9)).to(torch.float32)   # some exact zeros, no negatives needed
    x[0, 0, :8] = torch.tensor([4294.9673, 4294.9674, 2147.4836, 2147.4837, 1073.7418, 1073.7419, 8589.9346, 0.0])
    mn_np = np.zeros(N * G, np.float32)
    sc_np = oracle.scale(mn_np, mn_np, bits)
    top = float(x.max()) * float(sc_np[0])
    assert top > 2.0 ** 33 and sc_np[0] == np.float32((2 ** bits - 1) / 2e-6)
    mn = torch.zeros((N, G, 1), device="cuda")
    for stream, mode in (("deterministic", 0), ("reference", 2), ("fast", 3)):
        want = oracle.pack(x.numpy(), mn_np, sc_np, bits, mode, 5)
        packed, scale = ext_quantization.pack_single_precision(x.cuda(), mn, mn.clone(), bits, True, 5, rng_stream=stream)
        np.testing.assert_array_equal(bits_view(scale.cpu().numpy().reshape(-1)), bits_view(sc_np))
        np.testing.assert_array_equal(packed.cpu().numpy().view(np.uint8)[:want.size], want, err_msg=stream)


def test_pack_uses_the_min_max_it_is_given():
    # the entry point's contract: codes are taken against the caller's min / max, whatever the data holds
    x = torch.rand((16, 1, 256)) * 0.5 + 0.25
    mn = torch.zeros((16, 1, 1))
    mx = torch.ones((16, 1, 1))
    packed, scale = ext_quantization.pack_single_precision(x.cuda(), mn.cuda(), mx.cuda(), 4, True, 0,
                                                           rng_stream="deterministic")
    sc = oracle.scale(mn.numpy().ravel(), mx.numpy().ravel(), 4)
    want = oracle.pack(x.numpy(), mn.numpy().ravel(), sc, 4, 0, 0)
    np.testing.assert_array_equal(packed.cpu().numpy().view(np.uint8)[:want.size], want)


@pytest.mark.parametrize("n", [1, 31, 32, 33, 511, 512, 513, 1024, 1000 * 1000, 512 * 7 + 100, 77 * 100])
def test_dropout_mask(n):
    g = torch.Generator().manual_seed(n)
    data = (torch.rand(n, generator=g) < 0.3).to(torch.uint8)
    q = ops.op_quantize_mask(data.cuda())
    assert q[0].dtype == torch.int32 and q[0].numel() == (n + 31) // 32
    np.testing.assert_array_equal(q[0].cpu().numpy(), oracle.mask_pack(data.numpy()))
    out = ops.op_dequantize_mask(q)
    assert out.dtype == torch.uint8 and torch.equal(out.cpu(), data)


def test_dropout_mask_views_that_start_at_an_odd_offset():
    # a contiguous slice or chunk of a mask starts where it starts: the reference's kernel takes any alignment
    g = torch.Generator().manual_seed(9)
    whole = (torch.rand(5000, generator=g) < 0.4).to(torch.uint8).cuda()
    for view in (whole[1:], whole[3:4100], whole.view(50, 100)[7:], whole.view(torch.bool)[5:]):
        assert view.is_contiguous() and view.data_ptr() % 16 != 0
        data = view.view(torch.uint8) if view.dtype == torch.bool else view
        q = ops.op_quantize_mask(data)
        np.testing.assert_array_equal(q[0].cpu().numpy(), oracle.mask_pack(data.cpu().numpy().reshape(-1)))
        assert torch.equal(ops.op_dequantize_mask(q), data)


def test_dropout_mask_every_count_of_blocks_a_wave_can_end_on():
    # a wave takes 8 blocks of 512 elements: every residue of the block count, with and without a partial block
    g = torch.Generator().manual_seed(5)
    for blocks in range(0, 18):
        for rest in (0, 1, 33, 511):
            n = 512 * blocks + rest
            if n == 0:
                continue
            data = (torch.rand(n, generator=g) < 0.5).to(torch.uint8)
            q = ops.op_quantize_mask(data.cuda())
            np.testing.assert_array_equal(q[0].cpu().numpy(), oracle.mask_pack(data.numpy()), err_msg="n=%d" % n)
            assert torch.equal(ops.op_dequantize_mask(q).cpu(), data), n


def test_dropout_mask_one_hot_identity():
    # tests/test_act_quantized_ops.py:16-21 of the reference
    data = torch.nn.functional.one_hot(torch.arange(1000), 1000).to(torch.uint8).cuda()
    out = ops.op_dequantize_mask(ops.op_quantize_mask(data))
    assert out.shape == data.shape and torch.equal(out, data)


def _swin_like(rng, L):
    shapes = [(8, 3136, 96), (8, 784, 192), (8, 196, 384), (8, 49, 768)]
    return [shapes[rng.integers(0, 4)] for _ in range(L)]


@pytest.mark.parametrize("L,init,avg", [(120, 8, 2.0), (120, 32, 2.0), (7, 8, 3.0), (64, 8, 1.0), (65, 8, 4.0),
                                        (300, 32, 2.5)])
def test_calc_precision_device_matches_host_and_oracle(L, init, avg):
    rng = np.random.default_rng(L)
    C = np.exp(rng.normal(0, 2, L)).astype(np.float32)
    w = np.array([int(np.prod(s)) for s in _swin_like(rng, L)], dtype=np.int64)
    target = avg * float(w.sum())
    want = oracle.calc_precision(np.full(L, init, np.int32), C, w, target)
    host = ext_calc_precision.calc_precision(torch.full((L,), init, dtype=torch.int32), torch.from_numpy(C),
                                             torch.from_numpy(w), target)
    np.testing.assert_array_equal(host.numpy(), want)
    status = torch.full((1,), 99, dtype=torch.int32, device="cuda")
    dev = ext_calc_precision.calc_precision_device(torch.full((L,), init, dtype=torch.int32, device="cuda"),
                                                   torch.from_numpy(C).cuda(), torch.from_numpy(w).cuda(), target,
                                                   status)
    np.testing.assert_array_equal(dev.cpu().numpy(), want)
    assert status.item() == 0


def test_calc_precision_device_adversarial_orders():
    # ties, near ties, zero and infinite sensitivities (the last two leave the sorting path), long tables
    rng = np.random.default_rng(77)
    cases = []
    for t in range(40):
        L = int(rng.integers(1, 300))
        base = np.float32(np.exp(rng.normal(0, 1)))
        C = (np.full(L, base, np.float32).view(np.int32) + rng.integers(-2, 3, L).astype(np.int32)).view(np.float32)
        w = np.full(L, int(rng.choice([256, 4096, 65536])), np.int64)
        cases.append((C, w, int(rng.choice([8, 32])), float(rng.choice([1.0, 1.5, 2.0, 3.0, 5.0]))))
    cases.append((np.zeros(50, np.float32), np.full(50, 1024, np.int64), 8, 2.0))
    cases.append((np.array([0.0, 1.0, 0.0, 2.0, 0.0], np.float32), np.full(5, 512, np.int64), 32, 2.0))
    cases.append((np.array([np.inf, 1.0, np.inf, 2.0], np.float32), np.full(4, 512, np.int64), 8, 2.0))
    # long tables: the sorting path up to its limit of 4096 tensors (1024 threads, 128 KB of LDS), and the
    # sequential path at a length only it is asked to handle (an infinite sensitivity leaves the sorting path)
    for big, init, avg in ((1500, 8, 2.0), (1024, 32, 3.0), (4096, 8, 1.5), (3000, 32, 2.5)):
        cases.append((np.exp(rng.normal(0, 2, big)).astype(np.float32), (rng.integers(1, 50, big) * 256).astype(np.int64), init, avg))
    C_inf = np.exp(rng.normal(0, 2, 1500)).astype(np.float32)
    C_inf[700] = np.inf
    cases.append((C_inf, (rng.integers(1, 50, 1500) * 256).astype(np.int64), 8, 2.0))
    ties = np.full(2500, 1.0, np.float32)            # every key equal: the order is decided by the index alone
    cases.append((ties, np.full(2500, 4096, np.int64), 8, 3.0))
    for C, w, init, avg in cases:
        L = C.size
        target = avg * float(w.sum())
        want = oracle.calc_precision(np.full(L, init, np.int32), C, w, target)
        status = torch.full((1,), 99, dtype=torch.int32, device="cuda")
        dev = ext_calc_precision.calc_precision_device(torch.full((L,), init, dtype=torch.int32, device="cuda"),
                                                       torch.from_numpy(C).cuda(), torch.from_numpy(w).cuda(), target,
                                                       status)
        np.testing.assert_array_equal(dev.cpu().numpy(), want)
        assert status.item() == 0


def test_calc_precision_device_rejects_unknown_widths():
    b = torch.tensor([8, 3, 8], dtype=torch.int32, device="cuda")
    status = torch.zeros((1,), dtype=torch.int32, device="cuda")
    ext_calc_precision.calc_precision_device(b, torch.ones(3, device="cuda"),
                                             torch.full((3,), 256, dtype=torch.int64, device="cuda"), 100.0, status)
    assert status.item() == -1 and b.cpu().tolist() == [8, 3, 8]


def test_calc_precision_device_reports_unreachable_budget():
    L = 5
    b = torch.full((L,), 8, dtype=torch.int32, device="cuda")
    status = torch.zeros((1,), dtype=torch.int32, device="cuda")
    ext_calc_precision.calc_precision_device(b, torch.ones(L, device="cuda"),
                                             torch.full((L,), 256, dtype=torch.int64, device="cuda"), 100.0, status)
    assert status.item() == -5 and b.cpu().tolist() == [1] * L


@pytest.mark.parametrize("stream,mix", [("deterministic", "both"), ("fast", "both"), ("reference", "both"),
                                        ("fast", "float"), ("fast", "half")])
def test_batched_equals_tensor_by_tensor(stream, mix):
    rng = np.random.default_rng(3)
    L = 24
    shapes = _swin_like(rng, L) + [(100, 77), (3, 5)]
    # element types of the table: mixed, or one type only (then only that type's kernels are launched)
    dtypes = [{"float": torch.float32, "half": torch.float16}.get(mix, torch.float16 if i % 3 else torch.float32)
              for i in range(len(shapes))]
    L = len(shapes)
    g = torch.Generator().manual_seed(0)
    tensors = [torch.randn(s, generator=g).to(d).cuda() for s, d in zip(shapes, dtypes)]
    C = np.exp(rng.normal(0, 2, L)).astype(np.float32)
    w = np.array([t.numel() for t in tensors], dtype=np.int64)
    target = 2.0 * float(w.sum())
    bits = ext_calc_precision.calc_precision_device(torch.full((L,), 8, dtype=torch.int32, device="cuda"),
                                                    torch.from_numpy(C).cuda(), torch.from_numpy(w).cuda(), target)
    seeds = [i + 5 for i in range(L)]
    bq = BatchedQuantizer([t.numel() for t in tensors], dtypes, "cuda")
    assert bq.dtype_mask == {"both": 3, "float": 1, "half": 2}[mix]
    q = bq.quantize(tensors, bits, seeds, arena_bytes=bq.arena_bytes_for_budget(target), rng_stream=stream)
    ok, need = q.ok()
    assert ok and need <= q.packed.numel()
    outs = bq.dequantize(q)
    torch.cuda.synchronize()
    host_bits = bits.cpu().tolist()
    assert set(host_bits) <= {1, 2, 4, 8} and len(set(host_bits)) > 1
    for i, t in enumerate(tensors):
        single = ops.op_quantize(t, host_bits[i], seeds[i], rng_stream=stream)
        pk, b, sc, mn = q.per_tensor(i)
        assert b == host_bits[i]
        n = pk.numel()
        assert torch.equal(pk, single[0][:n]), "packed bytes of tensor %d differ" % i
        assert torch.equal(sc.view(torch.int16 if t.dtype == torch.float16 else torch.int32),
                           single[2].view(torch.int16 if t.dtype == torch.float16 else torch.int32))
        assert torch.equal(mn, single[3])
        d = ops.op_dequantize(single, t.shape)
        assert torch.equal(outs[i], d), "dequantized tensor %d differs" % i


def test_batched_refuses_an_arena_that_is_too_small():
    tensors = [torch.randn(4096, 256, device="cuda") for _ in range(3)]
    bq = BatchedQuantizer([t.numel() for t in tensors], [torch.float32] * 3, "cuda")
    bits = torch.full((3,), 8, dtype=torch.int32, device="cuda")
    q = bq.quantize(tensors, bits, [0, 1, 2], arena_bytes=1 << 20)
    ok, need = q.ok()
    assert not ok and need == 3 * 4096 * 256
    # a void launch is an error as soon as its result is used
    with pytest.raises(RuntimeError, match="void"):
        q.per_tensor(0)
    with pytest.raises(RuntimeError, match="void"):
        bq.dequantize(q)


def test_batched_refuses_a_width_it_cannot_pack():
    # calc_precision started from 32 bits with a loose budget leaves tensors at 32: not a packable width
    tensors = [torch.randn(512, 256, device="cuda") for _ in range(3)]
    bq = BatchedQuantizer([t.numel() for t in tensors], [torch.float32] * 3, "cuda")
    bits = torch.tensor([4, 32, 2], dtype=torch.int32, device="cuda")
    q = bq.quantize(tensors, bits, [0, 1, 2])
    assert not q.ok()[0]
    with pytest.raises(RuntimeError, match="void"):
        bq.dequantize(q)


def test_random_cases_on_general_shapes_masks_and_minimax():
    """600 seeded random cases on what the fixed parametrisations above only sample: (N, G, D) of any kind
    through pack / unpack, masks of any length, minimax on any row length and alignment."""
    rng = np.random.default_rng(2024)
    modes = {"deterministic": 0, "reference": 2, "fast": 3}
    for case in range(600):
        kind = case % 3
        dtype = DTYPES[int(rng.integers(0, 2))]
        if kind == 0:
            N, G = int(rng.integers(1, 60)), int(rng.integers(1, 4))
            D = int(rng.choice([8, 24, 40, 64, 100, 128, 256, 264, 512]))
            bits, stream, seed = int(rng.choice([1, 2, 4, 8])), str(rng.choice(list(modes))), int(rng.integers(0, 2 ** 31 - 1))
            x = torch.randn((N, G, D), generator=torch.Generator().manual_seed(case)).to(dtype)
            rows = x.reshape(N * G, D)
            mn_np, mx_np = rows.min(1).values.numpy(), rows.max(1).values.numpy()
            sc_np = oracle.scale(mn_np, mx_np, bits)
            want = oracle.pack(x.numpy(), mn_np, sc_np, bits, modes[stream], seed)
            mn = torch.from_numpy(mn_np).reshape(N, G, 1).cuda()
            mx = torch.from_numpy(mx_np).reshape(N, G, 1).cuda()
            packed, scale = ext_quantization.pack_single_precision(x.cuda(), mn, mx, bits, True, seed, rng_stream=stream)
            tag = "case %d: %s N=%d G=%d D=%d bits=%d %s" % (case, dtype, N, G, D, bits, stream)
            np.testing.assert_array_equal(packed.cpu().numpy().view(np.uint8)[:want.size], want, err_msg=tag)
            out = ext_quantization.unpack_single_precision(packed, bits, scale, mn, N, G, D)
            ref = oracle.unpack(want, bits, sc_np, mn_np, N, G, D)
            np.testing.assert_array_equal(bits_view(out.cpu().numpy().reshape(-1)), bits_view(ref.reshape(-1)), err_msg=tag)
        elif kind == 1:
            n = int(rng.integers(1, 70000))
            data = (torch.rand(n, generator=torch.Generator().manual_seed(case)) < float(rng.random())).to(torch.uint8)
            q = ops.op_quantize_mask(data.cuda())
            np.testing.assert_array_equal(q[0].cpu().numpy(), oracle.mask_pack(data.numpy()), err_msg="mask n=%d" % n)
            assert torch.equal(ops.op_dequantize_mask(q).cpu(), data), n
        else:
            N, D, off = int(rng.integers(1, 300)), 32 * int(rng.integers(2, 80)), int(rng.integers(0, 2))
            buf = torch.randn(N * D + off, generator=torch.Generator().manual_seed(case)).to(dtype).cuda()
            x = buf[off:].view(N, D)
            mn, mx = ext_minimax.minimax(x)
            assert torch.equal(mn, x.min(1).values) and torch.equal(mx, x.max(1).values), (N, D, off, dtype)


def test_occupancy_caps_are_what_the_launches_get():
    """On large tensors some kernels cap their occupancy by asking for dynamic LDS they never touch.  What the
    runtime grants for exactly the kernel, workgroup size and LDS request of a launch (gact_launch_geometry:
    hipOccupancyMaxActiveBlocksPerMultiprocessor) must be the cap the geometry tables mean - and no cap where
    none is meant."""
    import ctypes

    lib = _abi.lib()

    def geometry(kind, dtype, bits, N):
        t, l, w = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
        _abi.check(lib.gact_launch_geometry(kind, dtype, bits, N, ctypes.addressof(t), ctypes.addressof(l), ctypes.addressof(w)))
        return t.value, l.value, w.value

    Q, DQ = 0, 1
    big, small = 1 << 19, 1 << 14
    # dequantize, float, every width: 3 workgroups of 256 threads per compute unit from 2^17 groups on
    for bits in (1, 2, 4, 8):
        threads, lds, per_cu = geometry(DQ, _abi.F32, bits, big)
        assert (threads, per_cu) == (256, 3) and lds > 0, (bits, threads, lds, per_cu)
        threads, lds, per_cu = geometry(DQ, _abi.F32, bits, small)
        assert threads == 256 and lds == 0 and per_cu >= 6, (bits, per_cu)
    # dequantize, half: capped at 8 bit (4 workgroups) and, from 2^18 groups on, at 1 bit (6 workgroups)
    assert geometry(DQ, _abi.F16, 8, big)[1:] == (40000, 4)
    assert geometry(DQ, _abi.F16, 1, big)[1:] == (26000, 6) and geometry(DQ, _abi.BF16, 1, big)[1:] == (26000, 6)
    assert geometry(DQ, _abi.F16, 1, 1 << 17)[1] == 0 and geometry(DQ, _abi.F16, 1, 1 << 17)[2] >= 7
    for bits in (2, 4):
        assert geometry(DQ, _abi.F16, bits, big)[1] == 0 and geometry(DQ, _abi.F16, bits, big)[2] >= 6
    # quantize, float: 16 one-wave workgroups per compute unit at 4 bit, 8 at 2 bit, on large tensors only
    assert geometry(Q, _abi.F32, 4, big) == (64, 10000, 16)
    assert geometry(Q, _abi.F32, 2, big) == (64, 20000, 8)
    assert geometry(Q, _abi.F32, 4, small)[1] == 0 and geometry(Q, _abi.F32, 2, small)[1] == 0
    for bits in (1, 8):
        assert geometry(Q, _abi.F32, bits, big)[1] == 0
    for dtype in (_abi.F16, _abi.BF16):
        for bits in (1, 2, 4, 8):
            assert geometry(Q, dtype, bits, big)[1] == 0
    # uncapped one-wave workgroups: the registers decide (float 1 bit holds 8 groups per lane: two waves per SIMD)
    assert geometry(Q, _abi.F32, 1, big)[0] == 64 and geometry(Q, _abi.F32, 1, big)[2] >= 8
    # small 1-bit tensors take the wave-per-super-group kernel, four waves to a workgroup
    assert geometry(Q, _abi.F32, 1, small)[0] == 256 and geometry(Q, _abi.F16, 1, small)[0] == 256
    # arguments
    assert lib.gact_launch_geometry(2, _abi.F32, 4, 100, None, None, None) == -1
    assert lib.gact_launch_geometry(0, _abi.F32, 3, 100, None, None, None) == -1
    assert lib.gact_launch_geometry(0, 7, 4, 100, None, None, None) == -1
    assert lib.gact_launch_geometry(1, _abi.F16, 4, 0, None, None, None) == -1
    assert lib.gact_launch_geometry(1, _abi.F16, 4, 100, None, None, None) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_fused_quantize_also_writes_the_maxima_when_asked(dtype, bits):
    """gact_quantize's optional `mx` output: the per-group maxima of minimax (minimax_cuda_kernel.cu:23-67) from the
    same pass, for small tensors (at 1 bit: the wave-per-super-group kernel), large ones, and ragged ends."""
    lib = _abi.lib()
    torch.manual_seed(3)
    for numel in (256 * 37 + 100, 256 * 8, 256 * 70001 + 17):
        x = (torch.randn(numel) * 2).to(dtype)
        N = (numel + 255) // 256
        xd = x.cuda()
        packed = torch.empty((lib.gact_packed_bytes(bits, N, 1, 256) + 1,), dtype=torch.int8, device="cuda")
        sc, mn, mx = (torch.empty((N,), dtype=dtype, device="cuda") for _ in range(3))
        _abi.check(lib.gact_quantize(xd.data_ptr(), _abi.dtype_code(dtype), numel, bits, _abi.NOISE_FAST, 5, None,
                                     packed.data_ptr(), sc.data_ptr(), mn.data_ptr(), mx.data_ptr(),
                                     torch.cuda.current_stream().cuda_stream))
        padded = torch.zeros(N * 256, dtype=dtype)
        padded[:numel] = x
        rmn, rmx = oracle.minimax(padded.reshape(N, 256).numpy())
        np.testing.assert_array_equal(mn.cpu().numpy(), rmn)
        np.testing.assert_array_equal(mx.cpu().numpy(), rmx)
        ref = oracle.op_quantize(x.numpy(), bits, oracle.NOISE_FAST, 5)
        np.testing.assert_array_equal(packed.cpu().numpy().view(np.uint8)[:ref[0].size], ref[0])
        np.testing.assert_array_equal(sc.cpu().numpy(), ref[2].reshape(-1))
