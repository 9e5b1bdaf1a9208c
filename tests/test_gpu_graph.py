"""The kernels under HIP graph capture: the library allocates nothing and launches on the stream it is handed,
so a captured quantize -> dequantize pair must replay with the same bytes as eager launches on new data."""
import pytest
import torch

from gact import ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,bits,stream", [(torch.float32, 4, "fast"), (torch.float16, 2, "reference"),
                                               (torch.float32, 1, "deterministic"), (torch.float16, 8, "fast")])
def test_captured_pair_replays_like_eager(dtype, bits, stream):
    g = torch.Generator(device="cuda").manual_seed(bits)
    x = torch.randn(300, 1000, generator=g, device="cuda").to(dtype)      # 300000 elements: a padded last group
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                          # warm-up outside the capture
        ops.op_dequantize(ops.op_quantize(x, bits, 5, rng_stream=stream), x.shape)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        q = ops.op_quantize(x, bits, 5, rng_stream=stream)
        out = ops.op_dequantize(q, x.shape)
    for rep in range(4):
        x.copy_(torch.randn(300, 1000, generator=g, device="cuda").to(dtype) * (rep + 1))
        graph.replay()
        torch.cuda.synchronize()
        eq = ops.op_quantize(x, bits, 5, rng_stream=stream)
        eout = ops.op_dequantize(eq, x.shape)
        torch.cuda.synchronize()
        assert torch.equal(q[0][:-1], eq[0][:-1]), "replay %d: packed bytes" % rep
        assert torch.equal(q[2], eq[2]) and torch.equal(q[3], eq[3])
        assert torch.equal(out, eout), "replay %d: dequantized" % rep
