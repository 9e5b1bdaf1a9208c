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


@pytest.mark.parametrize("device_seed", [False, True], ids=["host-seed", "device-seed"])
def test_whole_training_step_under_the_hooks_replays_as_a_graph(device_seed):
    """The hooks only allocate and launch (no synchronisation for float tensors), so a forward + backward pass
    under them can be captured whole; replays on new data must give the gradients of the eager hooked step on
    that data (the seeds are those of the captured iteration, which the eager step is given as well).  Several
    replays with eager work and synchronisations in between, each one checked."""
    import gact
    from gact.conf import config
    from gact.controller import Controller

    saved = dict(vars(config))
    try:
        torch.manual_seed(0)
        net = torch.nn.Sequential(torch.nn.Linear(512, 1024), torch.nn.GELU(), torch.nn.Linear(1024, 1024),
                                  torch.nn.ReLU(), torch.nn.Linear(1024, 10)).cuda()
        x = torch.randn(256, 512, device="cuda")
        y = torch.randint(0, 10, (256,), device="cuda")
        gact.set_optimization_level("L1")
        config.device_seed = device_seed     # the iteration count of the seeds read from device memory by the kernels
        ctl = Controller(net)
        ctl.install_hook()
        try:
            def step():
                net.zero_grad(set_to_none=False)
                loss = torch.nn.functional.cross_entropy(net(x), y)
                loss.backward()
                ctl.quantizer.iterate()                     # tensor ids restart; the seed offset stays
                return loss

            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    step()
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                captured_loss = step()
            assert len(ctl.quantizer.bits) >= 3
            seen = []
            for trial in range(4):
                x.copy_(torch.randn(256, 512, generator=torch.Generator().manual_seed(trial % 2)).cuda())
                if device_seed:
                    ctl.quantizer.seed_iter = 10 + trial      # what Controller.iterate does once per iteration
                graph.replay()
                torch.cuda.synchronize()
                got = torch.cat([p.grad.ravel() for p in net.parameters()]).clone()
                got_loss = captured_loss.item()
                eager_loss = step().item()
                torch.cuda.synchronize()
                want = torch.cat([p.grad.ravel() for p in net.parameters()])
                # the same kernels on the same data: equal up to what the GEMM library may reorder between launches
                assert abs(got_loss - eager_loss) <= 1e-6 * abs(eager_loss), trial
                assert (got - want).norm().item() <= 1e-5 * want.norm().item(), trial
                seen.append(got)
            # trials 0 / 2 and 1 / 3 saw the same data: with the seed in device memory the replays drew fresh
            # noise, with the seed frozen at capture they repeat themselves
            assert torch.equal(seen[0], seen[2]) != device_seed and torch.equal(seen[1], seen[3]) != device_seed
        finally:
            ctl.uninstall_hook()
    finally:
        vars(config).update(saved)
