#!/usr/bin/env python3
"""Throughput of the saved-activation compression path on one MI355X.

One step = one fused quantize (min/max + scale + rounding + pack) followed by one dequantize (unpack +
affine) of one synthetic activation tensor, through the C ABI, with the input already resident in HBM.
The headline workload is the one the metric string names ("2-bit group=256"): BASELINE.json's first
configuration, a float32 [4096,1024] tensor ~N(0,1) at 2 bit with deterministic rounding ("config1").
Every other BASELINE configuration is measured in the same run and reported under "configs".
Bytes are the algorithmic input + output bytes: numel*sizeof(T) + packed bytes + 2*N*sizeof(T) per direction.

Timing.  The K steps of a block are recorded once into a HIP graph (the launches go through the C ABI on
the capturing stream) and the graph is replayed between two events on that stream; blocks are repeated
until at least one second has been measured (the rule of the reference's tests/timeit_v2.py:246-257), the
mean over all timed steps is reported.  Every workload is given several buffer sets used in rotation (4 GB
between two uses of a buffer, whatever K is), so that every step streams from and to HBM.  The duration of
each kernel comes from the same construction with K launches of that kernel alone; `roofline` is the
slower of the two kernels of the headline workload.  `cpu_baseline` is the C restatement of the reference
arithmetic (oracle/) with OpenMP on the host cores.

Every workload also carries `probe`: compute-free kernels (gact-icml_amd/csrc/stream_probe.hip) that move the bytes of
its quantize and of its dequantize kernel - the same bytes per wave in, the same out, nothing computed - timed the same
way in the same run, and the kernel's duration as a multiple of the probe's.

Beside the workloads the line carries what plain streams reach in the same run: `ceilings` (device copy, fill,
pure read, torch's element-wise kernel at the 8:1 and 1:8 read:write mixes, and the duration of a one-group
launch, on config2's tensor), `ceilings_headline` (the same on config1's tensor) and `ceilings_by_size` (fill and
pure read at the sizes of the mid-sized workloads); `configs["config1-cached"]` is the headline tensor with one
buffer set.  `entry_points` times the entry points no workload goes through (gact_pack with the caller's min / max,
gact_unpack, the dropout-mask bit packing) on config2's tensor.

Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "gact-icml_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
MIN_SECONDS = 1.0      # every timed loop runs at least this long

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known size
# in the same runs (profiles/<workload>_*.txt name the runs and the factors); absent = no counter run
TRAFFIC_BYTES = {
    ("config1", "quantize"): 18.06e6,    # 16.84 MB read + 1.22 MB written; algorithmic 17.96 MB
    ("config1", "dequantize"): 18.02e6,  # 1.25 MB read + 16.78 MB written; algorithmic 17.96 MB
    ("config2", "quantize"): 468.27e6,    # 411.06 MB read + 57.21 MB written; algorithmic 465.63 MB
    ("config2", "dequantize"): 465.68e6,  # 54.64 MB read + 411.04 MB written; algorithmic 465.63 MB
    ("config3-hidden", "quantize"): 50.63e6,    # 33.59 MB read + 17.04 MB written; algorithmic 50.59 MB
    ("config3-hidden", "dequantize"): 50.69e6,  # 17.13 MB read + 33.55 MB written; algorithmic 50.59 MB
    ("config3-gelu", "quantize"): 168.87e6,    # 134.27 MB read + 34.60 MB written; algorithmic 168.82 MB
    ("config3-gelu", "dequantize"): 168.88e6,  # 34.66 MB read + 134.22 MB written; algorithmic 168.82 MB
    ("config3-probs", "quantize"): 304.20e6,    # 268.55 MB read + 35.65 MB written; algorithmic 304.09 MB
    ("config3-probs", "dequantize"): 304.15e6,  # 35.71 MB read + 268.44 MB written; algorithmic 304.09 MB
    ("config2-refstream", "quantize"): 467.41e6,    # 411.15 MB read + 56.26 MB written; algorithmic 465.63 MB
    ("config2-refstream", "dequantize"): 465.68e6,  # 54.64 MB read + 411.04 MB written; algorithmic 465.63 MB
    ("config3-probs-refstream", "quantize"): 304.29e6,    # 268.64 MB read + 35.65 MB written; algorithmic 304.09 MB
    ("config3-probs-refstream", "dequantize"): 304.15e6,  # 35.71 MB read + 268.44 MB written; algorithmic 304.09 MB
    ("config4", "quantize"): 180.23e6,    # 173.46 MB read + 6.77 MB written; algorithmic 180.18 MB
    ("config4", "dequantize"): 180.33e6,  # 6.84 MB read + 173.49 MB written; algorithmic 180.18 MB
    ("config5", "quantize"): 4143.29e6,    # 3661.90 MB read + 481.39 MB written; algorithmic 4142.23 MB
    ("config5", "dequantize"): 4144.33e6,  # 483.49 MB read + 3660.84 MB written; algorithmic 4142.23 MB
}

BASELINE_METRIC = "quantize+dequantize GB/s and % of HBM peak, 1×MI355X, 2-bit group=256"

# A workload is timed over as many buffer sets, used in rotation, as it takes to touch this many bytes before a
# buffer comes round again.  The GPU's last-level cache holds 256 MB and does not evict in strict LRU order: with
# 0.8 GB between reuses a 411 MB tensor still read 3-4 % faster (and a 173 MB one was written 8 % faster) than
# from HBM; the figures stop moving at 3 GB.
ROTATE_BYTES = 4 * 1000 * 1000 * 1000

WORKLOADS = {
    # name: (shape, dtype, bits, rng_stream, data kind, description)
    "config1": ((4096, 1024), "float32", 2, "deterministic", "randn",
                "fp32 [4096,1024] ~N(0,1) seed 0, 2 bit, deterministic rounding"),
    "config2": ((128, 256, 56, 56), "float32", 4, "fast", "relu",
                "ResNet-50 conv activation fp32 [128,256,56,56] post-ReLU, 4 bit, stochastic rounding, Philox seed 42"),
    "config2-2bit": ((128, 256, 56, 56), "float32", 2, "fast", "relu", "config2's tensor at 2 bit"),
    "config2-refstream": ((128, 256, 56, 56), "float32", 4, "reference", "relu",
                          "config2 with the reference's one-Philox-state-per-byte noise stream"),
    "config3-hidden": ((16384, 1024), "float16", 8, "fast", "randn", "BERT-large hidden states fp16, 8 bit"),
    "config3-gelu": ((16384, 4096), "float16", 4, "fast", "randn", "BERT-large GELU inputs fp16, 4 bit"),
    "config3-probs": ((32, 16, 512, 512), "float16", 2, "fast", "softmax", "BERT-large attention probs fp16, 2 bit"),
    "config3-probs-refstream": ((32, 16, 512, 512), "float16", 2, "reference", "softmax",
                                "config3's attention probs with the reference's one-Philox-state-per-byte noise stream"),
    "config4": ((169343, 256), "float32", 1, "fast", "relu60", "GCN node features fp32 [169343,256], ~60% zeros, 1 bit"),
    # the reference's own micro-benchmark (tests/test_speed.py:6-15): torch.rand [256,256,14,14] at 2 bit
    "reference-test-speed": ((256, 256, 14, 14), "float32", 2, "fast", "rand",
                             "the reference's tests/test_speed.py tensor: fp32 [256,256,14,14] ~U(0,1), 2 bit, stochastic rounding"),
    # not a BASELINE workload: the GELU-input tensor of config 3 as mixed-precision training on this GPU holds it
    "bf16-gelu": ((16384, 4096), "bfloat16", 4, "fast", "randn", "GELU inputs in bfloat16, 4 bit (float scale, bfloat16 min)"),
}
# what a default run measures besides the headline workload (config5 is the batched one)
BASELINE_SET = ["config1", "config2", "config2-refstream", "config2-2bit", "config3-hidden", "config3-gelu", "config3-probs",
                "config3-probs-refstream", "config4", "reference-test-speed"]


def make_input(torch, shape, dtype, kind, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32)
    if kind == "rand":
        x = torch.rand(shape, generator=g, device="cuda", dtype=torch.float32)
    elif kind == "relu":
        x = torch.relu(x)
    elif kind == "relu60":
        x = torch.relu(x - 0.2533)  # P(N(0,1) < 0.2533) = 0.6
    elif kind == "softmax":
        x = torch.softmax(x, dim=-1)
    return x.to(getattr(torch, dtype)).contiguous()


def algorithmic_bytes(numel, esize, bits, scale_esize=None):
    N = (numel + 255) // 256
    wpt = 8 // bits
    n_round = (N + wpt - 1) // wpt * wpt
    return numel * esize + n_round * 32 * bits + N * (esize + (scale_esize or esize))


_PROBE = None


def probe_lib():
    """The compute-free traffic probes (libgact_probe.so, built next to the library)."""
    global _PROBE
    if _PROBE is None:
        import ctypes

        from gact.cpp_extension import _abi
        lib = ctypes.CDLL(os.path.join(os.path.dirname(_abi.LIB_PATH), "libgact_probe.so"))
        vp, i32, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
        for name in ("gact_probe_quantize_like", "gact_probe_dequantize_like"):
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = i32, [vp, vp, i64, i32, i32, vp]
        _PROBE = lib
    return _PROBE


class Timer:
    """Mean duration of fn(k) over blocks of `steps` calls, at least MIN_SECONDS of them.  `period` is the
    number of distinct k the workload tells apart (its buffer sets): when it exceeds `steps`, consecutive blocks
    continue the count, so that all of them come round whatever `steps` is."""

    def __init__(self, torch, steps, warmup, min_seconds, graph=True):
        self.torch, self.steps, self.warmup, self.min_seconds, self.graph = torch, steps, warmup, min_seconds, graph

    def __call__(self, fn, period=1):
        torch = self.torch
        for k in range(self.warmup):
            fn(k)
        torch.cuda.synchronize()
        n_blocks = max(1, min(64, -(-period // self.steps)))
        blocks = None
        if self.graph:
            # every block's launches, recorded once on a side stream (capture cannot run on the null stream)
            blocks = []
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for b in range(n_blocks):
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g, stream=side):
                        for k in range(self.steps):
                            fn(b * self.steps + k)
                    blocks.append(g)
            torch.cuda.current_stream().wait_stream(side)
            for g in blocks:    # untimed: the first replay uploads the graph
                g.replay()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        total_ms, calls, b = 0.0, 0, 0
        t_begin = time.perf_counter()
        while True:
            e0.record()
            if blocks is not None:
                blocks[b].replay()
            else:
                for k in range(self.steps):
                    fn(b * self.steps + k)
            e1.record()
            e1.synchronize()
            total_ms += e0.elapsed_time(e1)
            calls += self.steps
            b = (b + 1) % n_blocks
            if time.perf_counter() - t_begin >= self.min_seconds:
                break
        return total_ms / calls, calls


def run_workload(torch, name, timer, seed=42, keep_input=False, rotate=True):
    """One step = quantize then dequantize of the workload's tensor.  rotate = False: one buffer set whatever
    its size (a small tensor then stays in the last-level cache between steps)."""
    from gact.cpp_extension import _abi

    shape, dtype, bits, stream, kind, desc = WORKLOADS[name]
    lib = _abi.lib()
    x = make_input(torch, shape, dtype, kind)
    numel = x.numel()
    N = (numel + 255) // 256
    esize = x.element_size()
    packed_len = lib.gact_packed_bytes(bits, N, 1, 256) + 1
    working_set = 2 * numel * esize + packed_len
    sets = max(1, -(-ROTATE_BYTES // working_set)) if rotate else 1
    scale_dtype = torch.float32 if x.dtype == torch.bfloat16 else x.dtype      # bfloat16 tensors keep a float scale
    bufs = []
    for r in range(sets):
        bufs.append((x if r == 0 else x.clone(),
                     torch.empty((packed_len,), dtype=torch.int8, device="cuda"),
                     torch.empty((N,), dtype=scale_dtype, device="cuda"), torch.empty((N,), dtype=x.dtype, device="cuda"),
                     torch.empty_like(x)))
    dt = _abi.dtype_code(x.dtype)
    mode = _abi.NOISE_MODES[stream]

    def quantize(k):
        xi, packed, scale, mn, _ = bufs[k % sets]
        _abi.check(lib.gact_quantize(xi.data_ptr(), dt, numel, bits, mode, seed, None, packed.data_ptr(),
                                     scale.data_ptr(), mn.data_ptr(), None, torch.cuda.current_stream().cuda_stream))

    def dequantize(k):
        _, packed, scale, mn, out = bufs[k % sets]
        _abi.check(lib.gact_dequantize(packed.data_ptr(), bits, scale.data_ptr(), mn.data_ptr(), dt, numel,
                                       out.data_ptr(), torch.cuda.current_stream().cuda_stream))

    def step(k):
        quantize(k)
        dequantize(k)

    for k in range(sets):   # every set holds valid codes before a dequantize-only loop reads them
        step(k)
    step_ms, timed_steps = timer(step, sets)
    q_ms, _ = timer(quantize, sets)
    d_ms, _ = timer(dequantize, sets)

    # the same traffic without the arithmetic: a wave reads 8 groups (8 KB float, 4 KB half) and writes their 256 * bits
    # bytes of codes, or the reverse - into the very buffers the kernels use (scale and min, under 1 % of the bytes,
    # are left out)
    probe = probe_lib()
    kb = 8 if esize == 4 else 4
    whole = numel * esize // (kb * 1024)

    def quantize_like(k):
        xi, packed, _, _, _ = bufs[k % sets]
        rc = probe.gact_probe_quantize_like(xi.data_ptr(), packed.data_ptr(), numel * esize, kb, bits,
                                            torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc

    def dequantize_like(k):
        _, packed, _, _, out = bufs[k % sets]
        rc = probe.gact_probe_dequantize_like(packed.data_ptr(), out.data_ptr(), numel * esize, bits, kb,
                                              torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc

    pq_ms, _ = timer(quantize_like, sets)
    pd_ms, _ = timer(dequantize_like, sets)
    probe_bytes = whole * (kb * 1024 + 256 * bits)
    for k in range(sets):   # the probes overwrote codes and outputs: leave every set as the kernels left it
        step(k)

    per_dir = algorithmic_bytes(numel, esize, bits, 4 if x.dtype == torch.bfloat16 else None)
    gbs = lambda ms: per_dir / (ms * 1e-3) / 1e9
    res = {
        "workload": name, "desc": desc, "shape": list(shape), "dtype": dtype, "bits": bits, "rng_stream": stream,
        "bytes_per_direction": per_dir, "buffer_sets": sets, "ms_per_step": step_ms, "timed_steps": timed_steps,
        "gbs": 2 * per_dir / (step_ms * 1e-3) / 1e9,
        "quantize": {"ms": q_ms, "gbs": gbs(q_ms)},
        "dequantize": {"ms": d_ms, "gbs": gbs(d_ms)},
        "probe": {"what": "compute-free kernels with the traffic of the two kernels (%d KB and %d bytes per wave)" % (kb, 256 * bits),
                  "bytes": probe_bytes,
                  "quantize_like": {"us": pq_ms * 1e3, "frac": probe_bytes / (pq_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                    "kernel_over_probe": q_ms / pq_ms},
                  "dequantize_like": {"us": pd_ms * 1e3, "frac": probe_bytes / (pd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                      "kernel_over_probe": d_ms / pd_ms}},
    }
    return res, (x if keep_input else None)


def run_ceilings(torch, timer, name="config2", full=True):
    """What this GPU's memory system gives plain streams over a workload's tensor (config2's 411 MB; config1's
    16 MB, in as many buffer sets as its own measurement rotates over), in the same run: the runtime's
    device-to-device copy, a fill, a pure read (the library's row min/max, which reads the tensor with the fused
    kernel's access pattern and writes 2 values per 256), and torch's element-wise conversion kernel at the 8:1
    and 1:8 read:write mixes of quantize and dequantize.  full = False: the fill and the pure read only."""
    from gact.cpp_extension import _abi

    lib = _abi.lib()
    shape, dtype, _, _, kind, _ = WORKLOADS[name]
    x0 = make_input(torch, shape, dtype, kind)
    nbytes = x0.numel() * x0.element_size()
    N = x0.numel() // 256
    sets = max(1, -(-ROTATE_BYTES // (2 * nbytes + nbytes // 8)))
    xs = [x0 if r == 0 else x0.clone() for r in range(sets)]
    ys = [torch.empty_like(x0) for _ in range(sets)]
    mn = torch.empty((N,), dtype=x0.dtype, device="cuda")
    mx = torch.empty((N,), dtype=x0.dtype, device="cuda")

    def copy(k):
        ys[k % sets].copy_(xs[k % sets])

    def fill(k):
        ys[k % sets].fill_(1.0)

    def read(k):
        _abi.check(lib.gact_minimax(xs[k % sets].data_ptr(), _abi.dtype_code(x0.dtype), N, 256, mn.data_ptr(), mx.data_ptr(),
                                    torch.cuda.current_stream().cuda_stream))

    # the traffic mix of quantize / dequantize at 4 bit (8 bytes read per byte written, and the reverse) through
    # torch's own element-wise kernel: the tensor's bytes as int64, narrowed to int8 and widened back
    narrow = [torch.empty((nbytes // 8 if full else 8,), dtype=torch.int8, device="cuda") for _ in range(sets)]

    def narrow8(k):
        narrow[k % sets].copy_(xs[k % sets].view(torch.int64).view(-1))

    def widen8(k):
        ys[k % sets].view(torch.int64).view(-1).copy_(narrow[k % sets])

    out = {"tensor": "%s's (%d bytes)" % (name, nbytes), "buffer_sets": sets}
    esize = x0.element_size()
    for key, fn, moved in (("device_copy", copy, 2 * nbytes), ("fill", fill, nbytes), ("read_minimax", read, nbytes + 2 * esize * N),
                           ("torch_read8_write1", narrow8, nbytes + nbytes // 8),
                           ("torch_read1_write8", widen8, nbytes + nbytes // 8)):
        if not full and key not in ("fill", "read_minimax"):
            continue
        ms, _ = timer(fn, sets)
        out[key] = {"us": ms * 1e3, "gbs": moved / (ms * 1e-3) / 1e9, "frac": moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    # what a launch costs whatever it moves: one group of 256 elements through the same entry point, replayed the same way
    tiny, tq = x0.reshape(-1)[:256], torch.empty((65,), dtype=torch.int8, device="cuda")
    ts, tm = torch.empty((1,), dtype=x0.dtype, device="cuda"), torch.empty((1,), dtype=x0.dtype, device="cuda")

    def one_group(k):
        _abi.check(lib.gact_quantize(tiny.data_ptr(), _abi.F32, 256, 2, _abi.NOISE_CONST, 0, None, tq.data_ptr(),
                                     ts.data_ptr(), tm.data_ptr(), None, torch.cuda.current_stream().cuda_stream))

    if full:
        ms, _ = timer(one_group)
        out["launch_floor_us"] = ms * 1e3
    return out


def run_entry_points(torch, timer, name="config2", seed=42):
    """The entry points no workload above goes through, each alone on config2's tensor: the reference's
    three-step quantize (gact_minimax, then gact_pack with the caller's min / max; gact_unpack is the way back)
    and the dropout-mask bit packing on a mask with one byte per element of that tensor."""
    from gact.cpp_extension import _abi

    lib = _abi.lib()
    shape, dtype, bits, stream, kind, _ = WORKLOADS[name]
    x0 = make_input(torch, shape, dtype, kind)
    n = x0.numel()
    N = n // 256
    esize = x0.element_size()
    packed_len = lib.gact_packed_bytes(bits, N, 1, 256)
    sets = max(1, -(-ROTATE_BYTES // (n * esize + packed_len)))
    xs = [x0 if r == 0 else x0.clone() for r in range(sets)]
    ys = [torch.empty_like(x0) for _ in range(sets)]
    qs = [torch.empty((packed_len,), dtype=torch.int8, device="cuda") for _ in range(sets)]
    mn, mx, sc = (torch.empty((N,), dtype=x0.dtype, device="cuda") for _ in range(3))
    mode = {"deterministic": _abi.NOISE_CONST, "reference": _abi.NOISE_REF, "fast": _abi.NOISE_FAST}[stream]
    code = _abi.dtype_code(x0.dtype)

    def st():
        return torch.cuda.current_stream().cuda_stream

    _abi.check(lib.gact_minimax(x0.data_ptr(), code, N, 256, mn.data_ptr(), mx.data_ptr(), st()))

    def pack(k):
        _abi.check(lib.gact_pack(xs[k % sets].data_ptr(), mn.data_ptr(), mx.data_ptr(), code, bits, N, 1, 256, mode, seed + k,
                                 None, qs[k % sets].data_ptr(), sc.data_ptr(), st()))

    def unpack(k):
        _abi.check(lib.gact_unpack(qs[k % sets].data_ptr(), bits, sc.data_ptr(), mn.data_ptr(), code, N, 1, 256,
                                   ys[k % sets].data_ptr(), st()))

    for k in range(sets):
        pack(k)
    out = {"tensor": "%s's (%d bytes), %d bit" % (name, n * esize, bits), "buffer_sets": sets}
    for key, fn, moved in (("pack", pack, n * esize + packed_len + 3 * esize * N),
                           ("unpack", unpack, n * esize + packed_len + 2 * esize * N)):
        ms, _ = timer(fn, sets)
        out[key] = {"us": ms * 1e3, "gbs": moved / (ms * 1e-3) / 1e9, "frac": moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    del xs, ys, qs
    torch.cuda.empty_cache()
    words = (n + 31) // 32
    msets = max(1, -(-ROTATE_BYTES // (n + 4 * words)))
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    m0 = (torch.rand((n,), device="cuda", generator=g) < 0.9).to(torch.uint8)
    ms_ = [m0 if r == 0 else m0.clone() for r in range(msets)]
    ws = [torch.empty((words,), dtype=torch.int32, device="cuda") for _ in range(msets)]

    def mask_pack(k):
        _abi.check(lib.gact_mask_pack(ms_[k % msets].data_ptr(), n, ws[k % msets].data_ptr(), st()))

    def mask_unpack(k):
        _abi.check(lib.gact_mask_unpack(ws[k % msets].data_ptr(), n, ms_[k % msets].data_ptr(), st()))

    for k in range(msets):
        mask_pack(k)
    for key, fn in (("mask_pack", mask_pack), ("mask_unpack", mask_unpack)):
        ms, _ = timer(fn, msets)
        moved = n + 4 * words
        out[key] = {"us": ms * 1e3, "gbs": moved / (ms * 1e-3) / 1e9, "frac": moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                    "bytes": moved}
    return out


def run_config5(torch, timer, seed=42):
    """Workload "config5", the full adaptive step: 120 fp16 tensors with Swin-Tiny-like shapes, per-tensor
    sensitivities ~LogNormal(0,2), budget 2 bits per element.  One step = greedy calc_precision on the GPU
    (widths stay in device memory), offset planning, one batched mixed-width quantize and one batched
    dequantize, all through the C ABI."""
    import numpy as np

    from gact.batched import BatchedQuantizer
    from gact.cpp_extension import _abi

    lib = _abi.lib()
    shapes = [(128, 3136, 96)] * 20 + [(128, 784, 192)] * 20 + [(128, 196, 384)] * 60 + [(128, 49, 768)] * 20
    g = torch.Generator(device="cuda").manual_seed(0)
    xs = [torch.randn(s, generator=g, device="cuda", dtype=torch.float16) for s in shapes]
    outs = [torch.empty_like(x) for x in xs]
    L = len(xs)
    rng = np.random.default_rng(0)
    C = torch.from_numpy(np.exp(rng.normal(0.0, 2.0, L)).astype(np.float32)).cuda()
    w = torch.tensor([x.numel() for x in xs], dtype=torch.int64, device="cuda")
    target = 2.0 * float(sum(x.numel() for x in xs))
    init = torch.full((L,), 8, dtype=torch.int32, device="cuda")
    bits = init.clone()
    status = torch.zeros((1,), dtype=torch.int32, device="cuda")
    bq = BatchedQuantizer([x.numel() for x in xs], [torch.float16] * L, "cuda")
    seeds = [i + seed for i in range(L)]
    table_q = bq._table(xs, seeds)
    table_d = bq._table(outs, seeds)
    packed = torch.empty((bq.arena_bytes_for_budget(target),), dtype=torch.uint8, device="cuda")
    sc = torch.empty((bq.total_groups * 4,), dtype=torch.uint8, device="cuda")
    mn = torch.empty((bq.total_groups * 4,), dtype=torch.uint8, device="cuda")
    ws_q, ws_d = bq.new_workspace(), bq.new_workspace()
    cur = lambda: torch.cuda.current_stream().cuda_stream

    def allocate(k):
        bits.copy_(init)
        _abi.check(lib.gact_calc_precision_device(bits.data_ptr(), C.data_ptr(), w.data_ptr(), L, target,
                                                  status.data_ptr(), cur()))

    def quantize(k):
        bq.launch_quantize(table_q, bits, packed, sc, mn, ws_q, _abi.NOISE_FAST)

    def dequantize(k):
        bq.launch_dequantize(table_d, bits, packed, sc, mn, ws_d)

    def step(k):
        allocate(k)
        quantize(k)
        dequantize(k)

    step(0)
    step_ms, timed_steps = timer(step)
    a_ms, _ = timer(allocate)
    q_ms, _ = timer(quantize)
    d_ms, _ = timer(dequantize)
    torch.cuda.synchronize()
    host_bits = bits.cpu().tolist()
    assert status.item() == 0 and bq.plan_ok(ws_q) and bq.plan_ok(ws_d)
    per_dir = sum(algorithmic_bytes(x.numel(), 2, b) for x, b in zip(xs, host_bits))
    return {
        "workload": "config5", "desc": "120 fp16 Swin-Tiny-like tensors, widths by calc_precision on the GPU (budget "
                                       "2 bits/element), one batched mixed-width quantize + dequantize",
        "tensors": L, "elements": int(sum(x.numel() for x in xs)), "dtype": "float16", "rng_stream": "fast",
        "bits": "1/2/4/8 by calc_precision", "width_histogram": {str(b): host_bits.count(b) for b in (1, 2, 4, 8)},
        "bytes_per_direction": per_dir, "buffer_sets": 1, "ms_per_step": step_ms, "timed_steps": timed_steps,
        "gbs": 2 * per_dir / (step_ms * 1e-3) / 1e9,
        "calc_precision": {"ms": a_ms},
        "quantize": {"ms": q_ms, "gbs": per_dir / (q_ms * 1e-3) / 1e9},
        "dequantize": {"ms": d_ms, "gbs": per_dir / (d_ms * 1e-3) / 1e9},
    }


def cpu_baseline(torch, x, bits, stream, budget_s=10.0, max_elems=1 << 23):
    """The C restatement on the host cores: the whole tensor when it has at most 8 M elements, else a leading
    slice of that size."""
    import oracle

    mode = {"deterministic": oracle.NOISE_CONST, "reference": oracle.NOISE_REF, "fast": oracle.NOISE_FAST}[stream]
    flat = x.reshape(-1)
    sample_elems = min(flat.numel(), max_elems) // 256 * 256
    xs = flat[:sample_elems].cpu().numpy()
    N = sample_elems // 256
    groups = xs.reshape(N, 256)
    esize = xs.dtype.itemsize

    def one_pass():
        q = oracle.op_quantize(groups, bits, mode, 42)
        oracle.op_dequantize(q, groups.shape)

    one_pass()  # warm-up (also loads the library)
    t0 = time.perf_counter()
    reps = 0
    while True:
        one_pass()
        reps += 1
        if time.perf_counter() - t0 >= budget_s:
            break
    dt = (time.perf_counter() - t0) / reps
    per_dir = algorithmic_bytes(sample_elems, esize, bits)
    what = "the whole tensor" if sample_elems == flat.numel() else "a sample: the first %d of %d elements" % (sample_elems, flat.numel())
    return {
        "value": 2 * per_dir / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
        "sample": "%s (%d groups), %d quantize+dequantize passes of the C restatement (oracle/gact_oracle.c, "
                  "OpenMP) in %.1f s" % (what, N, reps, dt * reps),
    }


def python_ops_us(torch, name, min_seconds):
    """op_quantize and op_dequantize of the Python face, launched from the host one call after the other."""
    from gact import ops

    shape, dtype, bits, stream, kind, _ = WORKLOADS[name]
    x = make_input(torch, shape, dtype, kind)
    out = {}
    q = ops.op_quantize(x, bits, 0, rng_stream=stream)
    for key, fn in (("quantize", lambda: ops.op_quantize(x, bits, 0, rng_stream=stream)),
                    ("dequantize", lambda: ops.op_dequantize(q, x.shape))):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        calls, t0 = 0, time.perf_counter()
        while True:
            for _ in range(100):
                fn()
            torch.cuda.synchronize()
            calls += 100
            if time.perf_counter() - t0 >= min(min_seconds, 0.5):
                break
        out[key] = (time.perf_counter() - t0) / calls * 1e6
    return out


def compact(res):
    """The per-configuration entry of the JSON line."""
    out = {
        "desc": res["desc"], "dtype": res["dtype"], "bits": res["bits"], "rng_stream": res["rng_stream"],
        "bytes_per_direction": res["bytes_per_direction"],
        "buffer_sets": res["buffer_sets"],
        "step": {"us": res["ms_per_step"] * 1e3, "gbs": res["gbs"], "frac": res["gbs"] / HBM_PEAK_GBS},
    }
    for k in ("quantize", "dequantize"):
        out[k] = {"us": res[k]["ms"] * 1e3, "gbs": res[k]["gbs"], "frac": res[k]["gbs"] / HBM_PEAK_GBS,
                  "traffic": TRAFFIC_BYTES.get((res["workload"], k))}    # HBM bytes per launch by the counters, or null
    for k in ("width_histogram", "tensors", "elements", "probe"):
        if k in res:
            out[k] = res[k]
    if "calc_precision" in res:
        out["calc_precision_us"] = res["calc_precision"]["ms"] * 1e3
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="config1", choices=sorted(WORKLOADS) + ["config5"],
                    help="the workload `value`, `roofline` and `cpu_baseline` are about")
    ap.add_argument("--only", action="store_true", help="measure the headline workload only (profiling runs)")
    ap.add_argument("--min-seconds", type=float, default=MIN_SECONDS, help="minimum measured time of every loop")
    ap.add_argument("--eager", action="store_true", help="launch every step from the host instead of replaying a graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the timed region also launch 20 plain device copies of the workload tensor, so "
                         "that a counter run of this command holds a copy kernel of known size to scale by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no cross-GPU step (each rank compresses its own "
                 "activations); run with --gpus 1")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    torch.cuda.set_device(0)
    timer = Timer(torch, args.steps, args.warmup, args.min_seconds, graph=not args.eager)

    def run(name, keep_input=False):
        if name == "config5":
            # the batched step is milliseconds long and allocates nothing: launched from the host
            return run_config5(torch, Timer(torch, max(5, args.steps // 5), max(2, args.warmup // 5), args.min_seconds,
                                            graph=False)), None
        r = run_workload(torch, name, timer, keep_input=keep_input)
        torch.cuda.empty_cache()
        return r

    res, x = run(args.workload, keep_input=True)
    dom = "quantize" if res["quantize"]["ms"] >= res["dequantize"]["ms"] else "dequantize"
    achieved = res[dom]["gbs"]
    line = {
        "metric": BASELINE_METRIC,
        "value": res["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"float32": "f32", "float16": "f16", "bfloat16": "bf16"}[res["dtype"]], "data": "synthetic",
        "config": {"workload": "%s: %s" % (args.workload, res["desc"]), "bits": res["bits"], "group_size": 256,
                   "rng_stream": res["rng_stream"], "bytes_per_step": 2 * res["bytes_per_direction"],
                   "bytes_counted": "algorithmic input + output bytes of both kernels",
                   "buffer_sets": res["buffer_sets"],
                   "timing": ("blocks of `steps` steps launched from the host" if args.eager or args.workload == "config5" else
                              "blocks of `steps` steps recorded as one HIP graph and replayed") +
                             " between two events, repeated for at least %.1f s" % args.min_seconds},
        "timed_steps": res["timed_steps"],
        "frac_of_hbm_peak": res["gbs"] / HBM_PEAK_GBS,
        "kernels": {k: {"us": res[k]["ms"] * 1e3, "gbs": res[k]["gbs"]} for k in ("quantize", "dequantize")},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": TRAFFIC_BYTES.get((args.workload, dom))},
    }
    if args.copy_calibration:
        # a copy kernel of known size for a counter run to scale by: the workload's tensor, or 256 MiB where the
        # workload has no single tensor (config5)
        src = x if x is not None else torch.zeros((1 << 28,), dtype=torch.uint8, device="cuda")
        y = torch.empty_like(src)
        for _ in range(20):
            y.copy_(src)
        torch.cuda.synchronize()
        line["copy_calibration"] = {"kernel": "device-to-device copy", "launches": 20,
                                    "bytes_read": src.numel() * src.element_size(),
                                    "bytes_written": src.numel() * src.element_size()}
        del y, src
    if not args.only:
        configs = {args.workload: compact(res)}
        for name in BASELINE_SET + ["config5"]:
            if name not in configs:
                configs[name] = compact(run(name)[0])
        # config 3 as BASELINE.json words it: the three BERT-large tensors of one layer, one after the other
        parts = [configs[n] for n in ("config3-hidden", "config3-gelu", "config3-probs")]
        c3_bytes = sum(p["bytes_per_direction"] for p in parts)
        c3_us = sum(p["step"]["us"] for p in parts)
        configs["config3"] = {"desc": "sum of config3-hidden (8 bit), config3-gelu (4 bit), config3-probs (2 bit)",
                              "bytes_per_direction": c3_bytes,
                              "step": {"us": c3_us, "gbs": 2 * c3_bytes / c3_us / 1e3,
                                       "frac": 2 * c3_bytes / c3_us / 1e3 / HBM_PEAK_GBS}}
        # the headline tensor again with ONE buffer set: 37 MB that stay in the 256 MB last-level cache between
        # steps, which is how a training step meets an activation the previous kernel has just written.  Not a
        # BASELINE figure (those stream from HBM); it separates the kernels from the cold 16 MB stream.
        cached = compact(run_workload(torch, "config1", timer, rotate=False)[0])
        cached["desc"] = "config1 with one buffer set (cache-resident between steps)"
        configs["config1-cached"] = cached
        torch.cuda.empty_cache()
        # the same tensor the way the reference's test times it: op_quantize / op_dequantize called from Python
        # (allocations included), synchronised around each batch of calls
        configs["reference-test-speed"]["python_ops_us"] = python_ops_us(torch, "reference-test-speed", args.min_seconds)
        line["configs"] = configs
        line["ceilings"] = run_ceilings(torch, timer, "config2")
        torch.cuda.empty_cache()
        line["entry_points"] = run_entry_points(torch, timer, "config2")
        torch.cuda.empty_cache()
        # the same plain streams at the headline workload's size, where the launch and the ramp of a 16 MB
        # stream count: what a kernel that only reads (or only fills) this tensor takes
        line["ceilings_headline"] = run_ceilings(torch, timer, "config1")
        torch.cuda.empty_cache()
        # and the fill and the pure read at the sizes of the other small and mid-sized workloads
        line["ceilings_by_size"] = {}
        for name in ("config3-hidden", "config3-gelu", "config4"):
            line["ceilings_by_size"][name] = run_ceilings(torch, timer, name, full=False)
            torch.cuda.empty_cache()
    if not args.no_cpu and x is not None:
        line["cpu_baseline"] = cpu_baseline(torch, x, res["bits"], res["rng_stream"])
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
