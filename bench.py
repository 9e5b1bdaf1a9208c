#!/usr/bin/env python3
"""Throughput of the saved-activation compression path on one MI355X.

One step = one fused quantize (min/max + scale + stochastic rounding + pack) followed by one
dequantize (unpack + affine) of one synthetic activation tensor, through the C ABI, with the input
already resident in HBM.  The default workload is the headline one ("config2"): a ResNet-50 conv
activation, fp32 NCHW [128,256,56,56], post-ReLU, group 256, 4 bit, stochastic rounding with Philox
seed 42.  Bytes are the algorithmic input + output bytes of both directions:
numel*sizeof(T) + packed bytes + 2*N*sizeof(T) per direction.

Prints ONE JSON line.  `value` and `ms_per_step` come from K steps launched back to back between two
synchronisations.  `roofline` is for the slower of the two kernels, timed in a second pass over the same
K steps with an event pair around every launch on the stream the kernels run on; `cpu_baseline` is the C
restatement of the reference arithmetic (oracle/) run with OpenMP on the host cores over a bounded sample.
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

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by
# a copy kernel of known size (profiles/config2_fp32_4bit_quantize_dequantize.txt: the copy kernel reads
# FETCH_SIZE x 1.99988 and WRITE_SIZE x 1.00000 KiB); None for workloads without a counter run
TRAFFIC_BYTES = {
    ("config2", "quantize"): 466.5e6,    # 411.1 MB read + 55.4 MB written; algorithmic 465.6 MB
    ("config2", "dequantize"): 465.7e6,  # 54.7 MB read + 411.1 MB written; algorithmic 465.6 MB
}

# BASELINE.json's metric, verbatim.  Its text says 2 bit while the configuration it is quoted on (configs[1], the
# default workload here) is 4 bit: the line carries the default workload as `value` and the same tensor at
# 2 bit under `two_bit_same_tensor`.
BASELINE_METRIC = "quantize+dequantize GB/s and % of HBM peak, 1\u00d7MI355X, 2-bit group=256"

# a workload whose buffers are smaller than this is timed over several buffer sets in rotation
ROTATE_BYTES = 800 * 1000 * 1000

WORKLOADS = {
    # name: (shape, dtype, bits, rng_stream, data kind, description)
    "config1": ((4096, 1024), "float32", 2, "deterministic", "randn",
                "fp32 [4096,1024] ~N(0,1), 2 bit, deterministic rounding"),
    "config2": ((128, 256, 56, 56), "float32", 4, "fast", "relu",
                "ResNet-50 conv activation fp32 [128,256,56,56] post-ReLU, 4 bit, stochastic rounding, Philox seed 42"),
    "config2-2bit": ((128, 256, 56, 56), "float32", 2, "fast", "relu",
                     "config2's tensor at 2 bit (the width BASELINE.json's metric string names)"),
    "config2-refstream": ((128, 256, 56, 56), "float32", 4, "reference", "relu",
                          "config2 with the reference's one-Philox-state-per-byte noise stream"),
    "config3-hidden": ((16384, 1024), "float16", 8, "fast", "randn", "BERT-large hidden states fp16, 8 bit"),
    "config3-gelu": ((16384, 4096), "float16", 4, "fast", "randn", "BERT-large GELU inputs fp16, 4 bit"),
    "config3-probs": ((32, 16, 512, 512), "float16", 2, "fast", "softmax", "BERT-large attention probs fp16, 2 bit"),
    "config4": ((169343, 256), "float32", 1, "fast", "relu60", "GCN node features fp32 [169343,256], ~60% zeros, 1 bit"),
    # not a BASELINE workload: the GELU-input tensor of config 3 as mixed-precision training on this GPU holds it
    "bf16-gelu": ((16384, 4096), "bfloat16", 4, "fast", "randn", "GELU inputs in bfloat16, 4 bit (float scale, bfloat16 min)"),
}


def make_input(torch, shape, dtype, kind, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32)
    if kind == "relu":
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


def run_workload(torch, name, steps, warmup, seed=42):
    """One step = quantize then dequantize of the workload's tensor.  A tensor whose buffers would fit the
    256 MB last-level cache is given several buffer sets used in rotation, so that every step streams from
    and to HBM as it does inside a training step."""
    from gact.cpp_extension import _abi

    shape, dtype, bits, stream, kind, desc = WORKLOADS[name]
    lib = _abi.lib()
    x = make_input(torch, shape, dtype, kind)
    numel = x.numel()
    N = (numel + 255) // 256
    esize = x.element_size()
    packed_len = lib.gact_packed_bytes(bits, N, 1, 256) + 1
    working_set = 2 * numel * esize + packed_len
    sets = max(1, -(-ROTATE_BYTES // working_set))
    scale_dtype = torch.float32 if x.dtype == torch.bfloat16 else x.dtype      # bfloat16 tensors keep a float scale
    bufs = []
    for r in range(sets):
        bufs.append((x if r == 0 else x.clone(),
                     torch.empty((packed_len,), dtype=torch.int8, device="cuda"),
                     torch.empty((N,), dtype=scale_dtype, device="cuda"), torch.empty((N,), dtype=x.dtype, device="cuda"),
                     torch.empty_like(x)))
    st = torch.cuda.current_stream().cuda_stream
    dt = _abi.dtype_code(x.dtype)
    mode = _abi.NOISE_MODES[stream]

    def quantize(k):
        xi, packed, scale, mn, _ = bufs[k % sets]
        _abi.check(lib.gact_quantize(xi.data_ptr(), dt, numel, bits, mode, seed, None, packed.data_ptr(),
                                     scale.data_ptr(), mn.data_ptr(), None, st))

    def dequantize(k):
        _, packed, scale, mn, out = bufs[k % sets]
        _abi.check(lib.gact_dequantize(packed.data_ptr(), bits, scale.data_ptr(), mn.data_ptr(), dt, numel,
                                       out.data_ptr(), st))

    for k in range(max(warmup, sets)):
        quantize(k)
        dequantize(k)

    # the timed steps: nothing but the launches between the two synchronisations
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        quantize(k)
        dequantize(k)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / steps

    # the same steps again with an event pair around every launch, for the duration of each kernel (an
    # event between two launches drains the pipeline, about 5 us per step, so this pass is not the one the
    # step time comes from)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    torch.cuda.synchronize()
    for k in range(steps):
        ev[k][0].record()
        quantize(k)
        ev[k][1].record()
        dequantize(k)
        ev[k][2].record()
    torch.cuda.synchronize()

    per_dir = algorithmic_bytes(numel, esize, bits, 4 if x.dtype == torch.bfloat16 else None)
    q_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / steps
    d_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / steps
    res = {
        "workload": name, "desc": desc, "shape": list(shape), "dtype": dtype, "bits": bits, "rng_stream": stream,
        "bytes_per_direction": per_dir, "buffer_sets": sets, "ms_per_step": wall_ms,
        "gbs": 2 * per_dir / (wall_ms * 1e-3) / 1e9,
        "quantize": {"ms": q_ms, "gbs": per_dir / (q_ms * 1e-3) / 1e9},
        "dequantize": {"ms": d_ms, "gbs": per_dir / (d_ms * 1e-3) / 1e9},
    }
    return res, x


def run_config5(torch, steps, warmup, seed=42):
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
    plan = torch.empty((6,), dtype=torch.int64, device="cuda")
    st = torch.cuda.current_stream().cuda_stream

    def allocate():
        bits.copy_(init)
        _abi.check(lib.gact_calc_precision_device(bits.data_ptr(), C.data_ptr(), w.data_ptr(), L, target,
                                                  status.data_ptr(), st))

    def quantize():
        _abi.check(lib.gact_batch_plan(table_q.data_ptr(), bits.data_ptr(), L, packed.numel(), plan.data_ptr(), st))
        _abi.check(lib.gact_quantize_batched(table_q.data_ptr(), bits.data_ptr(), L, bq.total_blocks, _abi.NOISE_FAST,
                                             bq.dtype_mask, plan.data_ptr(), bq.block_map.data_ptr(), packed.data_ptr(),
                                             sc.data_ptr(), mn.data_ptr(), st))

    def dequantize():
        _abi.check(lib.gact_batch_plan(table_d.data_ptr(), bits.data_ptr(), L, packed.numel(), plan.data_ptr(), st))
        _abi.check(lib.gact_dequantize_batched(table_d.data_ptr(), bits.data_ptr(), L, bq.total_blocks,
                                               plan.data_ptr(), bq.block_map.data_ptr(), packed.data_ptr(),
                                               sc.data_ptr(), mn.data_ptr(), st))

    for _ in range(warmup):
        allocate(); quantize(); dequantize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        allocate(); quantize(); dequantize()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / steps

    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]
    for k in range(steps):
        ev[k][0].record(); allocate()
        ev[k][1].record(); quantize()
        ev[k][2].record(); dequantize()
        ev[k][3].record()
    torch.cuda.synchronize()
    host_bits = bits.cpu().tolist()
    assert status.item() == 0 and plan.cpu().tolist()[1] == 1
    per_dir = sum(algorithmic_bytes(x.numel(), 2, b) for x, b in zip(xs, host_bits))
    a_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / steps
    q_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / steps
    d_ms = sum(e[2].elapsed_time(e[3]) for e in ev) / steps

    # the same tensors and widths one call per tensor (what a hook-driven loop does), for comparison
    singles = []
    for x, o, b, sd in zip(xs, outs, host_bits, seeds):
        N = (x.numel() + 255) // 256
        singles.append((x, o, b, sd, torch.empty((lib.gact_packed_bytes(b, N, 1, 256) + 1,), dtype=torch.int8, device="cuda"),
                        torch.empty((N,), dtype=x.dtype, device="cuda"), torch.empty((N,), dtype=x.dtype, device="cuda")))

    def loop_q():
        for x, o, b, sd, pk, s1, m1 in singles:
            lib.gact_quantize(x.data_ptr(), 1, x.numel(), b, _abi.NOISE_FAST, sd, None, pk.data_ptr(), s1.data_ptr(),
                              m1.data_ptr(), None, st)

    def loop_d():
        for x, o, b, sd, pk, s1, m1 in singles:
            lib.gact_dequantize(pk.data_ptr(), b, s1.data_ptr(), m1.data_ptr(), 1, x.numel(), o.data_ptr(), st)

    loop_ms = []
    for fn in (loop_q, loop_d):
        fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            fn()
        e1.record()
        torch.cuda.synchronize()
        loop_ms.append(e0.elapsed_time(e1) / 5)
    return {
        "workload": "config5", "desc": "120 fp16 Swin-Tiny-like tensors, widths by calc_precision on the GPU (budget "
                                       "2 bits/element), one batched mixed-width quantize + dequantize",
        "tensors": L, "elements": int(sum(x.numel() for x in xs)), "dtype": "float16", "rng_stream": "fast",
        "width_histogram": {str(b): host_bits.count(b) for b in (1, 2, 4, 8)},
        "bytes_per_direction": per_dir, "ms_per_step": wall_ms, "gbs": 2 * per_dir / (wall_ms * 1e-3) / 1e9,
        "calc_precision": {"ms": a_ms},
        "quantize": {"ms": q_ms, "gbs": per_dir / (q_ms * 1e-3) / 1e9},
        "dequantize": {"ms": d_ms, "gbs": per_dir / (d_ms * 1e-3) / 1e9},
        "tensor_by_tensor": {"quantize_ms": loop_ms[0], "dequantize_ms": loop_ms[1],
                             "quantize_gbs": per_dir / (loop_ms[0] * 1e-3) / 1e9,
                             "dequantize_gbs": per_dir / (loop_ms[1] * 1e-3) / 1e9},
    }


def cpu_baseline(torch, x, bits, stream, budget_s=12.0):
    """The C restatement on the host cores over a leading slice of the same tensor."""
    import numpy as np

    import oracle

    mode = {"deterministic": oracle.NOISE_CONST, "reference": oracle.NOISE_REF, "fast": oracle.NOISE_FAST}[stream]
    flat = x.reshape(-1)
    sample_elems = min(flat.numel(), 256 * 32768)  # 8M elements
    xs = flat[:sample_elems].cpu().numpy()
    N = sample_elems // 256
    groups = xs.reshape(N, 256)
    esize = xs.dtype.itemsize

    def one_pass():
        q = oracle.op_quantize(groups, bits, mode, 42)
        oracle.op_dequantize(q, groups.shape)

    one_pass()  # warm-up (also builds / loads the library)
    t0 = time.perf_counter()
    reps = 0
    while True:
        one_pass()
        reps += 1
        if time.perf_counter() - t0 >= budget_s:
            break
    dt = (time.perf_counter() - t0) / reps
    per_dir = algorithmic_bytes(sample_elems, esize, bits)
    return {
        "value": 2 * per_dir / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
        "sample": "first %d of %d elements of the same tensor (%d groups), %d quantize+dequantize passes of the C "
                  "restatement (oracle/gact_oracle.c, OpenMP) in %.1f s" % (sample_elems, flat.numel(), N, reps, dt * reps),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="config2", choices=sorted(WORKLOADS) + ["config5"])
    ap.add_argument("--all", action="store_true", help="also time the other single-tensor workloads (extra key)")
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

    if args.workload == "config5":
        res, x = run_config5(torch, args.steps, args.warmup), None
        res.update(bits="1/2/4/8 by calc_precision", dtype="float16")
        args.copy_calibration, args.no_cpu = False, True     # no single tensor to copy or to hand to the CPU leg
    else:
        res, x = run_workload(torch, args.workload, args.steps, args.warmup)
    dom = "quantize" if res["quantize"]["ms"] >= res["dequantize"]["ms"] else "dequantize"
    achieved = res[dom]["gbs"]
    line = {
        "metric": BASELINE_METRIC,
        "value": res["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"float32": "f32", "float16": "f16", "bfloat16": "bf16"}[res["dtype"]], "data": "synthetic",
        "config": {"workload": "%s: %s" % (args.workload, res["desc"]), "bits": res["bits"], "group_size": 256,
                   "rng_stream": res["rng_stream"], "bytes_per_step": 2 * res["bytes_per_direction"]},
        "frac_of_hbm_peak": res["gbs"] / HBM_PEAK_GBS,
        "kernels": {"quantize": res["quantize"], "dequantize": res["dequantize"]},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": TRAFFIC_BYTES.get((args.workload, dom))},
    }
    line["config"]["bytes_counted"] = "algorithmic input + output bytes of both kernels"
    if args.workload == "config2":
        r2, _ = run_workload(torch, "config2-2bit", args.steps, args.warmup)
        line["two_bit_same_tensor"] = {"value": r2["gbs"], "unit": "GB/s", "ms_per_step": r2["ms_per_step"],
                                       "frac_of_hbm_peak": r2["gbs"] / HBM_PEAK_GBS,
                                       "kernels": {"quantize": r2["quantize"], "dequantize": r2["dequantize"]}}
        torch.cuda.empty_cache()
    if args.copy_calibration:
        y = torch.empty_like(x)
        for _ in range(20):
            y.copy_(x)
        torch.cuda.synchronize()
        line["copy_calibration"] = {"kernel": "torch elementwise copy", "launches": 20,
                                    "bytes_read": x.numel() * x.element_size(),
                                    "bytes_written": x.numel() * x.element_size()}
        del y
    if args.all:
        extra = []
        for name in sorted(WORKLOADS):
            if name == args.workload:
                continue
            r, _ = run_workload(torch, name, max(20, args.steps // 4), max(3, args.warmup // 4))
            extra.append(r)
            torch.cuda.empty_cache()
        if args.workload != "config5":
            extra.append(run_config5(torch, 20, 3))
        torch.cuda.empty_cache()
        line["other_workloads"] = extra
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(torch, x, res["bits"], res["rng_stream"])
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
