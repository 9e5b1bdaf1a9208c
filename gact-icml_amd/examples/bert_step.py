"""Training step of a randomly initialised BERT-base classifier with and without activation compression:
time per iteration and peak device memory per optimisation level.

    python gact-icml_amd/examples/bert_step.py [--batch 16] [--seq 512] [--amp | --amp-bf16] [--levels L0 L1 L1.2]

Needs the `transformers` package (no download: the model is built from a default BertConfig).  The usage
is the reference's: build a Controller on the model, install its hooks, call controller.iterate(backprop)
after every optimizer step.
"""
import argparse
import os
import sys
import time

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import gact  # noqa: E402
from gact.conf import config  # noqa: E402


def run(level, batch, seq, amp, steps, amp_dtype=torch.float16):
    import transformers
    model_config = transformers.BertConfig()
    model_config._attn_implementation = "eager"
    torch.manual_seed(0)
    model = transformers.BertForSequenceClassification(model_config).cuda().train()
    optimizer = torch.optim.SGD(model.parameters(), lr=1e-3)
    ids = torch.randint(0, model_config.vocab_size, (batch, seq), device="cuda")
    labels = torch.randint(0, 2, (batch,), device="cuda")

    config.__init__()
    controller = None
    if level != "L0":
        gact.set_optimization_level(level)
        controller = gact.controller.Controller(model)
        controller.install_hook()

    def backprop():
        model.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=amp_dtype, enabled=amp):
            loss = model(input_ids=ids, labels=labels).loss
        loss.backward()
        return loss

    torch.cuda.reset_peak_memory_stats()
    times = []
    for _ in range(steps):
        torch.cuda.synchronize()
        start = time.perf_counter()
        backprop()
        optimizer.step()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - start)
        if controller is not None:
            controller.iterate(backprop)      # auto precision runs its extra passes here, outside the timing
    if controller is not None:
        controller.uninstall_hook()
    median = sorted(times[2:])[len(times[2:]) // 2]
    mode = "fp32" if not amp else "autocast " + str(amp_dtype)[6:]
    print("%-5s %s batch=%d seq=%d: %6.1f ms/iteration  %6.1f samples/s  peak %5.2f GiB"
          % (level, mode, batch, seq, median * 1e3, batch / median, torch.cuda.max_memory_allocated() / 2 ** 30), flush=True)


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("--batch", type=int, default=16)
    parser.add_argument("--seq", type=int, default=512)
    parser.add_argument("--steps", type=int, default=8)
    parser.add_argument("--amp", action="store_true", help="float16 autocast")
    parser.add_argument("--amp-bf16", action="store_true", help="bfloat16 autocast")
    parser.add_argument("--levels", nargs="+", default=["L0", "L1", "L1.2"])
    args = parser.parse_args()
    for level in args.levels:
        run(level, args.batch, args.seq, args.amp or args.amp_bf16, args.steps,
            torch.bfloat16 if args.amp_bf16 else torch.float16)
        torch.cuda.empty_cache()
