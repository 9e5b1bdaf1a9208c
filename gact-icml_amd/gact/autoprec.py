"""Adaptive per-tensor widths.

Every `adapt_interval` iterations the sensitivity of each saved tensor is measured from how much the
parameter gradient moves when only that tensor is quantized differently (1 bit with two seeds, and 8 bit);
the widths are then allocated greedily under the budget `avg_bits * total elements` by calc_precision.
Same constructor, attributes and call order as gact/gact/autoprec.py of the reference, whose numbers
(three probes per tensor, max(d01, 2 max(d02, d12)), the 1e10 cap, the variance warning) are kept.
"""
import contextlib
import os
import random

import numpy as np
import torch
import torch.nn as nn

from .conf import config
from .cpp_extension import calc_precision as ext_calc_precision
from .utils import exp_recorder

SENSITIVITY_CAP = 1e10
DEVICE_CALC_PRECISION_MAX_TENSORS = 4096     # what one launch of the device allocation takes


def _seed_everything(seed):
    random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    if torch.cuda.is_available():
        torch.cuda.manual_seed_all(seed)


@contextlib.contextmanager
def _probe_context(model, seed):
    """An extra forward/backward must not move batch-norm running statistics nor the caller's CPU random
    stream, and must itself be reproducible: fixed seed inside, state restored afterwards
    (gact/gact/autoprec.py:80-100)."""
    kinds = (nn.BatchNorm1d, nn.BatchNorm2d, nn.BatchNorm3d)
    norms = [m for m in model.modules() if isinstance(m, kinds)] if model is not None else []
    for m in norms:
        m.track_running_stats = False
    cpu_state = torch.get_rng_state().clone()
    _seed_everything(seed)
    try:
        yield
    finally:
        torch.set_rng_state(cpu_state)
        for m in norms:
            m.track_running_stats = True


def _sq_dist(a, b):
    return ((a - b) ** 2).sum()


class AutoPrecision:
    def __init__(self, model, quantizer, bits, max_bits, work_dir, adapt_interval, log_interval,
                 momentum=0.99, warmup_iter=100, debug=False):
        self.model, self.quantizer = model, quantizer
        self.avg_bits, self.max_bits = bits, max_bits
        self.adapt_interval, self.log_iter = adapt_interval, log_interval
        self.work_dir, self.debug = work_dir, debug
        self.iter = 0

        self.dims = None     # tensor id -> element count (the quantizer's table, adopted on first use)
        self.bits = {}       # tensor id -> width
        self.C = {}          # tensor id -> sensitivity

        # exponential averages behind the "quantization variance is too large" warning
        self.momentum = momentum
        self.warmpup_iter = warmup_iter
        self.beta1 = 1e-7
        self.batch_grad = 0
        self.grad_var = 0

    # ------------------------------------------------------------------ set-up
    def init_from_dims(self):
        """Adopt the element counts the quantizer recorded on its first iteration; every tensor starts at
        the average width with sensitivity 1 (gact/gact/autoprec.py:39-46)."""
        self.dims = self.quantizer.dims
        self.C = {l: 1.0 for l in self.dims}
        self.bits = {l: self.avg_bits for l in self.dims}
        self.total_bits = self.avg_bits * sum(self.dims.values())

    def iterate_wrapper(self, backprop):
        if self.dims is None:
            self.init_from_dims()
        self.iterate(backprop)

    # ------------------------------------------------------------------ probes
    def _get_grad(self, backprop):
        """Flattened parameter gradient of one extra pass; the quantizer's per-iteration state is reset after."""
        with _probe_context(self.model, self.iter):
            backprop()
        flat = [p.grad.ravel() for p in self.model.parameters() if p.grad is not None]
        self.quantizer.iterate()
        return torch.cat(flat, 0)

    def _sensitivity_of(self, l, backprop):
        """Three passes with only tensor l changed: 1 bit, 1 bit under the next seed, 8 bit."""
        q = self.quantizer
        kept = q.bits[l]
        try:
            q.bits[l] = 1
            g_a = self._get_grad(backprop)
            q.seeds[l] += 1
            g_b = self._get_grad(backprop)
            q.seeds[l] -= 1
            q.bits[l] = 8
            g_c = self._get_grad(backprop)
        finally:
            q.bits[l] = kept
        # a 0-d tensor on the gradients' device: comparing or reading it here would wait for the three passes,
        # the caller reads all tensors' values back at once
        sens = torch.maximum(_sq_dist(g_a, g_b), 2 * torch.maximum(_sq_dist(g_a, g_c), _sq_dist(g_b, g_c)))
        cap = torch.full_like(sens, SENSITIVITY_CAP)
        return torch.where(torch.isfinite(sens) & (sens <= SENSITIVITY_CAP), sens, cap)

    def _predicted_variance(self, shift):
        C = np.array([self.C[l] for l in self.C])
        b = np.array([self.bits[l] for l in self.C])
        return (C * 2 ** (-2.0 * (b - shift))).sum()

    def _record_state(self, **extra):
        exp_recorder.record("iter", self.iter)
        exp_recorder.record("layer sensitivity", self.C)
        exp_recorder.record("bits", self.bits)
        exp_recorder.record("dims", self.dims)
        for k, v in extra.items():
            exp_recorder.record(k, v)
        os.makedirs(self.work_dir, exist_ok=True)
        exp_recorder.dump(os.path.join(self.work_dir, "autoprec.log"))

    # ------------------------------------------------------------------ per iteration
    def iterate(self, backprop):
        """gact/gact/autoprec.py:57-186."""
        adapting = self.iter % self.adapt_interval == 0
        if adapting:
            print('GACT: Initializing AutoPrec..., run extra %d iters' % (len(self.quantizer.bits)))
            # the probes of all tensors are queued without a host synchronisation between them (the reference
            # reads every sensitivity back as soon as its three passes are queued); one read-back at the end
            layers = list(self.quantizer.bits)
            sens = [self._sensitivity_of(l, backprop) for l in layers]
            if sens and self._allocates_on_device(layers, sens):
                # the sensitivities never visit the host before the allocation: the greedy runs on the GPU
                # behind the probes, and widths and sensitivities come back in one copy afterwards
                self.refresh_bits_on_device(torch.stack(sens).float())
            else:
                if sens:
                    values = torch.stack([v.double() for v in sens]).tolist()
                    for l, v in zip(layers, values):
                        self.C[l] = SENSITIVITY_CAP if v >= SENSITIVITY_CAP else v
                self.refresh_bits()

        if adapting and self.debug:
            # the variance model against a measurement: gradient at the allocated widths vs uncompressed
            noisy = self._get_grad(backprop)
            allocated = dict(self.quantizer.bits)
            self.quantizer.bits = {l: 32 for l in allocated}
            exact = self._get_grad(backprop)
            print('Exact Variance %f, Predicted Variance %f'
                  % (_sq_dist(noisy, exact).item(), self._predicted_variance(1).item()))
            for b in (4,):
                self.quantizer.bits = {l: b for l in allocated}
                uniform = self._get_grad(backprop)
                model_var = (np.array(list(self.C.values())) * 2 ** (-2.0 * (b - 1))).sum()
                print('use %d bit to compare, exact variance %f, predicted variance %f'
                      % (b, _sq_dist(uniform, exact).item(), model_var.item()))
            self.quantizer.bits = self.bits.copy()

        if self.log_iter > 0 and self.iter % self.log_iter == 0:
            g = self._get_grad(backprop)
            m = self.momentum
            self.beta1 = self.beta1 * m + 1 - m
            self.batch_grad = self.batch_grad * m + (1 - m) * g
            self.grad_var = self.grad_var * m + (1 - m) * _sq_dist(self.batch_grad / self.beta1, g)
            self._record_state()

        self.iter += 1

    def _allocates_on_device(self, layers, sens):
        """config.device_calc_precision, and the probes cover the dims table in its order on a GPU (they do
        whenever the quantizer's tables come from one first iteration) with few enough tensors for one launch."""
        return (config.device_calc_precision and sens[0].is_cuda and layers == list(self.dims)
                and len(layers) <= DEVICE_CALC_PRECISION_MAX_TENSORS)

    def refresh_bits(self):
        """Greedy allocation from the current sensitivities: every tensor starts at max_bits, tensors are
        listed in the order of the dims table (gact/gact/autoprec.py:188-209)."""
        order = list(self.dims)
        start = torch.full((len(self.bits),), self.max_bits, dtype=torch.int32)
        chosen = ext_calc_precision.calc_precision(start,
                                                   torch.tensor([self.C[l] for l in order], dtype=torch.float),
                                                   torch.tensor([self.dims[l] for l in order], dtype=torch.int64),
                                                   self.total_bits)
        self._adopt_bits(order, chosen.tolist())

    def refresh_bits_on_device(self, C_dev):
        """The same allocation (calc_precision.cc:66-118) by the device kernel, from sensitivities that are still
        on the GPU: float32[len(dims)] in the order of the dims table.  One read-back, after the launch, brings
        the widths (and the sensitivities, for the log and the variance model) to the host."""
        order = list(self.dims)
        dev = C_dev.device
        start = torch.full((len(order),), self.max_bits, dtype=torch.int32, device=dev)
        if getattr(self, "_dims_dev", None) is None or self._dims_dev.device != dev or self._dims_dev.numel() != len(order):
            self._dims_dev = torch.tensor([self.dims[l] for l in order], dtype=torch.int64, device=dev)
        status = torch.zeros((1,), dtype=torch.int32, device=dev)
        ext_calc_precision.calc_precision_device(start, C_dev.contiguous(), self._dims_dev, self.total_bits, status)
        back = torch.cat([start.double(), status.double(), C_dev.double()]).tolist()
        L = len(order)
        if int(back[L]) != 0:
            raise RuntimeError("calc_precision on the device failed with status %d" % int(back[L]))
        for l, v in zip(order, back[L + 1:]):
            self.C[l] = SENSITIVITY_CAP if v >= SENSITIVITY_CAP else v
        self._adopt_bits(order, [int(b) for b in back[:L]])

    def _adopt_bits(self, order, chosen):
        for l, b in zip(order, chosen):
            self.bits[l] = b
        self.quantizer.bits = self.bits.copy()

        if self.log_iter > 0 and self.iter > self.warmpup_iter:
            overall_var = self.grad_var / self.beta1
            quantization_var = self._predicted_variance(0)
            if quantization_var > overall_var * 0.1:
                print('GACT Warning: Quantization variance is too large. Consider increasing number of bits.',
                      quantization_var, overall_var)
                self._record_state(**{"warning": True, "quantization var": float(quantization_var),
                                      "overall var": float(overall_var)})
