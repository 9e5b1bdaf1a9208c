"""Adaptive per-tensor widths: estimate each saved tensor's sensitivity from gradient differences, then
allocate widths greedily under an average-bits budget.  Mirrors gact/gact/autoprec.py of the reference."""
import os
import random

import numpy as np
import torch
import torch.nn as nn

from .cpp_extension import calc_precision as ext_calc_precision
from .utils import exp_recorder


class AutoPrecision:
    def __init__(self, model, quantizer, bits, max_bits, work_dir, adapt_interval, log_interval,
                 momentum=0.99, warmup_iter=100, debug=False):
        self.model = model
        self.quantizer = quantizer
        self.debug = debug

        self.dims = None
        self.bits = {}   # width per tensor id
        self.C = {}      # sensitivity per tensor id

        self.avg_bits = bits
        self.max_bits = max_bits

        # running estimate of the gradient variance, used for the "variance too large" warning
        self.momentum = momentum
        self.warmpup_iter = warmup_iter
        self.beta1 = 1e-7
        self.batch_grad = 0
        self.grad_var = 0
        self.adapt_interval = adapt_interval

        self.iter = 0
        self.log_iter = log_interval
        self.work_dir = work_dir

    def init_from_dims(self):
        """gact/gact/autoprec.py:39-46."""
        self.dims = self.quantizer.dims
        total_ele = 0
        for l in self.dims:
            self.C[l] = 1.0
            self.bits[l] = self.avg_bits
            total_ele += self.dims[l]
        self.total_bits = self.avg_bits * total_ele

    def iterate_wrapper(self, backprop):
        if self.dims is None:
            self.init_from_dims()
        self.iterate(backprop)

    # ---- helpers of iterate() ----
    def _sample_grad(self):
        return torch.cat([p.grad.ravel() for p in self.model.parameters() if p.grad is not None], 0)

    @staticmethod
    def _setup_seed(seed):
        random.seed(seed)
        np.random.seed(seed)
        torch.manual_seed(seed)
        if torch.cuda.is_available():
            torch.cuda.manual_seed_all(seed)

    @staticmethod
    def _batch_norms(model):
        return [m for m in model.modules() if isinstance(m, (nn.BatchNorm1d, nn.BatchNorm2d, nn.BatchNorm3d))]

    def _get_grad(self, backprop):
        """One extra forward + backward under a fixed seed, leaving running statistics and the global RNG
        untouched.  gact/gact/autoprec.py:80-100."""
        bns = self._batch_norms(self.model)
        for bn in bns:
            bn.track_running_stats = False
        state = torch.get_rng_state().clone()
        self._setup_seed(self.iter)
        backprop()
        torch.set_rng_state(state)
        for bn in bns:
            bn.track_running_stats = True
        grad = self._sample_grad()
        self.quantizer.iterate()
        return grad

    def iterate(self, backprop):
        """gact/gact/autoprec.py:57-186."""
        if self.iter % self.adapt_interval == 0:
            print('GACT: Initializing AutoPrec..., run extra %d iters' % (len(self.quantizer.bits)))
            for l in self.quantizer.bits:
                b = self.quantizer.bits[l]
                # the same tensor at 1 bit with two seeds, and at 8 bits
                self.quantizer.bits[l] = 1
                grad0 = self._get_grad(backprop)
                self.quantizer.seeds[l] += 1
                grad1 = self._get_grad(backprop)
                self.quantizer.seeds[l] -= 1
                self.quantizer.bits[l] = 8
                grad2 = self._get_grad(backprop)
                diff01 = ((grad0 - grad1) ** 2).sum()
                diff02 = ((grad0 - grad2) ** 2).sum()
                diff12 = ((grad1 - grad2) ** 2).sum()
                sens = max(diff01, max(diff02, diff12) * 2)
                del grad0, grad1, grad2
                if torch.isnan(sens) or torch.isinf(sens) or sens > 1e10:
                    self.C[l] = 1e10
                else:
                    self.C[l] = sens.item()
                self.quantizer.bits[l] = b
            self.refresh_bits()

        if self.debug and self.iter % self.adapt_interval == 0:
            grad = self._get_grad(backprop)
            saved = dict(self.quantizer.bits)
            for l in self.quantizer.bits:
                self.quantizer.bits[l] = 32
            det_grad = self._get_grad(backprop)
            ap_var = ((grad - det_grad) ** 2).sum()
            predicted = (np.array([self.C[l] for l in self.C]) *
                         2 ** (-2.0 * (np.array([self.bits[l] for l in self.C]) - 1))).sum()
            print('Exact Variance %f, Predicted Variance %f' % (ap_var.item(), predicted.item()))
            self.quantizer.bits = saved

        if self.log_iter > 0 and self.iter % self.log_iter == 0:
            det_grad = self._get_grad(backprop)
            m = self.momentum
            self.beta1 = self.beta1 * m + 1 - m
            self.batch_grad = self.batch_grad * m + (1 - m) * det_grad
            bgrad = self.batch_grad / self.beta1
            gvar = ((bgrad - det_grad) ** 2).sum()
            self.grad_var = self.grad_var * m + (1 - m) * gvar
            exp_recorder.record("iter", self.iter)
            exp_recorder.record("layer sensitivity", self.C)
            exp_recorder.record("bits", self.bits)
            exp_recorder.record("dims", self.dims)
            os.makedirs(self.work_dir, exist_ok=True)
            exp_recorder.dump(os.path.join(self.work_dir, "autoprec.log"))

        self.iter += 1

    def refresh_bits(self):
        """Greedy allocation from the current sensitivities.  gact/gact/autoprec.py:188-209: every tensor
        starts at max_bits, the budget is avg_bits * total elements."""
        l_list = list(self.dims)
        dims_list = [self.dims[l] for l in l_list]
        C_list = [self.C[l] for l in l_list]

        bits_tensor = torch.ones(len(self.bits), dtype=torch.int32) * self.max_bits
        bits_tensor = ext_calc_precision.calc_precision(bits_tensor, torch.tensor(C_list, dtype=torch.float),
                                                        torch.tensor(dims_list, dtype=torch.int64), self.total_bits)
        for i, l in enumerate(l_list):
            self.bits[l] = bits_tensor[i].item()
        self.quantizer.bits = self.bits.copy()

        if self.log_iter > 0 and self.iter > self.warmpup_iter:
            overall_var = self.grad_var / self.beta1
            quantization_var = (np.array([self.C[l] for l in self.C]) *
                                2 ** (-2.0 * np.array([self.bits[l] for l in self.C]))).sum()
            if quantization_var > overall_var * 0.1:
                print('GACT Warning: Quantization variance is too large. Consider increasing number of bits.',
                      quantization_var, overall_var)
                exp_recorder.record("iter", self.iter)
                exp_recorder.record("layer sensitivity", self.C)
                exp_recorder.record("bits", self.bits)
                exp_recorder.record("dims", self.dims)
                exp_recorder.record("warning", True)
                exp_recorder.record("quantization var", float(quantization_var))
                exp_recorder.record("overall var", float(overall_var))
                os.makedirs(self.work_dir, exist_ok=True)
                exp_recorder.dump(os.path.join(self.work_dir, "autoprec.log"))
