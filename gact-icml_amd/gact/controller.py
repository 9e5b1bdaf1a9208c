"""The object a training script holds: it installs the saved-tensor hooks and advances the per-iteration
state of the quantizer and of auto precision.  Same constructor and methods as gact/gact/controller.py of
the reference; also usable as a context manager (`with Controller(model) as c:` installs and removes the
hooks).
"""
import bisect

import torch

from .autoprec import AutoPrecision
from .conf import config
from .quantizer import Quantizer

_hooks = torch._C._autograd


def default_bit_for(bit):
    """Width used until auto precision has allocated widths: the next of 2, 4, 8 at or above the average
    (gact/gact/controller.py:13-23: 2 -> 2, 3..4 -> 4, 5..16 -> 8)."""
    assert 1 < bit <= 16
    steps = (2, 4, 8)
    return steps[min(bisect.bisect_left(steps, bit), 2)]


def _to_pinned_host(t):
    host = torch.empty(t.shape, dtype=t.dtype, device='cpu', pin_memory=True)
    host.copy_(t, non_blocking=True)
    return host


class Controller:
    def __init__(self, model):
        self._hooked = False
        if not config.compress_activation:
            return      # hooks still work: they pass tensors through (or swap them when config.swap is set)
        self.model = model
        self.bit = config.bit
        self.iter = 0
        self.quantizer = Quantizer(default_bit=default_bit_for(config.bit), swap=config.swap,
                                   prefetch=config.prefetch)
        # parameters are saved for backward too, and must stay exact; buffers (running statistics, constant
        # masks) live as long as the model, so a packed copy of one would only add memory
        self.quantizer.filter_tensors(model.named_parameters())
        self.quantizer.filter_tensors(model.named_buffers())
        self.auto_prec = config.auto_prec
        if self.auto_prec:
            self.ap = AutoPrecision(model, self.quantizer, config.bit, config.max_bit, config.work_dir,
                                    config.adapt_interval, config.log_interval)

    # ---- hooks (controller.py:53-60 of the reference: the default saved-tensor hooks of autograd) ----
    def install_hook(self):
        _hooks._push_saved_tensors_default_hooks(self.quantize, self.dequantize)
        self._hooked = True

    def uninstall_hook(self):
        if getattr(self, "_hooked", False):
            _hooks._pop_saved_tensors_default_hooks()
            self._hooked = False

    def __enter__(self):
        self.install_hook()
        return self

    def __exit__(self, *exc):
        self.uninstall_hook()
        return False

    def __del__(self):
        try:
            self.uninstall_hook()
        except Exception:
            pass

    # ---- what the hooks do ----
    def quantize(self, input):
        if config.compress_activation:
            return self.quantizer.quantize(input)
        return _to_pinned_host(input) if config.swap else input

    def dequantize(self, input):
        if config.compress_activation:
            return self.quantizer.dequantize(input)
        return input.cuda(non_blocking=True) if config.swap else input

    # ---- once per training iteration, after the optimizer step ----
    def iterate(self, get_grad):
        """`get_grad` runs one forward + backward pass; auto precision calls it when it re-measures the
        sensitivities.  Order as in controller.py:74-78: reset the quantizer, let auto precision run, then
        move the seed offset to the new iteration."""
        if not config.compress_activation:
            return
        self.quantizer.iterate()
        if self.auto_prec:
            self.ap.iterate_wrapper(get_grad)
        self.iter += 1
        self.quantizer.seed_iter = self.iter
