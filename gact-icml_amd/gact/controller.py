"""User-facing driver: installs the saved-tensor hooks and advances the per-iteration state.
Mirrors gact/gact/controller.py of the reference (same constructor, same methods)."""
import torch

from .autoprec import AutoPrecision
from .conf import config
from .quantizer import Quantizer


def default_bit_for(bit):
    """Width used before auto precision has run: 2 stays 2, up to 4 -> 4, anything wider -> 8
    (gact/gact/controller.py:13-23)."""
    assert 1 < bit <= 16
    if bit == 2:
        return 2
    if bit <= 4:
        return 4
    return 8


class Controller:
    def __init__(self, model):
        if not config.compress_activation:
            return
        self.model = model
        self.quantizer = Quantizer(default_bit=default_bit_for(config.bit), swap=config.swap,
                                   prefetch=config.prefetch)
        self.quantizer.filter_tensors(model.named_parameters())   # parameters are never compressed

        self.auto_prec = config.auto_prec
        if self.auto_prec:
            self.ap = AutoPrecision(self.model, self.quantizer, config.bit, config.max_bit, config.work_dir,
                                    config.adapt_interval, config.log_interval)
        self.bit = config.bit
        self.iter = 0
        self._hooked = False

    def __del__(self):
        try:
            self.uninstall_hook()
        except Exception:
            pass

    def install_hook(self):
        def pack_hook(x):
            return self.quantize(x)

        def unpack_hook(x):
            return self.dequantize(x)

        torch._C._autograd._push_saved_tensors_default_hooks(pack_hook, unpack_hook)
        self._hooked = True

    def uninstall_hook(self):
        if getattr(self, "_hooked", False):
            torch._C._autograd._pop_saved_tensors_default_hooks()
            self._hooked = False

    def iterate(self, get_grad):
        """Call once per training iteration, after the optimizer step.  `get_grad` runs one forward +
        backward pass; auto precision calls it when it refreshes the sensitivities."""
        if not config.compress_activation:
            return
        self.quantizer.iterate()
        if self.auto_prec:
            self.ap.iterate_wrapper(get_grad)
        self.iter += 1
        self.quantizer.seed_iter = self.iter

    def quantize(self, input):
        if not config.compress_activation:
            if config.swap:
                host = torch.empty(input.shape, dtype=input.dtype, device='cpu', pin_memory=True)
                host.copy_(input, non_blocking=True)
                return host
            return input
        return self.quantizer.quantize(input)

    def dequantize(self, input):
        if not config.compress_activation:
            if config.swap:
                input = input.cuda(non_blocking=True)
            return input
        return self.quantizer.dequantize(input)
