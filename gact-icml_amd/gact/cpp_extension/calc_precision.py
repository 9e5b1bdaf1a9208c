"""``gact.cpp_extension.calc_precision`` of the reference (gact/gact/cpp_extension/calc_precision.cc:66-123)."""
import torch

from . import _abi


def _check_cpu(t, name):
    if t.device.type != "cpu":
        raise RuntimeError(name + " must be a CPU tensor!")
    if not t.is_contiguous():
        raise RuntimeError(name + " must be contiguous!")


def calc_precision(b, C, w, target):
    """Greedy bit allocation on CPU tensors: b int32[L] (updated in place and returned), C float32[L]
    sensitivities, w int64[L] element counts, target = total bit budget."""
    _check_cpu(b, "b")
    _check_cpu(C, "C")
    _check_cpu(w, "w")
    if b.dtype != torch.int32 or C.dtype != torch.float32 or w.dtype != torch.int64:
        raise RuntimeError("expected b int32, C float32, w int64")
    L = b.numel()
    if C.numel() < L or w.numel() < L:
        raise RuntimeError("C and w must hold one value per entry of b")
    _abi.check(_abi.lib().gact_calc_precision(b.data_ptr(), C.data_ptr(), w.data_ptr(), L, float(target)))
    return b


def calc_precision_device(b, C, w, target, status=None):
    """The same allocation on device tensors, without leaving the GPU (no counterpart in the reference)."""
    for t, name in ((b, "b"), (C, "C"), (w, "w")):
        if not t.is_cuda:
            raise RuntimeError(name + " must be a CUDA tensor!")
        if not t.is_contiguous():
            raise RuntimeError(name + " must be contiguous!")
    if b.dtype != torch.int32 or C.dtype != torch.float32 or w.dtype != torch.int64:
        raise RuntimeError("expected b int32, C float32, w int64")
    with torch.cuda.device(b.device):
        _abi.check(_abi.lib().gact_calc_precision_device(b.data_ptr(), C.data_ptr(), w.data_ptr(), b.numel(),
                                                         float(target), _abi.ptr(status), _abi.stream_of(b)))
    return b
