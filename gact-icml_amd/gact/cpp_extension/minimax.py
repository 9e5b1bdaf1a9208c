"""``gact.cpp_extension.minimax`` of the reference (gact/gact/cpp_extension/minimax.cc:7-14)."""
import torch

from . import _abi


def _check_cuda_float(t, name):
    # CHECK_CUDA_TENSOR_FLOAT, gact/gact/cpp_extension/ext_common.h:15-19
    if not t.is_cuda:
        raise RuntimeError(name + " must be a CUDA tensor!")
    if not t.is_contiguous():
        raise RuntimeError(name + " must be contiguous!")
    if t.dtype not in (torch.float32, torch.float16):
        raise RuntimeError("The type of " + name + " is not correct!")


def minimax(data):
    """Per-row (min, max) of a contiguous [N, D] float32/float16 tensor on the GPU."""
    _check_cuda_float(data, "data")
    if data.dim() != 2:
        raise RuntimeError("The dimension of data is not correct!")
    N, D = data.shape
    if not (D % 32 == 0 and D > 32):  # minimax_cuda_kernel.cu:80
        raise RuntimeError("Expected D % 32 == 0 && D > 32 to be true, but got false.")
    mn = torch.empty((N,), dtype=data.dtype, device=data.device)
    mx = torch.empty((N,), dtype=data.dtype, device=data.device)
    with torch.cuda.device(data.device):
        _abi.check(_abi.lib().gact_minimax(data.data_ptr(), _abi.dtype_code(data.dtype), N, D, mn.data_ptr(),
                                           mx.data_ptr(), _abi.stream_of(data)))
    return mn, mx
