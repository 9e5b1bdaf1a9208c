"""``gact.cpp_extension.quantization`` of the reference (gact/gact/cpp_extension/quantization.cc:26-69).

Same four functions, same argument order, same shapes and dtypes of the results, same argument
checks (raised as RuntimeError, like TORCH_CHECK).  Additions are keyword-only and optional.
"""
import torch

from . import _abi

_INT32_MIN, _INT32_MAX = -(1 << 31), (1 << 31) - 1


def _check_cuda(t, name):
    if not t.is_cuda:
        raise RuntimeError(name + " must be a CUDA tensor!")
    if not t.is_contiguous():
        raise RuntimeError(name + " must be contiguous!")


def _check_cuda_dim_float(t, name, dim):
    # CHECK_CUDA_TENSOR_DIM_FLOAT, gact/gact/cpp_extension/ext_common.h:22-27
    _check_cuda(t, name)
    if t.dim() != dim:
        raise RuntimeError("The dimension of " + name + " is not correct!")
    if t.dtype not in (torch.float32, torch.float16):
        raise RuntimeError("The type of " + name + " is not correct!")


def _check_bits(bits):
    # TORCH_CHECK(8 % bits == 0), quantization_cuda_kernel.cu:86,191
    if not isinstance(bits, int) or isinstance(bits, bool):
        raise TypeError("bits must be an int")
    if bits <= 0 or 8 % bits != 0:
        raise RuntimeError("Expected 8 % bits == 0 to be true, but got false.")


def _noise_mode(noise, stream):
    if noise is not None:
        return _abi.NOISE_INJECT
    if stream is None:
        from ..conf import config
        stream = config.rng_stream
    try:
        return _abi.NOISE_MODES[stream]
    except KeyError:
        raise RuntimeError("unknown rng_stream %r (expected one of %s)" % (stream, sorted(_abi.NOISE_MODES)))


def _seed_u64(seed):
    # the binding takes `int seed` and widens it to uint64_t (quantization.cc:55,60): sign extension
    if not isinstance(seed, int) or isinstance(seed, bool):
        raise TypeError("seed must be an int")
    if not (_INT32_MIN <= seed <= _INT32_MAX):
        raise TypeError("seed does not fit a C int")
    return seed & 0xFFFFFFFFFFFFFFFF


def packed_numel(bits, N, G, D):
    """Length of the int8 tensor pack_single_precision returns: (total_bits + 8) / 8, one byte more
    than is ever written (quantization_cuda_kernel.cu:88-91)."""
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt
    return (bits * n_round * G * D + 8) // 8


def pack_single_precision(data, min, max, bits, stochastic, seed, *, noise=None, rng_stream=None):
    """Quantize data[N,G,D] against min/max[N,G,1] to `bits` bits -> (packed int8, scale[N,G,1]).

    `stochastic` is accepted and ignored, exactly as in the reference, whose kernel always adds the
    rounding noise (quantization_cuda_kernel.cu:65-66).  `noise` (float32, same number of elements as
    data) injects the uniforms instead of drawing them; `rng_stream` overrides gact.conf.config.rng_stream.
    """
    _check_cuda_dim_float(data, "data", 3)
    _check_cuda_dim_float(min, "min", 3)
    _check_cuda_dim_float(max, "max", 3)
    _check_bits(bits)
    seed = _seed_u64(seed)
    if min.dtype != data.dtype or max.dtype != data.dtype:
        raise RuntimeError("expected scalar type of min/max to match data")
    N, G, D = data.shape
    if min.numel() != N * G or max.numel() != N * G:
        raise RuntimeError("min/max must hold one value per (row, group)")
    mode = _noise_mode(noise, rng_stream)
    if noise is not None:
        _check_cuda(noise, "noise")
        if noise.dtype != torch.float32 or noise.numel() != data.numel():
            raise RuntimeError("noise must be float32 with one value per element of data")
    packed = torch.empty((packed_numel(bits, N, G, D),), dtype=torch.int8, device=data.device)
    scale = torch.empty((N, G, 1), dtype=data.dtype, device=data.device)
    with torch.cuda.device(data.device):
        _abi.check(_abi.lib().gact_pack(data.data_ptr(), min.data_ptr(), max.data_ptr(), _abi.dtype_code(data.dtype),
                                        bits, N, G, D, mode, seed, _abi.ptr(noise), packed.data_ptr(),
                                        scale.data_ptr(), _abi.stream_of(data)))
    return packed, scale


def unpack_single_precision(data, bits, scale, min, N, num_groups, group_size):
    """Inverse of pack_single_precision -> [N, num_groups, group_size] of scale.dtype."""
    # CHECK_CUDA_TENSOR_DIM_TYPE(data, 1, kInt8), quantization.cc:43
    _check_cuda(data, "data")
    if data.dim() != 1:
        raise RuntimeError("The dimension of data is not correct!")
    if data.dtype != torch.int8:
        raise RuntimeError("The type of data is not correct!")
    _check_cuda_dim_float(scale, "scale", 3)
    _check_cuda_dim_float(min, "min", 3)
    _check_bits(bits)
    N, G, D = int(N), int(num_groups), int(group_size)
    if min.dtype != scale.dtype:
        raise RuntimeError("expected scalar type of min to match scale")
    need = packed_numel(bits, N, G, D) - 1
    if data.numel() < need or scale.numel() < N * G or min.numel() < N * G:
        raise RuntimeError("packed data / scale / min are too short for N=%d, num_groups=%d, group_size=%d" % (N, G, D))
    out = torch.empty((N, G, D), dtype=scale.dtype, device=data.device)
    with torch.cuda.device(data.device):
        _abi.check(_abi.lib().gact_unpack(data.data_ptr(), bits, scale.data_ptr(), min.data_ptr(),
                                          _abi.dtype_code(scale.dtype), N, G, D, out.data_ptr(),
                                          _abi.stream_of(data)))
    return out


def act_quantize_dropout_mask(data):
    """uint8 0/1 mask of any shape -> int32[ceil(n/32)] bit mask."""
    # CHECK_CUDA_TENSOR_TYPE(data, kUInt8), quantization.cc:27
    _check_cuda(data, "data")
    if data.dtype != torch.uint8:
        raise RuntimeError("The type of data is not correct!")
    n = data.numel()
    mask = torch.empty(((n + 31) // 32,), dtype=torch.int32, device=data.device)
    with torch.cuda.device(data.device):
        _abi.check(_abi.lib().gact_mask_pack(data.data_ptr(), n, mask.data_ptr(), _abi.stream_of(data)))
    return mask


def act_dequantize_dropout_mask(mask, N):
    """int32 bit mask -> uint8[N] of 0/1."""
    N = int(N)
    if not mask.is_cuda:
        raise RuntimeError("mask must be a CUDA tensor!")
    if mask.dtype != torch.int32 or mask.numel() < (N + 31) // 32:
        raise RuntimeError("mask must be int32 with ceil(N/32) words")
    out = torch.empty((N,), dtype=torch.uint8, device=mask.device)
    with torch.cuda.device(mask.device):
        _abi.check(_abi.lib().gact_mask_unpack(mask.data_ptr(), N, out.data_ptr(), _abi.stream_of(mask)))
    return out
