"""Quantize / dequantize operators with the reference's names and return conventions
(gact/gact/ops.py:11-69), running on the fused HIP kernels.

``op_quantize`` reads the activation once: min/max, scale, stochastic rounding and packing happen in a
single kernel, and the zero padding to whole groups of 256 is done by the kernel's bounds handling
instead of a concatenated copy.  ``op_dequantize`` writes straight into a tensor of the original
shape.  The extension-style entry points (minimax, pack_single_precision, unpack_single_precision)
stay available in gact.cpp_extension for callers that use them directly.
"""
import math
import torch

from .conf import config
from .cpp_extension import _abi
from .cpp_extension import quantization as ext_quantization


# the raw HIP stream torch currently launches on for a device (what _abi.stream_of wraps), bound once: these two
# operators run once per saved tensor and iteration
_current_stream = torch._C._cuda_getCurrentRawStream


def _num_groups(numel):
    return (numel + config.group_size - 1) // config.group_size


def _fused():
    """The single-pass kernels are built for groups of 256; any other config.group_size takes the
    extension-style sequence minimax -> pack / unpack on the zero-padded tensor, as the reference does."""
    return config.group_size == _abi.GROUP


def _padded_groups(input):
    """gact/gact/ops.py:12-19: flatten, zero-pad to whole groups, [N, group_size]."""
    group = config.group_size
    pad = _num_groups(input.numel()) * group - input.numel()
    if pad > 0:
        input = torch.cat([input.reshape(1, -1), torch.zeros([1, pad], dtype=input.dtype, device=input.device)], dim=1)
    return input.reshape(-1, group)


def no_scheme_quantize_pack(input, q_bit, seed, *, noise=None, rng_stream=None, seed_offset=None):
    """gact/gact/ops.py:11-32 -> (q_input, q_scale, q_min).  `seed_offset` (one int64 on the GPU, optional) is added
    to `seed` when the kernel runs, for launches recorded in a HIP graph."""
    N = _num_groups(input.numel())
    if q_bit == 32:
        # the passthrough of ops.py:21-24: the padded [N, group] view itself, max - min, min
        input_groups = _padded_groups(input)
        q_min = input_groups.min(dim=-1, keepdim=True).values
        q_scale = input_groups.max(dim=-1, keepdim=True).values - q_min
        return input_groups, q_scale, q_min

    if not _fused():
        if seed_offset is not None:
            raise RuntimeError("seed_offset needs the single-pass kernels (config.group_size 256)")
        from .cpp_extension import minimax as ext_minimax
        input_groups = _padded_groups(input.contiguous()).contiguous()
        q_min, mx = ext_minimax.minimax(input_groups)
        q_input, q_scale = ext_quantization.pack_single_precision(
            input_groups.view(N, 1, -1), q_min.view(N, 1, 1), mx.view(N, 1, 1), q_bit, True, seed,
            noise=noise, rng_stream=rng_stream)
        return q_input, q_scale, q_min.view(N, 1, 1)

    if not input.is_cuda:
        raise RuntimeError("data must be a CUDA tensor!")
    dtype = input.dtype
    if dtype is not torch.float32 and dtype is not torch.float16 and dtype is not torch.bfloat16:
        raise RuntimeError("The type of data is not correct!")
    ext_quantization._check_bits(q_bit)
    seed = ext_quantization._seed_u64(seed)
    # the reference's reshape copies a non-contiguous input as well
    x = input if input.is_contiguous() else input.contiguous()
    if x.data_ptr() & 15:
        x = x.clone()
    if noise is None and rng_stream is None:
        mode = _abi.NOISE_MODES.get(config.rng_stream)
        if mode is None:
            mode = ext_quantization._noise_mode(None, None)      # raises, naming the streams there are
    else:
        mode = ext_quantization._noise_mode(noise, rng_stream)
        if noise is not None:
            if (not noise.is_cuda) or noise.dtype != torch.float32 or noise.numel() != N * config.group_size \
                    or not noise.is_contiguous():
                raise RuntimeError("noise must be a contiguous float32 CUDA tensor with one value per padded element")
    device = x.device
    q_input = torch.empty(ext_quantization.packed_numel(q_bit, N, 1, _abi.GROUP), dtype=torch.int8, device=device)
    # bfloat16 (not in the reference) is quantized as the float values it holds: float scale, bfloat16 min
    q_scale = torch.empty((N, 1, 1), dtype=torch.float32 if dtype is torch.bfloat16 else dtype, device=device)
    q_min = torch.empty((N, 1, 1), dtype=dtype, device=device)
    if seed_offset is None:
        _abi.call_on(device, _abi.lib().gact_quantize, x.data_ptr(), _abi.dtype_code(dtype),
                     x.numel(), q_bit, mode, seed, None if noise is None else noise.data_ptr(), q_input.data_ptr(),
                     q_scale.data_ptr(), q_min.data_ptr(), None, _current_stream(device.index))
    else:
        if seed_offset.dtype is not torch.int64 or seed_offset.numel() != 1 or seed_offset.device != device:
            raise RuntimeError("seed_offset must be one int64 on the device of the data")
        _abi.call_on(device, _abi.lib().gact_quantize_seeded, x.data_ptr(), _abi.dtype_code(dtype),
                     x.numel(), q_bit, mode, seed, seed_offset.data_ptr(), None if noise is None else noise.data_ptr(),
                     q_input.data_ptr(), q_scale.data_ptr(), q_min.data_ptr(), None, _current_stream(device.index))
    return q_input, q_scale, q_min


def dequantize_and_unpack(data, shape, q_bit, scale, mn):
    """gact/gact/ops.py:34-47 -> [num_groups, 1, group_size] tensor (the padded groups)."""
    if not isinstance(q_bit, int):
        print("bits must be intergers, now bits ", q_bit)
        assert(False)

    if q_bit == 32:
        return data

    group_size = config.group_size
    num_groups = (math.prod(shape) + group_size - 1) // group_size
    return ext_quantization.unpack_single_precision(data, q_bit, scale, mn, num_groups, 1, group_size)


def op_quantize_mask(input):
    """gact/gact/ops.py:49-50.  The mask kernel reads 16 bytes per lane: a contiguous view that starts at
    an odd storage offset (a slice, a chunk) is copied to a fresh allocation first, as the float path does
    (the reference's kernel takes any alignment)."""
    data = input.contiguous()
    if not _abi.aligned(data):
        data = data.clone()
    return [ext_quantization.act_quantize_dropout_mask(data), input.shape]


def op_dequantize_mask(input):
    """gact/gact/ops.py:52-55."""
    q_mask, input_shape = input
    output = ext_quantization.act_dequantize_dropout_mask(q_mask, math.prod(input_shape)).reshape(input_shape)
    return output


def op_quantize(input, q_bit, seed, *, noise=None, rng_stream=None, seed_offset=None):
    """gact/gact/ops.py:57-59 -> [q_input, q_bit, q_scale, q_min]."""
    q_input, q_scale, q_min = no_scheme_quantize_pack(input, q_bit, seed, noise=noise, rng_stream=rng_stream,
                                                      seed_offset=seed_offset)
    return [q_input, q_bit, q_scale, q_min]


def op_dequantize(input, input_shape):
    """gact/gact/ops.py:61-69 -> tensor of `input_shape`, contiguous, dtype of the scale."""
    q_input, q_bit, q_scale, q_min = input
    if not isinstance(q_bit, int):
        print("bits must be intergers, now bits ", q_bit)
        assert(False)
    num_features = math.prod(input_shape)
    if q_bit == 32:
        return q_input.ravel()[:num_features].reshape(*input_shape).contiguous()

    if not _fused():
        groups = dequantize_and_unpack(q_input, input_shape, q_bit, q_scale, q_min)
        return groups.ravel()[:num_features].reshape(*input_shape).contiguous()

    ext_quantization._check_bits(q_bit)
    if not q_input.is_cuda:
        raise RuntimeError("data must be a CUDA tensor!")
    if q_input.dtype is not torch.int8 or q_input.dim() != 1:
        raise RuntimeError("The type of data is not correct!")
    N = _num_groups(num_features)
    if q_input.numel() < ext_quantization.packed_numel(q_bit, N, 1, _abi.GROUP) - 1 \
            or q_scale.numel() < N or q_min.numel() < N:
        raise RuntimeError("packed data / scale / min are too short for shape %s" % (tuple(input_shape),))
    dtype = q_min.dtype      # the scale's type as well, except for bfloat16 tensors, whose scale is float
    if q_scale.dtype is not (torch.float32 if dtype is torch.bfloat16 else dtype):
        raise RuntimeError("expected scalar type of min to match scale")
    device = q_input.device
    out = torch.empty(tuple(input_shape), dtype=dtype, device=device)
    _abi.call_on(device, _abi.lib().gact_dequantize, q_input.data_ptr(), q_bit, q_scale.data_ptr(), q_min.data_ptr(),
                 _abi.dtype_code(dtype), num_features, out.data_ptr(), _current_stream(device.index))
    return out
