"""Host-side checks that need no GPU: the C-ABI library loads and exports every entry point the header
declares, status codes and sizes, and the Python faces raise the reference's errors for bad arguments."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import gact
from gact import ops
from gact.conf import config, set_optimization_level
from gact.controller import default_bit_for
from gact.cpp_extension import _abi
from gact.cpp_extension import minimax as ext_minimax
from gact.cpp_extension import quantization as ext_quantization

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gact_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gact_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 15
    lib = ctypes.CDLL(_abi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), "libgact_hip.so does not export %s" % n
    # and the Python binding covers exactly the header
    assert sorted(_abi.SIGNATURES) == names


def test_struct_layout_matches_the_header():
    assert ctypes.sizeof(_abi.BatchEntry) == 56


def test_status_codes_and_sizes():
    L = _abi.lib()
    assert L.gact_abi_version() == 7
    assert L.gact_strerror(0) == b"ok"
    for code in (-1, -2, -3, -4, -5):
        assert L.gact_strerror(code) not in (b"ok", b"unknown error")
    # b=2, N=5 -> 8 groups -> 512 bytes (+1 allocated by the reference)
    assert L.gact_packed_bytes(2, 5, 1, 256) == 512
    assert ext_quantization.packed_numel(2, 5, 1, 256) == 513
    assert L.gact_packed_bytes(4, 401408, 1, 256) == 51380224
    assert L.gact_packed_bytes(1, 169343, 1, 256) == 5419008
    assert L.gact_packed_bytes(3, 8, 1, 256) == -1


def test_entry_points_reject_bad_arguments_before_touching_the_gpu():
    L = _abi.lib()
    assert L.gact_quantize(None, 0, 256, 3, 0, 0, None, None, None, None, None, None) == -1      # bits
    assert L.gact_quantize(None, 7, 256, 2, 0, 0, None, None, None, None, None, None) == -1      # dtype
    assert L.gact_quantize(None, 0, 256, 2, 9, 0, None, None, None, None, None, None) == -1      # noise mode
    assert L.gact_quantize(None, 0, 256, 2, 0, 0, None, None, None, None, None, None) == -1      # null pointers
    assert L.gact_quantize(None, 0, 0, 2, 0, 0, None, None, None, None, None, None) == 0         # empty: nothing to do
    assert L.gact_quantize(8, 0, 256, 2, 0, 0, None, 16, 16, 16, None, None) == -2               # misaligned x
    assert L.gact_quantize_seeded(16, 0, 256, 2, 0, 0, 4, None, 16, 16, 16, None, None) == -2   # misaligned seed word
    assert L.gact_dequantize(16, 5, 16, 16, 0, 256, 16, None) == -1
    assert L.gact_minimax(16, 0, 4, 48, 16, 16, None) == -3                                      # D % 32 != 0
    assert L.gact_minimax(16, 0, 4, 32, 16, 16, None) == -3                                      # D > 32
    assert L.gact_pack(16, 16, 16, 0, 5, 4, 1, 256, 0, 0, None, 16, 16, None) == -1
    assert L.gact_unpack(16, 5, 16, 16, 0, 4, 1, 256, 16, None) == -1
    assert L.gact_mask_pack(None, -1, None, None) == -1
    assert L.gact_calc_precision_device(16, 16, 16, 5000, 1.0, None, None) == -3                 # beyond the LDS table
    assert L.gact_quantize_batched(16, 16, 3, 3, 1, 3, 16, 16, 16, 16, None) == -1               # injected noise
    assert L.gact_quantize_batched(16, 16, 3, 3, 0, 8, 16, 16, 16, 16, None) == -1               # dtype mask
    assert L.gact_quantize_batched(16, 16, 3, 3, 0, 3, 8, 16, 16, 16, None) == -2                # misaligned workspace
    assert L.gact_batch_plan(16, 16, 3, 3, -1, 16, None) == -1                                   # negative capacity
    assert L.gact_batch_plan(16, 16, 3, 3, 100, None, None) == -1                                # no workspace
    # header (32 int64) + one int32 per block, in whole 16-byte pieces
    assert L.gact_batch_workspace_bytes(3, 5) == 256 + 2 * 16
    assert L.gact_quantize_batched_static(16, 16, 10, 262145, 1 << 20, 3, 0, 16, 16, 16, None, None) == -6   # beyond its array
    assert L.gact_batch_workspace_bytes(-1, 5) == -1
    assert L.gact_quantize(16, 3, 256, 4, 0, 0, None, 16, 16, 16, None, None) == -1               # element type
    assert L.gact_quantize(0, 2, 256, 4, 0, 0, None, 16, 16, 16, None, None) == -1                # bfloat16, null data
    assert L.gact_minimax(16, 2, 4, 64, 16, 16, None) == -1                                      # no bfloat16 here


def test_python_faces_raise_the_reference_errors():
    x = torch.randn(4, 1, 256)
    mn = x.amin(dim=2, keepdim=True)
    mx = x.amax(dim=2, keepdim=True)
    with pytest.raises(RuntimeError, match="data must be a CUDA tensor!"):
        ext_quantization.pack_single_precision(x, mn, mx, 2, True, 0)
    with pytest.raises(RuntimeError, match="data must be a CUDA tensor!"):
        ext_minimax.minimax(x.reshape(4, 256))
    with pytest.raises(RuntimeError, match="data must be a CUDA tensor!"):
        ext_quantization.unpack_single_precision(torch.zeros(10, dtype=torch.int8), 2, mn, mn, 4, 1, 256)
    with pytest.raises(RuntimeError, match="data must be a CUDA tensor!"):
        ext_quantization.act_quantize_dropout_mask(torch.zeros(10, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="data must be a CUDA tensor!"):
        ops.op_quantize(x, 2, 0)
    with pytest.raises(RuntimeError, match="8 % bits == 0"):
        ext_quantization._check_bits(3)
    with pytest.raises(TypeError):
        ext_quantization._seed_u64(1 << 40)          # the binding takes a C int
    assert ext_quantization._seed_u64(-1) == 0xFFFFFFFFFFFFFFFF   # and sign-extends it to uint64_t


def test_32_bit_passthrough_needs_no_kernel():
    # gact/gact/ops.py:21-24,39-40 and tests/test_act_quantized_ops.py:73-91 of the reference
    x = torch.rand(7, 100)
    q = ops.op_quantize(x, 32, 0)
    q_input, q_bit, q_scale, q_min = q
    groups = torch.cat([x.reshape(-1), torch.zeros(3 * 256 - 700)]).reshape(3, 256)
    assert q_bit == 32 and torch.equal(q_input, groups)
    assert torch.equal(q_min.reshape(-1), groups.min(dim=1).values)
    assert torch.equal(q_scale.reshape(-1), groups.max(dim=1).values - groups.min(dim=1).values)
    assert torch.equal(ops.op_dequantize(q, x.shape), x)


def test_dequantize_rejects_non_int_bits():
    with pytest.raises(AssertionError):
        ops.op_dequantize([torch.zeros(1), 2.0, torch.zeros(1), torch.zeros(1)], (1,))


def test_config_levels_and_default_bits():
    saved = dict(vars(config))
    try:
        assert config.group_size == 256 and config.max_bit == 32 and config.adapt_interval == 1000
        expect = {"L1": (False, 4), "L1.1": (False, 8), "L1.2": (False, 2), "L2": (True, 4), "L2.1": (True, 3),
                  "L2.2": (True, 2)}
        for level, (auto, bit) in expect.items():
            set_optimization_level(level)
            assert (config.auto_prec, config.bit) == (auto, bit)
        set_optimization_level("L3")
        assert config.swap and config.prefetch and config.bit == 4
        set_optimization_level("L0")
        assert not config.compress_activation
        with pytest.raises(ValueError):
            set_optimization_level("L9")
        # gact/gact/controller.py:13-23
        assert [default_bit_for(b) for b in (2, 3, 4, 5, 8, 16)] == [2, 4, 4, 8, 8, 8]
    finally:
        vars(config).update(saved)
    assert gact.config is config
