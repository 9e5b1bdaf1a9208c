"""The compute-free traffic probes bench.py times beside the kernels (gact-icml_amd/csrc/stream_probe.hip): they must move
exactly the bytes they are priced with - whole tiles only, nothing past them."""
import os
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
import bench  # noqa: E402


@pytest.mark.parametrize("in_kb,out_dw", [(8, 1), (8, 2), (8, 4), (8, 8), (4, 1), (4, 2), (4, 4), (4, 8)])
def test_quantize_like_probe_writes_its_tiles_and_nothing_else(in_kb, out_dw):
    probe = bench.probe_lib()
    tiles = 37
    nbytes = tiles * in_kb * 1024 + 700                      # a ragged end: the last 700 bytes belong to no tile
    src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda")
    dst = torch.full((tiles * 256 * out_dw + 512,), 0xA5, dtype=torch.uint8, device="cuda")
    assert probe.gact_probe_quantize_like(src.data_ptr(), dst.data_ptr(), nbytes, in_kb, out_dw, None) == 0
    torch.cuda.synchronize()
    written = dst[:tiles * 256 * out_dw]
    assert (written != 0xA5).float().mean() > 0.9            # data-dependent values everywhere
    assert (dst[tiles * 256 * out_dw:] == 0xA5).all()
    # the output depends on the input: another input, another output
    dst2 = torch.full_like(dst, 0xA5)
    assert probe.gact_probe_quantize_like((src ^ 1).data_ptr(), dst2.data_ptr(), nbytes, in_kb, out_dw, None) == 0
    assert not torch.equal(dst, dst2)


@pytest.mark.parametrize("in_dw,out_kb", [(1, 8), (2, 8), (4, 8), (8, 8), (1, 4), (2, 4), (4, 4), (8, 4)])
def test_dequantize_like_probe_writes_its_tiles_and_nothing_else(in_dw, out_kb):
    probe = bench.probe_lib()
    tiles = 29
    nbytes = tiles * out_kb * 1024 + 300
    src = torch.randint(0, 255, (tiles * 256 * in_dw,), dtype=torch.uint8, device="cuda")
    dst = torch.full((nbytes + 1024,), 0xA5, dtype=torch.uint8, device="cuda")
    assert probe.gact_probe_dequantize_like(src.data_ptr(), dst.data_ptr(), nbytes, in_dw, out_kb, None) == 0
    torch.cuda.synchronize()
    assert (dst[:tiles * out_kb * 1024] != 0xA5).float().mean() > 0.9
    assert (dst[tiles * out_kb * 1024:] == 0xA5).all()
    dst2 = torch.full_like(dst, 0xA5)
    assert probe.gact_probe_dequantize_like((src ^ 1).data_ptr(), dst2.data_ptr(), nbytes, in_dw, out_kb, None) == 0
    assert not torch.equal(dst, dst2)


def test_probe_arguments():
    probe = bench.probe_lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    assert probe.gact_probe_quantize_like(p, p, 8192, 3, 1, None) == -1        # tile sizes are 4 or 8 KB
    assert probe.gact_probe_quantize_like(p, p, 8192, 8, 3, None) == -1        # 1, 2, 4 or 8 dwords per lane
    assert probe.gact_probe_quantize_like(p + 4, p, 8192, 8, 1, None) == -1    # 16-byte aligned
    assert probe.gact_probe_dequantize_like(p, p, 8192, 3, 8, None) == -1
    assert probe.gact_probe_dequantize_like(p, p, 8192, 1, 16, None) == -1
    assert probe.gact_probe_quantize_like(p, p, 100, 8, 1, None) == 0          # no whole tile: nothing to do
