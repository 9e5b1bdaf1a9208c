"""The reference's noise stream against an independent implementation of it.

cuRAND is not available on this platform, but torch's device generator draws through hipRAND's
cuRAND-compatible Philox4_32_10: thread `idx` of its uniform kernel initialises (seed, subsequence = idx,
offset) and writes the four outputs of one Philox block to elements idx + T*ii (T = threads of the launch,
256 per block, grid capped by the device size).  That is the same (seed, subsequence, offset) -> counter / key
layout the pack kernel uses per output byte (quantization_cuda_kernel.cu:55-56,65), so torch.rand pins

  * key = the 64-bit seed, counter = (offset / 4, 0, subsequence lo, subsequence hi),
  * the order of the four outputs of a block and the step to the next block (offset 4 = the 5th draw),
  * the uint32 -> (0, 1] map (up to the half-step 2^-33 by which hipRAND's and cuRAND's maps differ, which
    changes the float only for draws below 2^9),

of the oracle's restatement, and through the oracle of the kernels.
"""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

SEEDS = [0, 42, 0x123456789ABCDEF]


def block(seed, subsequence, index):
    key = [seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF]
    ctr = [index & 0xFFFFFFFF, index >> 32, subsequence & 0xFFFFFFFF, subsequence >> 32]
    return oracle.philox4x32_10(ctr, key)


def uniform_candidates(v):
    """cuRAND's map and hipRAND's map of a uint32 draw, each with torch's 1.0 -> 0.0."""
    vf = np.float32(v)
    cu = np.float32(vf * np.float32(2.0 ** -32) + np.float32(2.0 ** -33))
    hip = np.float32(np.float32(2.0 ** -32) + vf * np.float32(2.0 ** -32))
    return {float(0.0 if c == 1.0 else c) for c in (cu, hip)}


def launch_threads(numel):
    props = torch.cuda.get_device_properties(0)
    blocks = min(props.multi_processor_count * (props.max_threads_per_multi_processor // 256), (numel + 255) // 256)
    return 256 * blocks


@pytest.mark.parametrize("seed", SEEDS)
def test_first_draw_and_next_block(seed):
    torch.manual_seed(seed)
    a = torch.rand(1024, device="cuda").cpu().numpy()      # offset 0: draw 0 of block 0
    b = torch.rand(1024, device="cuda").cpu().numpy()      # offset 4: draw 0 of block 1 = the 5th draw
    for j in range(1024):
        assert float(a[j]) in uniform_candidates(block(seed, j, 0)[0]), (seed, j)
        assert float(b[j]) in uniform_candidates(block(seed, j, 1)[0]), (seed, j)
    # the same draws as the oracle's per-element noise of the reference stream: 1 bit packs 8 groups per
    # byte, so byte j = no*256 + d draws 8 times: rows no*8 + ni of the noise tensor
    u = oracle.noise(oracle.NOISE_REF, seed, 1, 32)
    for j in range(1024):
        no, d = divmod(j, 256)
        assert u[no * 8 + 0, 0, d] == np.float32(oracle.curand_uniform(block(seed, j, 0)[0]))
        assert u[no * 8 + 4, 0, d] == np.float32(oracle.curand_uniform(block(seed, j, 1)[0]))
        assert float(0.0 if u[no * 8, 0, d] == 1.0 else u[no * 8, 0, d]) in uniform_candidates(block(seed, j, 0)[0])


@pytest.mark.parametrize("seed", SEEDS[1:])
def test_all_four_draws_of_a_block(seed):
    T = launch_threads(1 << 26)
    numel = 4 * T                                          # every thread writes its four outputs
    assert launch_threads(numel) == T
    torch.manual_seed(seed)
    c = torch.rand(numel, device="cuda")
    picks = list(range(0, 512)) + list(range(T - 256, T))
    got = c.view(4, T)[:, picks].cpu().numpy()
    u = oracle.noise(oracle.NOISE_REF, seed, 2, 8)          # 2 bit: 4 draws per byte, bytes 0..511
    for col, j in enumerate(picks):
        r = block(seed, j, 0)
        for ii in range(4):
            assert float(got[ii, col]) in uniform_candidates(r[ii]), (seed, j, ii)
        if j < 512:
            no, d = divmod(j, 256)
            for ii in range(4):
                assert u[no * 4 + ii, 0, d] == np.float32(oracle.curand_uniform(r[ii]))
