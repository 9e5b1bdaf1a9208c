"""One launch for many saved tensors of mixed bit widths, with the widths resident on the GPU.

The reference quantizes one tensor per call (gact/gact/quantizer.py:95-142) and computes the widths on
the host (gact/gact/autoprec.py:188-209).  Here ``calc_precision_device`` leaves the widths in device
memory and one small planning launch turns them into packed-arena offsets (and says which tensor every
block of the grid belongs to); the batched kernels then quantize (one launch per element type over all
blocks, a block's width selecting its code path) or dequantize (one launch for every type and width)
every tensor at its own width.  Nothing is read back to the host; the results are identical to calling
``op_quantize`` / ``op_dequantize`` tensor by tensor.

Grid layout: a block owns 128 groups of 256 elements whatever the width, so the grid
(sum over tensors of ceil(N_i/128) blocks) is known on the host without knowing the widths.
"""
import torch

from .cpp_extension import _abi

GROUPS_PER_BLOCK = 128


class BatchedPacked:
    """What a batched quantize leaves behind: the arenas, the table and the per-tensor geometry.

    The widths come from device memory, so whether they were all valid (1, 2, 4 or 8 - a tensor that
    calc_precision left at 32 is not) and whether the arena was large enough is only known on the
    device: when either fails the kernels write nothing.  ``ok()`` reads that verdict back (it
    synchronises); ``per_tensor`` and ``BatchedQuantizer.dequantize`` call it and raise."""

    def __init__(self, owner, packed, scale, mn, table, bits, workspace, shapes, dtypes, seeds):
        self.owner = owner
        self.seeds = list(seeds)
        self.packed, self.scale, self.min = packed, scale, mn
        self.table, self.bits, self.workspace = table, bits, workspace
        self.shapes, self.dtypes = shapes, dtypes

    def ok(self):
        """(plan succeeded, arena bytes the table needs); synchronises."""
        vals = self.workspace[:16].view(torch.int64).tolist()
        return bool(vals[1]), vals[0]

    def require_ok(self):
        good, need = self.ok()
        if not good:
            raise RuntimeError("gact: the batched launch was void - a width outside {1, 2, 4, 8} or a packed arena "
                               "of %d bytes where %d are needed; nothing was quantized" % (self.packed.numel(), need))

    def per_tensor(self, i):
        """Views (packed bytes, bits, scale[N,1,1], min[N,1,1]) of tensor i in op_quantize's format.
        Reads the width and the offset back from the device (synchronises)."""
        self.require_ok()
        b = int(self.bits[i].item())
        numel = self.owner.numels[i]
        N = (numel + _abi.GROUP - 1) // _abi.GROUP
        nbytes = _abi.lib().gact_packed_bytes(b, N, 1, _abi.GROUP)
        table_host = self.table.cpu().numpy().view("int64").reshape(-1, 7)
        off = int(table_host[i, 5])
        so = self.owner.stats_offsets[i] * 4
        dt = self.dtypes[i]
        sdt = torch.float32 if dt == torch.bfloat16 else dt      # bfloat16 tensors keep a float scale
        sc = self.scale[so:so + N * sdt.itemsize].view(sdt).reshape(N, 1, 1)
        mn = self.min[so:so + N * dt.itemsize].view(dt).reshape(N, 1, 1)
        return self.packed[off:off + nbytes].view(torch.int8), b, sc, mn


class BatchedQuantizer:
    """Geometry of a fixed list of saved tensors (element counts and dtypes), reusable every iteration."""

    def __init__(self, numels, dtypes, device):
        if len(numels) != len(dtypes):
            raise ValueError("one dtype per tensor")
        self.device = torch.device(device)
        self.numels = [int(n) for n in numels]
        self.dtypes = list(dtypes)
        # which element types occur (bit 0 float, bit 1 half, bit 2 bfloat16): the library launches only their kernels
        self.dtype_mask = 0
        for dt in self.dtypes:
            self.dtype_mask |= 1 << _abi.dtype_code(dt)
        self.L = len(self.numels)
        self.first_blocks, self.stats_offsets = [], []
        blocks = 0
        groups = 0
        for n in self.numels:
            N = (n + _abi.GROUP - 1) // _abi.GROUP
            self.first_blocks.append(blocks)
            self.stats_offsets.append(groups)
            blocks += (N + GROUPS_PER_BLOCK - 1) // GROUPS_PER_BLOCK
            groups += (N + 7) // 8 * 8   # 32-byte aligned rows: the dequantize kernel reads them 16 bytes at a time
        self.total_blocks = blocks
        self.total_groups = groups
        self.workspace_bytes = int(_abi.lib().gact_batch_workspace_bytes(self.L, self.total_blocks))

    # ---- arena sizing (host-side bounds; the exact need is computed on the device) ----
    def arena_bytes_for_budget(self, target_bits):
        """Upper bound of the packed bytes when the widths come from calc_precision with this bit
        budget: the greedy stops at sum(b_i * numel_i) <= max(target, sum(numel_i)); padding to whole
        groups, to whole bytes of 8/b groups and to 256-byte offsets adds at most 768 bytes per tensor."""
        total = max(int(target_bits), sum(self.numels))
        return (total + 7) // 8 + 768 * self.L + 256

    def arena_bytes_worst_case(self):
        """Every tensor at 8 bits."""
        return sum(self.numels) + 768 * self.L + 256

    def new_workspace(self):
        """Device memory a plan of this geometry fills: a 256-byte header (the verdict) and the block -> tensor map."""
        return torch.empty((self.workspace_bytes,), dtype=torch.uint8, device=self.device)

    def plan_ok(self, workspace):
        """Whether the last plan written to this workspace succeeded; synchronises."""
        return bool(workspace[8:16].view(torch.int64).item())

    def _table(self, tensors, seeds):
        arr = (_abi.BatchEntry * self.L)()
        for i, t in enumerate(tensors):
            if t.numel() != self.numels[i] or t.dtype != self.dtypes[i]:
                raise RuntimeError("tensor %d does not match the geometry this batch was built for" % i)
            if not t.is_cuda or not t.is_contiguous():
                raise RuntimeError("tensor %d must be a contiguous CUDA tensor" % i)
            if not _abi.aligned(t):
                raise RuntimeError("tensor %d is not 16-byte aligned" % i)
            e = arr[i]
            e.x = t.data_ptr()
            e.numel = self.numels[i]
            e.dtype = _abi.dtype_code(t.dtype)
            e.seed = int(seeds[i]) & 0xFFFFFFFFFFFFFFFF
            e.first_block = self.first_blocks[i]
            e.packed_offset = 0
            e.stats_offset = self.stats_offsets[i]
        host = torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8)
        return host.to(self.device, non_blocking=False)

    # ---- the launches on caller-owned buffers (nothing is allocated, nothing synchronises) ----
    def launch_quantize(self, table, bits, packed, scale, mn, workspace, mode):
        """Plan into `workspace` from the device-resident `bits`, then quantize every tensor of `table`."""
        lib = _abi.lib()
        st = torch.cuda.current_stream(self.device).cuda_stream
        _abi.check(lib.gact_batch_plan(table.data_ptr(), bits.data_ptr(), self.L, self.total_blocks, packed.numel(),
                                       workspace.data_ptr(), st))
        _abi.check(lib.gact_quantize_batched(table.data_ptr(), bits.data_ptr(), self.L, self.total_blocks, mode,
                                             self.dtype_mask, workspace.data_ptr(), packed.data_ptr(),
                                             scale.data_ptr(), mn.data_ptr(), st))

    def launch_dequantize(self, table, bits, packed, scale, mn, workspace):
        """Plan into `workspace` (the table's x point at the outputs; planning again from the same widths gives
        the same offsets without reading anything back), then dequantize every tensor."""
        lib = _abi.lib()
        st = torch.cuda.current_stream(self.device).cuda_stream
        _abi.check(lib.gact_batch_plan(table.data_ptr(), bits.data_ptr(), self.L, self.total_blocks, packed.numel(),
                                       workspace.data_ptr(), st))
        _abi.check(lib.gact_dequantize_batched(table.data_ptr(), bits.data_ptr(), self.L, self.total_blocks,
                                               workspace.data_ptr(), packed.data_ptr(), scale.data_ptr(),
                                               mn.data_ptr(), st))

    def quantize(self, tensors, bits, seeds, arena_bytes=None, rng_stream=None):
        """Quantize all tensors in one batched launch.  `bits` is an int32 tensor on the device (e.g. the output
        of calc_precision_device) holding 1, 2, 4 or 8 for every tensor.  Returns a BatchedPacked; nothing
        synchronises, so a void launch (see BatchedPacked) shows when the result is used."""
        from .cpp_extension.quantization import _noise_mode
        if bits.dtype != torch.int32 or not bits.is_cuda or bits.numel() != self.L:
            raise RuntimeError("bits must be an int32 CUDA tensor with one entry per tensor")
        mode = _noise_mode(None, rng_stream)
        if arena_bytes is None:
            arena_bytes = self.arena_bytes_worst_case()
        with torch.cuda.device(self.device):
            table = self._table(tensors, seeds)
            packed = torch.empty((int(arena_bytes),), dtype=torch.uint8, device=self.device)
            scale = torch.empty((self.total_groups * 4,), dtype=torch.uint8, device=self.device)
            mn = torch.empty((self.total_groups * 4,), dtype=torch.uint8, device=self.device)
            ws = self.new_workspace()
            # the widths are kept as they were at quantize time: the caller may refresh its own copy
            kept = bits.clone()
            self.launch_quantize(table, kept, packed, scale, mn, ws, mode)
        return BatchedPacked(self, packed, scale, mn, table, kept, ws, [t.shape for t in tensors],
                             list(self.dtypes), seeds)

    def dequantize(self, q, outs=None, check=True):
        """Dequantize every tensor of a BatchedPacked in one launch into fresh tensors (or `outs`).
        check = True reads the plan's verdict back first (one synchronisation) and raises when the quantize
        launch was void; pass False where nothing may synchronise (stream capture) and the caller has
        checked ``q.ok()`` itself."""
        if check:
            q.require_ok()
        with torch.cuda.device(self.device):
            if outs is None:
                outs = [torch.empty(s, dtype=d, device=self.device) for s, d in zip(q.shapes, q.dtypes)]
            table = self._table(outs, q.seeds)
            ws = self.new_workspace()
            self.launch_dequantize(table, q.bits, q.packed, q.scale, q.min, ws)
            # keep the table alive until the stream has consumed it
            q._dq_table = (table, ws)
        return outs
