"""Which saved tensors get compressed, at what width and seed, and the bookkeeping that lets the backward
pass find them again.  The constructor, the methods, the tuples handed to the autograd hooks and the
tid / bits / dims / seeds tables are those of gact/gact/quantizer.py of the reference.

All kernels launch on the stream that is current when a hook runs; swapping uses two side streams.
"""
import torch

from .conf import config
from .ops import op_dequantize, op_dequantize_mask, op_quantize, op_quantize_mask
from .utils import sampled_key_with_sum

_COMPRESSIBLE = (torch.float32, torch.float16, torch.bfloat16)   # bfloat16: not in the reference
_RANKS = (2, 3, 4)
KEY_SAMPLES = 100
BOOL_MASK_MIN_ELEMENTS = 4096     # smaller bool tensors are not worth a kernel launch


class _Swap:
    """Streams and events of the host-swap path (quantizer.py:18-29 of the reference)."""

    def __init__(self, prefetch):
        self.out_stream = torch.cuda.Stream()
        self.in_stream = torch.cuda.Stream()
        self.prefetch_started = self.prefetch_done = None
        if prefetch:
            self.prefetch_started = torch.cuda.Event(blocking=True)
            self.prefetch_done = torch.cuda.Event(blocking=True)


class Quantizer:
    """default_bit: width used until auto precision has run.  swap: keep the packed codes in pinned host
    memory.  prefetch (needs swap): while tensor `tid` is dequantized, copy tensor `tid - 1` back to the GPU."""

    def __init__(self, default_bit, swap, prefetch):
        self.default_bit = default_bit
        self.swap, self.prefetch = swap, prefetch
        # the reference creates the prefetch events whenever prefetch is set, with or without swap
        # (quantizer.py:25-28): start_prefetch_event / end_prefetch_event exist in both cases
        self._swap = _Swap(prefetch) if (swap or prefetch) else None
        self.compute_stream = torch.cuda.current_stream() if torch.cuda.is_available() else None

        self.unrelated_tensors = set()   # data pointers of parameters: saved for backward, never compressed
        self.ptr_qtensor_map = {}        # key -> [q_inputs, references still to be consumed, tid]
        self.layer_key_map = {}          # tid -> key
        self.tid = 0                     # running index of compressed tensors within one iteration
        self.start_bwd = True

        # filled on the first iteration; read and rewritten by auto precision
        self.bits, self.dims, self.seeds = {}, {}, {}
        self.iter = 0        # iterations seen, the extra passes of auto precision included
        self._seed_dev = None   # config.device_seed: seed_iter as one int64 on the GPU, created on first use
        self.seed_iter = 0   # added to every seed; constant during one adaptive step so that probes are comparable

    @property
    def seed_iter(self):
        return self._seed_iter

    @seed_iter.setter
    def seed_iter(self, value):
        self._seed_iter = value
        if self._seed_dev is not None:
            self._seed_dev.fill_(value)       # an eager fill between graph replays

    # ---- streams of the swap path under their reference names ----
    @property
    def swap_out_stream(self):
        return self._swap.out_stream

    @property
    def swap_in_stream(self):
        return self._swap.in_stream

    @property
    def start_prefetch_event(self):
        return self._swap.prefetch_started

    @property
    def end_prefetch_event(self):
        return self._swap.prefetch_done

    # ---- selection ----
    def filter_tensors(self, pairs):
        self.unrelated_tensors.update(v.data_ptr() for _, v in pairs)

    def check_quantize(self, input_tensor):
        """-> (compress?, is it a 0/1 mask?).  The rules of quantizer.py:47-69 in their order: parameters stay;
        a non-empty uint8 tensor is a mask if it holds exactly the values 0 and 1 and is left alone otherwise;
        then float16 / float32 (and bfloat16, which the reference does not know) only, requires_grad only (batch-norm statistics do not), rank 2 to 4 only.
        One rule more than the reference has: a bool tensor on the GPU is a mask by construction (no
        values to inspect, no synchronisation) when config.compress_bool_masks is set."""
        t = input_tensor
        if t.data_ptr() in self.unrelated_tensors:
            return False, False
        if t.dtype == torch.uint8 and t.numel() > 0:
            # one reduction and one synchronisation for both ends
            is_mask = torch.stack(torch.aminmax(t)).tolist() == [0, 1]
            return is_mask, is_mask
        if t.dtype == torch.bool:
            # contiguous only: an expanded or strided view (a broadcast attention mask) may occupy far less than
            # numel bytes, and unpacking would hand back a dense copy
            is_mask = (config.compress_bool_masks and t.is_cuda and t.numel() >= BOOL_MASK_MIN_ELEMENTS
                       and t.is_contiguous())
            return is_mask, is_mask
        ok = t.dtype in _COMPRESSIBLE and t.requires_grad is not False and t.dim() in _RANKS
        if ok and t.dtype == torch.bfloat16 and config.group_size != 256:
            ok = False      # bfloat16 exists in the single-pass kernels (group size 256) only: left alone, as in the reference
        return ok, False

    def generate_tensor_key(self, t, tid):
        if not config.check_dup:
            return tid
        # the same tensor saved by two operators: address + strided sample + sum
        return tuple(sampled_key_with_sum(t, KEY_SAMPLES))

    def iterate(self):
        self.ptr_qtensor_map, self.layer_key_map = {}, {}
        self.tid = 0
        self.start_bwd = True
        self.iter += 1

    # ---- pack hook ----
    def quantize(self, input):
        """(False, tensor) when left alone, (True, True, q_mask) for a mask (a bool mask adds its dtype as a
        fourth entry), else (True, False, key, shape, tid)."""
        wanted, is_mask = self.check_quantize(input)
        if not wanted:
            return False, input
        if is_mask:
            if input.dtype == torch.bool:     # same bytes as a uint8 0/1 mask
                return True, True, op_quantize_mask(input.view(torch.uint8)), torch.bool
            return True, True, op_quantize_mask(input)

        tid = self.tid
        self.tid = tid + 1
        key = self.layer_key_map[tid] = self.generate_tensor_key(input, tid)
        held = self.ptr_qtensor_map.get(key)
        if held is None:
            self.ptr_qtensor_map[key] = [self._compress(input, tid), 1, tid]
        else:
            held[1] += 1        # saved again under the same key: one more consumer, no new codes
        return True, False, key, input.shape, tid

    def _compress(self, t, tid):
        if self.iter == 0:      # the first pass fixes the tables auto precision works on
            self.bits[tid], self.dims[tid], self.seeds[tid] = self.default_bit, t.numel(), tid
        if config.device_seed:
            if self._seed_dev is None:      # during the eager warm-up passes, never inside a capture
                self._seed_dev = torch.full((1,), self._seed_iter, dtype=torch.int64, device=t.device)
            q_inputs = op_quantize(t, self.bits[tid], self.seeds[tid], seed_offset=self._seed_dev)
        else:
            q_inputs = op_quantize(t, self.bits[tid], self.seeds[tid] + self.seed_iter)
        if self.swap:
            # On the current stream, as in the reference (quantizer.py:125-137, whose side-stream lines are
            # commented out).  Issuing the copy on the swap-out stream (wait_stream + record_stream) was
            # measured and is slower on this stack: 105 -> 159 ms per BERT-base iteration at 4 bit.
            codes = q_inputs[0]
            q_inputs[0] = torch.empty(codes.shape, dtype=codes.dtype, device="cpu", pin_memory=True)
            q_inputs[0].copy_(codes, non_blocking=True)
        return q_inputs

    # ---- unpack hook ----
    def dequantize(self, input):
        if not input[0]:
            return input[1]
        if input[1]:
            mask = op_dequantize_mask(input[2])
            return mask.view(input[3]) if len(input) > 3 else mask
        key, shape, tid = input[2:]
        held = self.ptr_qtensor_map[key]
        q_inputs = held[0]
        if self.swap:
            self._fetch(q_inputs, tid)
        out = op_dequantize(q_inputs, shape)
        held[1] -= 1
        if held[1] < 0:
            raise RuntimeError("[Error] Ref count < 0 for key %r" % (key,))
        if held[1] == 0:
            del self.ptr_qtensor_map[key]
        return out

    def _fetch(self, q_inputs, tid):
        """Codes back on the GPU for tensor tid; with prefetch, tensor tid - 1 starts its copy meanwhile
        (quantizer.py:156-183 of the reference)."""
        sw = self._swap
        if self.start_bwd:      # first unpack of the backward pass: all swap-outs must have landed
            self.compute_stream.wait_stream(sw.out_stream)
            self.start_bwd = False
        if self.prefetch:
            sw.prefetch_done.wait(self.compute_stream)
        if not q_inputs[0].is_cuda:     # not prefetched: a synchronous copy
            q_inputs[0] = q_inputs[0].cuda(non_blocking=False)
        if not self.prefetch:
            return
        sw.prefetch_started.record()
        with torch.cuda.stream(sw.in_stream):
            if tid > 0:
                sw.prefetch_started.wait(sw.in_stream)
                prev = self.ptr_qtensor_map.get(self.layer_key_map[tid - 1])
                if prev is not None and not prev[0][0].is_cuda:
                    prev[0][0] = prev[0][0].cuda(non_blocking=True)
                    prev[0][0].record_stream(self.compute_stream)   # allocated on the copy stream, used on compute
                sw.prefetch_done.record()
