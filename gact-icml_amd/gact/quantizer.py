"""Which saved tensors get compressed, with what width and seed, and the bookkeeping that lets the
backward pass find them again.  Mirrors gact/gact/quantizer.py of the reference: same constructor,
same methods, same tuples handed to the autograd hooks, same tid / bits / dims / seeds tables.

All kernels launch on the stream that is current when the hook runs.
"""
import torch

from .conf import config
from .ops import op_quantize, op_dequantize, op_quantize_mask, op_dequantize_mask
from .utils import uniform_sample


class Quantizer:
    """default_bit: width used until auto precision has run; swap: keep the packed codes in pinned host
    memory; prefetch: while layer l is dequantized, copy layer l-1 back to the GPU (needs swap)."""

    def __init__(self, default_bit, swap, prefetch):
        self.unrelated_tensors = set()   # data pointers of parameters: never compressed
        self.default_bit = default_bit

        self.swap = swap
        if swap:
            self.swap_out_stream = torch.cuda.Stream()
            self.swap_in_stream = torch.cuda.Stream()
        self.compute_stream = torch.cuda.current_stream() if torch.cuda.is_available() else None
        self.ptr_qtensor_map = {}        # key -> [q_inputs, reference count, tid]
        self.prefetch = prefetch
        if prefetch:
            self.start_prefetch_event = torch.cuda.Event(blocking=True)
            self.end_prefetch_event = torch.cuda.Event(blocking=True)
        self.layer_key_map = {}          # tid -> key
        self.tid = 0                     # running index of compressed tensors within one iteration
        self.start_bwd = True

        # filled on the first iteration, read and updated by auto precision
        self.seeds = {}
        self.bits = {}
        self.dims = {}

        self.iter = 0        # iterations seen, including the extra passes auto precision runs
        self.seed_iter = 0   # iteration number mixed into the seeds (constant within an adaptive step)

    def filter_tensors(self, pairs):
        for _, v in pairs:
            self.unrelated_tensors.add(v.data_ptr())

    def check_quantize(self, input_tensor):
        """-> (compress?, is a dropout mask?).  gact/gact/quantizer.py:47-69."""
        if input_tensor.data_ptr() in self.unrelated_tensors:
            return False, False
        if input_tensor.numel() > 0 and input_tensor.dtype == torch.uint8:
            # a saved 0/1 mask goes to the 1-bit mask kernel; one reduction, one synchronisation
            lo, hi = torch.aminmax(input_tensor)
            if int(hi) == 1 and int(lo) == 0:
                return True, True
            return False, False
        if input_tensor.dtype not in (torch.float32, torch.float16):
            return False, False
        if input_tensor.requires_grad is False:   # e.g. batch-norm running statistics
            return False, False
        if input_tensor.dim() not in (2, 3, 4):
            return False, False
        return True, False

    def iterate(self):
        self.ptr_qtensor_map = {}
        self.layer_key_map = {}
        self.tid = 0
        self.start_bwd = True
        self.iter += 1

    def generate_tensor_key(self, t, tid):
        if config.check_dup:
            key = uniform_sample(t, min(100, t.numel()), add_dataptr=True)
            key.append(t.sum().item())
            return tuple(key)
        return tid

    def quantize(self, input):
        """Pack hook.  Returns (False, tensor) | (True, True, q_mask) | (True, False, key, shape, tid)."""
        wanted, is_mask = self.check_quantize(input)
        if not wanted:
            return False, input
        if is_mask:
            return True, True, op_quantize_mask(input)

        tid, self.tid = self.tid, self.tid + 1
        key = self.generate_tensor_key(input, tid)
        self.layer_key_map[tid] = key
        entry = self.ptr_qtensor_map.get(key)
        if entry is not None:
            entry[1] += 1                       # saved again: one more reference, no new codes
        else:
            self.ptr_qtensor_map[key] = [self._compress(input, tid), 1, tid]
        return True, False, key, input.shape, tid

    def _compress(self, input, tid):
        """Quantize one tensor at its current width; the first iteration fills the tables auto precision reads."""
        if self.iter == 0:
            self.bits[tid] = self.default_bit
            self.dims[tid] = input.numel()
            self.seeds[tid] = tid
        q_inputs = op_quantize(input, self.bits[tid], self.seeds[tid] + self.seed_iter)
        if self.swap:
            host = torch.empty(q_inputs[0].shape, dtype=q_inputs[0].dtype, device="cpu", pin_memory=True)
            host.copy_(q_inputs[0], non_blocking=True)
            q_inputs[0] = host
        return q_inputs

    def _prefetch_previous(self, tid):
        """Start copying layer tid-1's codes back to the GPU while layer tid is dequantized."""
        self.start_prefetch_event.record()
        with torch.cuda.stream(self.swap_in_stream):
            if tid > 0:
                self.start_prefetch_event.wait(self.swap_in_stream)
                prev = self.ptr_qtensor_map.get(self.layer_key_map[tid - 1])
                if prev is not None and not prev[0][0].is_cuda:
                    prev[0][0] = prev[0][0].cuda(non_blocking=True)
                    # allocated on the copy stream, consumed on the compute stream
                    prev[0][0].record_stream(self.compute_stream)
                self.end_prefetch_event.record()

    def dequantize(self, input):
        """Unpack hook: the inverse of quantize()."""
        if not input[0]:
            return input[1]
        if input[1]:
            return op_dequantize_mask(input[2])

        _, _, key, input_shape, tid = input
        entry = self.ptr_qtensor_map[key]
        q_inputs = entry[0]

        if self.swap:
            if self.start_bwd:
                self.compute_stream.wait_stream(self.swap_out_stream)
                self.start_bwd = False
            if self.prefetch:
                self.end_prefetch_event.wait(self.compute_stream)
            if not q_inputs[0].is_cuda:         # swapped out and not prefetched: fetch it now
                q_inputs[0] = q_inputs[0].cuda(non_blocking=False)
            if self.prefetch:
                self._prefetch_previous(tid)

        ret = op_dequantize(q_inputs, input_shape)

        entry[1] -= 1
        if entry[1] < 0:
            raise RuntimeError("[Error] Ref count < 0 for key %r" % (key,))
        if entry[1] == 0:
            del self.ptr_qtensor_map[key]
        return ret
