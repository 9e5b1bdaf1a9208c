"""Small helpers used by the quantizer and the auto-precision driver (gact/gact/utils.py of the reference)."""
import json
from collections import OrderedDict

import numpy as np
import torch


def uniform_sample(input, sample_cnt, add_dataptr=True):
    """Evenly spaced sample of a tensor's values (optionally prefixed by its address): the key that
    recognises a tensor saved twice.  gact/gact/utils.py:16-24."""
    num_elem = input.numel()
    sample_cnt = min(num_elem, sample_cnt)
    key = [input.data_ptr()] if add_dataptr else []
    if sample_cnt > 0:
        idx = torch.arange(0, sample_cnt, dtype=torch.long, device=input.device) * (num_elem // sample_cnt)
        key += input.ravel()[idx].tolist()
    return key


def get_memory_usage(print_info=False):
    """Bytes currently allocated by torch on the GPU.  gact/gact/utils.py:40-47."""
    allocated = torch.cuda.memory_allocated()
    if print_info:
        print("allocated: %.2f MB" % (allocated / 1024 / 1024), flush=True)
        print("reserved:  %.2f MB" % (torch.cuda.memory_reserved() / 1024 / 1024), flush=True)
    return allocated


_ELEM_BYTES = {torch.long: 8, torch.float32: 4, torch.int: 4, torch.bfloat16: 2, torch.float16: 2, torch.int16: 2,
               torch.int8: 1, torch.uint8: 1}


def compute_tensor_bytes(tensors):
    """Bytes held by a tensor or a list of tensors / ints.  gact/gact/utils.py:49-70."""
    if not isinstance(tensors, (list, tuple)):
        tensors = [tensors]
    total = 0
    for x in tensors:
        if type(x) == int:
            total += 4
        elif x.dtype in _ELEM_BYTES:
            total += int(np.prod(x.size())) * _ELEM_BYTES[x.dtype]
        else:
            raise TypeError("unsupported dtype %s" % x.dtype)
    return total


class GlobalExpRecorder:
    """Key/value record appended to a file as one JSON line per dump.  gact/gact/utils.py:80-101."""

    def __init__(self):
        self.val_dict = OrderedDict()

    def record(self, key, value, float_round=6):
        if isinstance(value, (np.int32, np.int64)):
            value = int(value)
        if isinstance(value, (float, np.float32, np.float64)):
            value = round(float(value), float_round)
        self.val_dict[key] = value

    def dump(self, filename):
        with open(filename, "a") as fout:
            fout.write(json.dumps(self.val_dict) + '\n')

    def clear(self):
        pass


exp_recorder = GlobalExpRecorder()
