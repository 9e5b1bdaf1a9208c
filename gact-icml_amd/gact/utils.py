"""Helpers next to the compression path, with the names of gact/gact/utils.py of the reference: tensor
keys for duplicate detection, memory accounting, and the JSON-lines recorder auto precision logs to."""
import collections
import json
import math

import numpy as np
import torch

# ---------------------------------------------------------------- tensor keys (utils.py:6-38 of the reference)


def _key_prefix(t, add_dataptr):
    return [t.data_ptr()] if add_dataptr else []


def uniform_sample(input, sample_cnt, add_dataptr=True):
    """Key of a tensor: (its address and) min(sample_cnt, numel) values taken at a constant stride.  Two saved
    tensors with the same key are treated as the same tensor.  One gather on the tensor's device instead of
    one host read per value."""
    n = input.numel()
    take = min(n, sample_cnt)
    if take == 0:
        return _key_prefix(input, add_dataptr)
    positions = torch.arange(take, device=input.device) * (n // take)
    return _key_prefix(input, add_dataptr) + input.ravel()[positions].tolist()


def sampled_key_with_sum(input, sample_cnt):
    """uniform_sample(input, sample_cnt) + [input.sum().item()] with one device-to-host copy instead of two:
    the samples and the sum travel together as float64, which holds float16 and float32 values exactly."""
    n = input.numel()
    take = min(n, sample_cnt)
    total = input.sum().to(torch.float64).reshape(1)
    if take == 0:
        return _key_prefix(input, True) + total.tolist()
    positions = torch.arange(take, device=input.device) * (n // take)
    return _key_prefix(input, True) + torch.cat([input.ravel()[positions].to(torch.float64), total]).tolist()


def uniform_sample_ref(input, sample_cnt, add_dataptr=True):
    """The same key read value by value; what uniform_sample is tested against."""
    stride = max(input.numel() // sample_cnt, 1)
    flat = input.reshape(-1)
    return _key_prefix(input, add_dataptr) + [flat[i * stride].item() for i in range(min(sample_cnt, input.numel()))]


def random_sample(input, sample_cnt, add_dataptr=True):
    """Key from sample_cnt positions drawn with a generator seeded by the tensor's rank; the global random
    state is left as it was."""
    saved = torch.get_rng_state()
    torch.manual_seed(input.dim())
    positions = torch.randint(0, input.numel(), (sample_cnt,))
    torch.set_rng_state(saved)
    return _key_prefix(input, add_dataptr) + input.reshape(-1)[positions.to(input.device)].tolist()


# ---------------------------------------------------------------- memory accounting (utils.py:40-78)

_MB = 1024.0 * 1024.0


def get_memory_usage(print_info=False):
    """Bytes torch has allocated on the current GPU."""
    allocated = torch.cuda.memory_allocated()
    if print_info:
        print("allocated: %.2f MB" % (allocated / _MB), flush=True)
        print("reserved:  %.2f MB" % (torch.cuda.memory_reserved() / _MB), flush=True)
    return allocated


_COUNTED_DTYPES = (torch.long, torch.float32, torch.int, torch.bfloat16, torch.float16, torch.int16, torch.int8,
                   torch.uint8)


def compute_tensor_bytes(tensors):
    """Bytes held by a tensor or a list of tensors; a plain int in the list counts 4 bytes.  The dtypes the
    reference counts are accepted, anything else is an error."""
    items = tensors if isinstance(tensors, (list, tuple)) else [tensors]
    total = 0
    for x in items:
        if type(x) == int:
            total += 4
        elif x.dtype in _COUNTED_DTYPES:
            total += math.prod(x.size()) * x.element_size()
        else:
            raise TypeError("unsupported dtype %s" % x.dtype)
    return total


def empty_cache(ratio):
    """Return cached blocks to the driver when less than `ratio` of the reserved memory is in use."""
    if ratio is None:
        return
    reserved = torch.cuda.memory_reserved(0)
    if reserved > 0 and torch.cuda.memory_allocated(0) / reserved < ratio:
        torch.cuda.empty_cache()


# ---------------------------------------------------------------- experiment log (utils.py:80-101)


class GlobalExpRecorder:
    """Latest value per key; dump() appends them to a file as one JSON line."""

    def __init__(self):
        self.val_dict = collections.OrderedDict()

    def record(self, key, value, float_round=6):
        if isinstance(value, np.integer):
            value = int(value)
        elif isinstance(value, (float, np.floating)):
            value = round(float(value), float_round)
        self.val_dict[key] = value

    def dump(self, filename):
        with open(filename, "a") as out:
            out.write(json.dumps(self.val_dict))
            out.write("\n")

    def clear(self):
        pass


exp_recorder = GlobalExpRecorder()
