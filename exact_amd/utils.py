"""Small helpers kept from the reference's exact/exact/utils.py: index
down-casting (:9-28), host swap (:31-34), memory accounting (:37-65),
allocator trimming (:68-74) and the JSON-lines recorder (:85-105)."""
import json
from collections import OrderedDict

import numpy as np
import torch


def cast_low_bit_int(idx_vec):
    """int64 index vector -> int32 when every value fits (utils.py:9-19).
    The reference also narrows to int16; the SpMM kernels here take int32 or
    int64, so int16 is never produced."""
    if idx_vec is None:
        return idx_vec
    assert idx_vec.dtype == torch.int64
    if idx_vec.numel() == 0 or int(idx_vec.max()) < np.iinfo(np.int32).max:
        return idx_vec.to(torch.int32)
    return idx_vec


def cast_adj(data):
    """utils.py:22-28: narrow every cached index vector of data.adj_t."""
    st = data.adj_t.storage
    for name in ("_col", "_row", "_rowptr", "_rowcount", "_colptr", "_csr2csc"):
        setattr(st, name, cast_low_bit_int(getattr(st, name)))


def swap_to_cpu(tensor):
    tensor_cpu = torch.empty(tensor.shape, dtype=tensor.dtype, device="cpu", pin_memory=True)
    tensor_cpu.copy_(tensor, non_blocking=True)
    return tensor_cpu


def get_memory_usage(gpu, print_info=False):
    allocated = torch.cuda.memory_allocated(gpu)
    reserved = torch.cuda.memory_reserved(gpu)
    if print_info:
        print("allocated: %.2f MB" % (allocated / 1024 / 1024), flush=True)
        print("reserved:  %.2f MB" % (reserved / 1024 / 1024), flush=True)
    return allocated


_BYTES = {torch.int64: 8, torch.float32: 4, torch.int32: 4, torch.bfloat16: 2, torch.float16: 2,
          torch.int16: 2, torch.int8: 1, torch.uint8: 1}


def compute_tensor_bytes(tensors):
    if not isinstance(tensors, (list, tuple)):
        tensors = [tensors]
    total = 0
    for x in tensors:
        if x.dtype not in _BYTES:
            raise ValueError(x.dtype)
        total += int(np.prod(x.size())) * _BYTES[x.dtype]
    return total


def empty_cache(ratio):
    if ratio is None:
        return
    allocated = torch.cuda.memory_allocated(0)
    reserved = torch.cuda.memory_reserved(0)
    if reserved > 0 and allocated / reserved < ratio:
        torch.cuda.empty_cache()


class GlobalExpRecorder:
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
            fout.write(json.dumps(self.val_dict) + "\n")
        print("Save exp results to %s" % filename)

    def clear(self):
        pass


exp_recorder = GlobalExpRecorder()
