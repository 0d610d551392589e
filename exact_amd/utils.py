"""Small host-side helpers with the names the reference exports from
exact/exact/utils.py: index narrowing (cast_low_bit_int / cast_adj, :9-28),
memory accounting (get_memory_usage / compute_tensor_bytes, :37-65), allocator
trimming (empty_cache, :68-74) and the JSON-lines experiment recorder (:85-105)."""
import json

import torch

_INT32_MAX = 2 ** 31 - 1


def cast_low_bit_int(idx_vec):
    """Narrow an int64 index vector to int32 when all its values fit.  (The
    reference also narrows to int16; the SpMM kernels here read int32 or int64.)"""
    if idx_vec is None:
        return None
    if idx_vec.dtype != torch.int64:
        raise TypeError("expected an int64 index vector")
    fits = idx_vec.numel() == 0 or int(idx_vec.max()) < _INT32_MAX
    return idx_vec.to(torch.int32) if fits else idx_vec


def cast_adj(data):
    """Narrow every cached index vector of data.adj_t in place."""
    storage = data.adj_t.storage
    for field in ("_rowptr", "_col", "_row", "_rowcount", "_colptr", "_csr2csc"):
        setattr(storage, field, cast_low_bit_int(getattr(storage, field)))


def swap_to_cpu(tensor):
    """Asynchronous copy of a device tensor into pinned host memory on the
    current stream (reference utils.py:31-34).  The copy back
    (`.to(device, non_blocking=True)` on the same stream) is ordered after it."""
    host = torch.empty(tensor.shape, dtype=tensor.dtype, device="cpu", pin_memory=tensor.is_cuda)
    host.copy_(tensor, non_blocking=True)
    return host


def get_memory_usage(gpu, print_info=False):
    """Bytes currently allocated by torch on device `gpu`."""
    allocated = torch.cuda.memory_allocated(gpu)
    if print_info:
        mib = 1 << 20
        print(f"allocated: {allocated / mib:.2f} MB", flush=True)
        print(f"reserved:  {torch.cuda.memory_reserved(gpu) / mib:.2f} MB", flush=True)
    return allocated


def compute_tensor_bytes(tensors):
    """Bytes held by a tensor or a list / tuple of tensors."""
    if isinstance(tensors, torch.Tensor):
        tensors = (tensors,)
    return sum(t.numel() * t.element_size() for t in tensors)


def empty_cache(ratio):
    """Return cached blocks to the driver when less than `ratio` of the reserved
    memory is in use; None switches it off."""
    if ratio is None:
        return
    reserved = torch.cuda.memory_reserved(0)
    if reserved > 0 and torch.cuda.memory_allocated(0) < ratio * reserved:
        torch.cuda.empty_cache()


class GlobalExpRecorder:
    """Collects key/value results of one experiment and appends them to a
    JSON-lines file."""

    def __init__(self):
        self.val_dict = {}

    def record(self, key, value, float_round=6):
        if hasattr(value, "item"):
            value = value.item()
        self.val_dict[key] = round(value, float_round) if isinstance(value, float) else value

    def dump(self, filename):
        with open(filename, "a") as out:
            out.write(json.dumps(self.val_dict) + "\n")
        print(f"Save exp results to {filename}")

    def clear(self):
        self.val_dict.clear()


exp_recorder = GlobalExpRecorder()
