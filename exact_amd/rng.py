"""(seed, offset) pairs for the library's Philox streams, taken from torch's
default CUDA generator the way the reference reserves cuRAND offsets under the
generator lock (quantization_cuda_kernel.cu:116-122, 527-533)."""
import threading

import torch

_lock = threading.Lock()


def next_philox(device) -> tuple:
    """Reserve one call's worth of the stream.  Every call gets a distinct
    64-bit offset; the kernels put it in the upper half of the Philox counter,
    so streams of different calls never overlap."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    gen = torch.cuda.default_generators[idx]
    with _lock:
        seed = gen.initial_seed()
        offset = gen.get_offset()
        gen.set_offset(offset + 4)   # torch keeps offsets multiples of 4
    return seed & 0xFFFFFFFFFFFFFFFF, offset
