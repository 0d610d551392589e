"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def dev(a, device="cuda:0"):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def host_noise(shape, seed):
    """Uniform [0, 1) noise generated on the HOST with a seeded torch generator,
    so the oracle and the kernels see identical bits."""
    g = torch.Generator().manual_seed(seed)
    return torch.rand(shape, generator=g, dtype=torch.float32).numpy()


def host_randn(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).numpy()


def all_finite_halves():
    """Every finite fp16 value once (63,488 of them): an exhaustive operand for
    element-wise fp16 kernels, which therefore contains every input whose fp32
    result lies on a tie of the fp16 grid -- the inputs on which rounding the
    exact result once differs from rounding the fp32 result a second time."""
    bits = np.arange(1 << 16, dtype=np.uint16)
    v = bits.view(np.float16)
    return v[np.isfinite(v)].copy()


class FixedNoise:
    """config.noise_source that hands out pre-made tensors in call order."""

    def __init__(self, tensors):
        self.tensors = list(tensors)
        self.i = 0

    def __call__(self, shape, device):
        t = self.tensors[self.i]
        self.i += 1
        assert tuple(t.shape) == tuple(shape) or t.numel() == int(np.prod(shape))
        return t.to(device).contiguous()


def bytes_equal(t, arr):
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        t = t.view(torch.int16)
    a = t.numpy()
    return np.array_equal(a.view(np.uint8).reshape(-1), np.ascontiguousarray(arr).view(np.uint8).reshape(-1))


class SeededNoise:
    """Uniform [0, 1) noise (and projection matrices) that depends only on
    (seed, call index, shape): the product and the oracle model each hold one
    and, making their draws in the same order, see identical bits."""

    def __init__(self, seed):
        self.seed, self.calls = seed, 0

    def _gen(self):
        self.calls += 1
        return torch.Generator().manual_seed(self.seed * 1000003 + self.calls)

    def noise(self, shape, device=None):
        n = int(np.prod(shape))
        t = torch.rand(n, generator=self._gen(), dtype=torch.float32).view(*shape) if n else torch.zeros(shape)
        return t if device is None else t.to(device)

    def rademacher(self, D, k, device=None):
        bern = torch.randint(2, (D, k), generator=self._gen()).float()
        R = (2.0 * bern - 1) / k ** 0.5
        return R if device is None else R.to(device)

    # the two callables exact_amd.config expects
    def noise_source(self, shape, device):
        return self.noise(tuple(shape), device)

    def rp_matrix_source(self, D, k, device):
        return self.rademacher(D, k, device)


def powerlaw_csr(n, raw_edges, seed, alpha=2.1):
    """Host-side power-law graph of the benchmark's kind (out-degree with a
    Pareto tail of exponent alpha, uniformly random targets, symmetrised,
    de-duplicated, no self loops) as a scipy CSR pattern matrix."""
    import scipy.sparse as sp
    rng = np.random.default_rng(seed)
    raw = np.minimum(rng.random(n).clip(1e-9) ** (-1.0 / (alpha - 1.0)), max(64, n // 16))
    deg = np.clip(np.rint(raw * (raw_edges / raw.sum())), 1, max(64, n // 16)).astype(np.int64)
    src = np.repeat(np.arange(n), deg)
    dst = rng.integers(0, n, src.size)
    keep = src != dst
    src, dst = src[keep], dst[keep]
    A = sp.coo_matrix((np.ones(2 * src.size, np.float32), (np.concatenate([src, dst]), np.concatenate([dst, src]))),
                      shape=(n, n)).tocsr()
    A.data[:] = 1.0
    A.sort_indices()
    return A
