"""Rehearsal of the autocast path without a GPU (run by test_autocast_rehearsal.py
in a process of its own): torch.amp.custom_fwd / custom_bwd are re-targeted to
the cpu device type BEFORE exact_amd is imported, the kernels are the emulated
ones, and GCN / SAGE models train a few steps under torch.autocast("cpu",
dtype=float16).  Prints one line per model; the last line is "ok".  TESTS ONLY."""
import sys, itertools
import os
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for _p in (ROOT, os.path.join(ROOT, "tests"), os.path.join(ROOT, "oracle")):
    sys.path.insert(0, _p)
import torch, torch.amp as amp
_of, _ob = amp.custom_fwd, amp.custom_bwd
amp.custom_fwd = lambda fwd=None, *, device_type, cast_inputs=None: _of(fwd, device_type="cpu", cast_inputs=cast_inputs)
amp.custom_bwd = lambda bwd=None, *, device_type: _ob(bwd, device_type="cpu")
import numpy as np, scipy.sparse as sp
import emu_util
from exact_amd import _lib
from exact_amd.cpp_extension import _checks, quantization
_lib._lib = emu_util.emu()
_checks.on_device = lambda t: True
_checks.stream_ptr = lambda t: None
c = itertools.count(1)
quantization.next_philox = lambda device: (0xC0FFEE, 4 * next(c))
import exact_amd as exact
from exact_amd.models import GCN, SAGE
from exact_amd.sparse import SparseTensor, gcn_norm
from exact_amd.conf import config
import torch.nn.functional as F
seen = []
real = quantization.minmax_pack
quantization.minmax_pack = lambda data, bits, want_fp32=False: seen.append(data.dtype) or real(data, bits, want_fp32)
rng = np.random.default_rng(0)
A = sp.coo_matrix((np.ones(3000, np.float32), (rng.integers(0, 300, 3000), rng.integers(0, 300, 3000))), shape=(300, 300)).tocsr()
A.data[:] = 1
for kind in ("gcn", "sage", "sage_rp"):
    config.kept_frac = 0.25 if kind == "sage_rp" else 1.0
    adj = SparseTensor.from_scipy(A).set_value(None)
    if kind == "gcn":
        adj = gcn_norm(adj, add_self_loops=True)
    adj.fill_cache_()
    net = GCN(32, 64, 5, 3, dropout=0.5, batch_norm=True) if kind == "gcn" else SAGE(32, 64, 5, 3, dropout=0.5, batch_norm=True)
    model = exact.QModule(net).train()
    x = torch.randn(300, 32); labels = torch.randint(0, 5, (300,))
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    seen.clear()
    for step in range(3):
        opt.zero_grad()
        with torch.autocast("cpu", dtype=torch.float16):
            out = model(x, adj)
            loss = F.cross_entropy(out.float(), labels)
        loss.backward()
        opt.step()
    ok = all(p.grad.dtype == torch.float32 and torch.isfinite(p.grad).all() for p in model.parameters())
    print(kind, "loss", loss.item(), "out", out.dtype, "packed dtypes", sorted(str(d) for d in set(seen)), "grads ok", ok)
    assert ok and torch.isfinite(loss) and torch.float16 in seen
print("ok")
