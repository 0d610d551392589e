"""input2rp + quantize_activation as one launch (exact_rp_minmax_pack_f32) on
the Python side, both back ends: identical to the two calls it replaces
(reference ops.py:141-149, layers.py:153-159).  Both sides of the comparison
here are this library's own kernels: it shows that the host side's fused and
unfused routes agree, not that either is right.  The kernel itself is pinned
bit for bit against the oracle in test_emulated_kernels.py (emulator) and
test_gpu_rp.py (GPU, through the C ABI, every matrix-core path).  Collected
late on purpose: it switches config.fuse_epilogue and the projection sources."""
import pytest
import torch
import torch.nn.functional as F

import exact_amd as exact
from exact_amd import ops
from exact_amd.conf import config
from exact_amd.cpp_extension import quantization as extq
from gpu_util import SeededNoise


def _seeded(seed):
    s = SeededNoise(seed)
    config.noise_source, config.rp_matrix_source = s.noise_source, s.rp_matrix_source


@pytest.mark.parametrize("bits", [1, 2, 8])
@pytest.mark.parametrize("N,D,frac", [(300, 256, 0.125), (77, 602, 0.125), (130, 100, 0.25), (9, 40, 0.5)])
@pytest.mark.parametrize("supplied", [True, False])
def test_one_launch_equals_the_two_calls(backend, N, D, frac, bits, supplied):
    config.kept_frac = frac
    config.activation_compression_bits = [bits]
    x = torch.randn(N, D, generator=torch.Generator().manual_seed(N)).to(backend)
    results = []
    for fuse in (False, True):
        config.fuse_epilogue = fuse
        if supplied:
            _seeded(4)
        else:
            s = SeededNoise(4)
            config.noise_source, config.rp_matrix_source = None, s.rp_matrix_source
            if backend.type == "cuda":
                torch.cuda.manual_seed(77)              # the emulated back end restarts its Philox counter below
            else:
                import itertools
                counter = itertools.count(1)
                extq.next_philox = lambda device: (0xC0FFEE, 4 * next(counter))
        results.append(ops.project_and_quantize(x, None))
    (q_two, r_two, shape_two), (q_one, r_one, shape_one) = results
    assert shape_two == shape_one == torch.Size((N, ops.kept_columns(D)))
    assert torch.equal(r_two, r_one)
    assert q_two[1] == q_one[1] == bits
    for a, b in zip((q_two[0], q_two[2], q_two[3]), (q_one[0], q_one[2], q_one[3])):
        assert a.dtype == b.dtype and torch.equal(a.cpu(), b.cpu())
    # and it restores like any compressed activation
    kept = ops.CompressedActivation(q_one, r_one, x.shape, shape_one)
    assert kept.restore().shape == x.shape


def test_the_one_launch_form_is_used_and_has_its_limits(backend, monkeypatch):
    config.kept_frac = 0.25
    _seeded(1)
    calls = []
    real = extq.rp_minmax_pack
    monkeypatch.setattr(extq, "rp_minmax_pack", lambda *a: (calls.append(a[1].shape), real(*a))[1])
    layer = exact.QLinear(64, 8).to(backend).train()
    x = torch.randn(50, 64, device=backend, requires_grad=True)
    layer(x).sum().backward()
    assert calls == [torch.Size((64, 16))] and x.grad is not None
    # more than 128 projected columns: the two calls
    wide = torch.randn(10, 1024, device=backend)
    q, r, shape = ops.project_and_quantize(wide, None)
    assert shape == torch.Size((10, 256)) and len(calls) == 1
    # switched off
    config.fuse_epilogue = False
    ops.project_and_quantize(x.detach(), None)
    assert len(calls) == 1
    config.fuse_epilogue = True
    # QSAGEConv: one shared copy of x (aggregation + lin_r) and lin_l's copy of the aggregate
    from exact_amd.sparse import SparseTensor
    import scipy.sparse as sp
    A = sp.random(50, 50, 0.1, format="csr", random_state=1, dtype="float32")
    adj = SparseTensor.from_scipy(A, backend).set_value(None)
    conv = exact.QSAGEConv(64, 8).to(backend).train()
    config.sage_aggregate_projected = False
    conv(x.detach().requires_grad_(), adj).sum().backward()
    assert len(calls) == 3
    # aggregating the projected input (k + out = 24 < 64 columns): lin_l's copy is the quantised aggregate of x R,
    # so only the shared copy goes through the one-launch form
    config.sage_aggregate_projected = True
    conv(x.detach().requires_grad_(), adj).sum().backward()
    assert len(calls) == 4
    # the scheme's use counter still ticks
    class Scheme:
        n = 0

        def note_use(self):
            self.n += 1
    sch = Scheme()
    ops.project_and_quantize(x.detach(), sch)
    assert sch.n == 1


def test_shim_argument_checks(backend):
    x = torch.randn(6, 16, device=backend)
    with pytest.raises(RuntimeError):
        extq.rp_minmax_pack(x, torch.randn(8, 4, device=backend), 2)
    with pytest.raises(RuntimeError):
        extq.rp_minmax_pack(x, torch.randn(16, 200, device=backend), 2)
    with pytest.raises(RuntimeError):
        extq.rp_minmax_pack(x, torch.randn(16, 4, device=backend), 3)
