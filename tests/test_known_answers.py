"""The hand-made known-answer vectors of tests/golden/known_answers.json
against (1) the oracle, Python and C, and (2) the library through its Python
shims on both back ends (emulated kernels always, the GPU with -m gpu)."""
import json
import os

import numpy as np
import pytest
import torch

import c_oracle as co
import exact_oracle as o
import exact_oracle_extra as ox
from exact_amd import ops
from exact_amd.conf import config
from exact_amd.cpp_extension import quantization as extq
from exact_amd.cpp_extension import spmm as ext_spmm
from gpu_util import FixedNoise, bytes_equal

F32 = np.float32
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")) as _f:
    CASES = json.load(_f)


def f32(a):
    return np.asarray(a, dtype=F32)


def ident(case):
    return case["op"] + ("-" + str(case.get("bits", case.get("reduce", ""))) if ("bits" in case or "reduce" in case) else "")


def pick(op):
    return [pytest.param(c, id=f"{ident(c)}-{i}") for i, c in enumerate(CASES) if c["op"] == op]


def test_fixture_file_is_what_the_script_writes():
    import importlib.util
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_known_answers.py")
    spec = importlib.util.spec_from_file_location("make_known_answers", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert json.loads(json.dumps(mod.CASES)) == CASES and len({c["op"] for c in CASES}) == 13


# ------------------------------------------------------------------ oracle side
@pytest.mark.parametrize("c", pick("philox"))
def test_oracle_philox(c):
    assert o.philox4x32(np.array(c["ctr"]), c["key"]).tolist() == c["out"]
    assert co.philox4x32_10(c["ctr"], c["key"]).tolist() == c["out"]


@pytest.mark.parametrize("c", pick("pack"))
def test_oracle_pack(c):
    x, mn, sc, noise = f32(c["x"]), f32(c["mn"]), f32(c["scale"]), f32(c["noise"])
    assert o.pack_single_precision(x, mn, sc, c["bits"], noise).tolist() == c["packed"]
    assert co.pack(x, mn, sc, c["bits"], noise).tolist() == c["packed"]


@pytest.mark.parametrize("c", pick("minmax_pack"))
def test_oracle_minmax_pack(c):
    packed, _, sbf, mbf, scale, mn = o.quantize_activation(f32(c["x"]), c["bits"], f32(c["noise"]))
    assert packed.tolist() == c["packed"] and sbf.tolist() == c["scale_bf16"] and mbf.tolist() == c["min_bf16"]
    lo, hi = co.row_minmax(f32(c["x"]))
    assert co.pack(f32(c["x"]), lo, co.scale(lo, hi, c["bits"]), c["bits"], f32(c["noise"])).tolist() == c["packed"]


@pytest.mark.parametrize("c", pick("unpack"))
def test_oracle_unpack(c):
    packed = np.array(c["packed"], np.uint8)
    for fn in (o.unpack_single_precision, co.unpack):
        out = fn(packed, c["bits"], f32(c["scale"]), f32(c["mn"]), c["N"], c["G"])
        assert np.array_equal(out, f32(c["out"]))


@pytest.mark.parametrize("c", pick("relu") + pick("leaky_relu") + pick("dropout"))
def test_oracle_masks(c):
    x, dy = f32(c["x"]), f32(c["dy"])
    if c["op"] == "relu":
        runs = [(o.relu_fwd(x), o.relu_bwd), (co.relu_fwd(x), co.relu_bwd)]
    elif c["op"] == "leaky_relu":
        runs = [(ox.leaky_relu_fwd(x, c["slope"]), lambda g, m: ox.leaky_relu_bwd(g, m, c["slope"]))]
    else:
        runs = [(o.dropout_fwd(x, c["p"], f32(c["noise"])), lambda g, m: o.dropout_bwd(g, m, c["p"])),
                (co.dropout_fwd(x, c["p"], f32(c["noise"])), lambda g, m: co.dropout_bwd(g, m, c["p"]))]
    for (y, mask), bwd in runs:
        assert np.array_equal(y, f32(c["y"])) and np.asarray(mask).tolist() == c["mask"]
        assert np.array_equal(bwd(dy, mask), f32(c["dx"]))


@pytest.mark.parametrize("c", pick("spmm") + pick("sddmm"))
def test_oracle_sparse(c):
    rowptr, col, X = np.array(c["rowptr"]), np.array(c["col"]), f32(c["X"])
    val = None if c.get("val") is None else f32(c["val"])
    if c["op"] == "sddmm":
        row = np.repeat(np.arange(len(rowptr) - 1), np.diff(rowptr))
        assert np.array_equal(ox.sddmm(row, rowptr, col, X, f32(c["grad"]), c["reduce"]), f32(c["out"]))
    elif c["reduce"] in ("max", "min"):
        out, arg = ox.spmm_minmax(rowptr, col, val, X, c["reduce"] == "max")
        assert np.array_equal(out, f32(c["out"])) and arg.tolist() == c["arg"]
    else:
        assert np.array_equal(o.spmm_csr(rowptr, col, val, X, c["reduce"]), f32(c["out"]))
        assert np.array_equal(co.spmm_csr(rowptr, col, val, X, c["reduce"]), f32(c["out"]))


@pytest.mark.parametrize("c", pick("rp"))
def test_oracle_rp(c):
    X, R = f32(c["X"]), f32(c["R"])
    for fwd, bwd in ((o.input2rp, o.rp2input), (co.rp_fwd, co.rp_bwd)):
        assert np.array_equal(fwd(X, R), f32(c["fwd"])) and np.array_equal(bwd(f32(c["fwd"]), R), f32(c["bwd_of_fwd"]))


@pytest.mark.parametrize("c", pick("relu_dropout_pack"))
def test_oracle_chain(c):
    x = f32(c["x"])
    y1, m1 = o.relu_fwd(x.reshape(-1))
    y2, m2 = o.dropout_fwd(y1, c["p"], f32(c["act_noise"]).reshape(-1))
    packed, _, sbf, mbf, _, _ = o.quantize_activation(y2.reshape(x.shape), c["bits"], f32(c["noise"]))
    assert np.array_equal(y2.reshape(x.shape), f32(c["y"])) and (m1 & m2).tolist() == c["mask"]
    assert packed.tolist() == c["packed"] and sbf.tolist() == c["scale_bf16"] and mbf.tolist() == c["min_bf16"]


@pytest.mark.parametrize("c", pick("bn_relu_dropout_pack"))
def test_oracle_chain_after_batch_norm(c):
    x = f32(c["x"])
    normalised = ((x - f32(c["mean"])[None, :]) * f32(c["mult"])[None, :] + f32(c["shift"])[None, :]).astype(F32)
    y1, m1 = o.relu_fwd(normalised.reshape(-1))
    y2, m2 = o.dropout_fwd(y1, c["p"], f32(c["act_noise"]).reshape(-1))
    packed, _, sbf, mbf, _, _ = o.quantize_activation(y2.reshape(x.shape), c["bits"], f32(c["noise"]))
    assert np.array_equal(y2.reshape(x.shape), f32(c["y"])) and (m1 & m2).tolist() == c["mask"]
    assert packed.tolist() == c["packed"] and sbf.tolist() == c["scale_bf16"] and mbf.tolist() == c["min_bf16"]


@pytest.mark.parametrize("c", pick("rp_pack"))
def test_oracle_projection_then_quantisation(c):
    packed, _, sbf, mbf, _, _ = o.quantize_activation(o.input2rp(f32(c["X"]), f32(c["R"])), c["bits"], f32(c["noise"]))
    assert packed.tolist() == c["packed"] and sbf.tolist() == c["scale_bf16"] and mbf.tolist() == c["min_bf16"]


# ------------------------------------------------------------------ library side
def dev(a, backend, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return t.to(backend) if dtype is None else t.to(backend, dtype)


def supply(*noises):
    config.noise_source = FixedNoise([torch.from_numpy(f32(n)) for n in noises])


@pytest.mark.parametrize("c", pick("pack"))
def test_library_pack(backend, c):
    supply(c["noise"])
    mn, sc = dev(f32(c["mn"]), backend), dev(f32(c["scale"]), backend)
    packed = extq.pack_single_precision(dev(f32(c["x"]), backend), mn, mn, sc, c["bits"], True)
    assert packed.cpu().numpy().view(np.uint8).tolist() == c["packed"]


@pytest.mark.parametrize("c", pick("minmax_pack"))
def test_library_minmax_pack(backend, c):
    supply(c["noise"])
    config.activation_compression_bits = [c["bits"]]
    packed, bits, sbf, mbf = ops.quantize_activation(dev(f32(c["x"]), backend), None)
    assert bits == c["bits"] and packed.cpu().numpy().view(np.uint8).tolist() == c["packed"]
    assert bytes_equal(sbf, np.array(c["scale_bf16"], np.uint16)) and bytes_equal(mbf, np.array(c["min_bf16"], np.uint16))


@pytest.mark.parametrize("c", pick("unpack"))
def test_library_unpack(backend, c):
    packed = dev(np.array(c["packed"], np.uint8).view(np.int8), backend)
    out = extq.unpack_single_precision(packed, c["bits"], dev(f32(c["scale"]), backend), dev(f32(c["mn"]), backend),
                                       c["N"], c["G"])
    assert bytes_equal(out, f32(c["out"]))


@pytest.mark.parametrize("c", pick("relu") + pick("leaky_relu") + pick("dropout"))
def test_library_masks(backend, c):
    x = dev(f32(c["x"]), backend).requires_grad_()
    if c["op"] == "relu":
        y = extq.act_quantized_relu(x)
    elif c["op"] == "leaky_relu":
        y = extq.act_quantized_leaky_relu(x, c["slope"])
    else:
        supply(c["noise"])
        y = extq.act_quantized_dropout(x, c["p"], True)
    (mask,) = y.grad_fn.saved_tensors
    assert mask.cpu().numpy().view(np.uint32).tolist() == c["mask"]
    y.backward(dev(f32(c["dy"]), backend))
    assert bytes_equal(y, f32(c["y"]) + F32(0)) and bytes_equal(x.grad, f32(c["dx"]))


@pytest.mark.parametrize("c", pick("relu_dropout_pack"))
def test_library_fused_chain(backend, c):
    supply(c["act_noise"], c["noise"], c["act_noise"])
    x = dev(f32(c["x"]), backend)
    y, mask, packed, sbf, mbf = extq.relu_dropout_minmax_pack(x, c["p"], c["bits"])
    assert bytes_equal(y, f32(c["y"])) and mask.cpu().numpy().view(np.uint32).tolist() == c["mask"]
    assert packed.cpu().numpy().view(np.uint8).tolist() == c["packed"]
    assert bytes_equal(sbf, np.array(c["scale_bf16"], np.uint16)) and bytes_equal(mbf, np.array(c["min_bf16"], np.uint16))
    y2, mask2 = extq.relu_dropout_fwd(x, c["p"])
    assert bytes_equal(y2, f32(c["y"])) and mask2.cpu().numpy().view(np.uint32).tolist() == c["mask"]


@pytest.mark.parametrize("c", pick("bn_relu_dropout_pack"))
def test_library_fused_chain_after_batch_norm(backend, c):
    supply(c["act_noise"], c["noise"])
    x = dev(f32(c["x"]), backend)
    vectors = [dev(f32(c[name]), backend) for name in ("mean", "mult", "shift")]
    y, mask, packed, sbf, mbf = extq.bn_relu_dropout_minmax_pack(x, *vectors, c["p"], c["bits"])
    assert bytes_equal(y, f32(c["y"])) and mask.cpu().numpy().view(np.uint32).tolist() == c["mask"]
    assert packed.cpu().numpy().view(np.uint8).tolist() == c["packed"]
    assert bytes_equal(sbf, np.array(c["scale_bf16"], np.uint16)) and bytes_equal(mbf, np.array(c["min_bf16"], np.uint16))


@pytest.mark.parametrize("c", pick("rp_pack"))
def test_library_projection_then_quantisation(backend, c):
    supply(c["noise"])
    R = dev(f32(c["R"]), backend)
    packed, sbf, mbf = extq.rp_minmax_pack(dev(f32(c["X"]), backend), R, c["bits"])
    assert packed.cpu().numpy().view(np.uint8).tolist() == c["packed"]
    assert bytes_equal(sbf, np.array(c["scale_bf16"], np.uint16)) and bytes_equal(mbf, np.array(c["min_bf16"], np.uint16))
    # and through the public path
    supply(c["noise"])
    config.kept_frac, config.activation_compression_bits = 0.5, [c["bits"]]
    config.rp_matrix_source = lambda D, k, device: R
    (q, bits, s2, m2), used, shape = ops.project_and_quantize(dev(f32(c["X"]), backend), None)
    assert used is R and bits == c["bits"] and tuple(shape) == (2, 2) and q.cpu().numpy().view(np.uint8).tolist() == c["packed"]


@pytest.mark.parametrize("idx", [torch.int64, torch.int32])
@pytest.mark.parametrize("c", pick("spmm") + pick("sddmm"))
def test_library_sparse(backend, c, idx):
    rowptr, col = dev(np.array(c["rowptr"]), backend, idx), dev(np.array(c["col"]), backend, idx)
    X = dev(f32(c["X"]), backend)
    val = None if c.get("val") is None else dev(f32(c["val"]), backend)
    if c["op"] == "sddmm":
        row = dev(np.repeat(np.arange(len(c["rowptr"]) - 1), np.diff(c["rowptr"])), backend, idx)
        out = ext_spmm.spmm_value_bw(row, rowptr, col, X, dev(f32(c["grad"]), backend), c["reduce"])
        assert bytes_equal(out, f32(c["out"]))
    elif c["reduce"] in ("max", "min"):
        out, arg = (ext_spmm.spmm_max_fw if c["reduce"] == "max" else ext_spmm.spmm_min_fw)(rowptr, col, val, X)
        assert bytes_equal(out, f32(c["out"])) and arg.cpu().tolist() == c["arg"]
    else:
        assert bytes_equal(ext_spmm.spmm_csr(rowptr, col, val, X, c["reduce"]), f32(c["out"]))


@pytest.mark.parametrize("c", pick("rp"))
def test_library_rp(backend, c):
    R = dev(f32(c["R"]), backend)
    config.rp_matrix_source = lambda D, k, device: R
    X = dev(f32(c["X"]), backend)
    xr, used = ops.input2rp(X, R.shape[1])
    assert used is R and bytes_equal(xr, f32(c["fwd"]))
    assert bytes_equal(ops.rp2input(xr, X.shape, R), f32(c["bwd_of_fwd"]))
