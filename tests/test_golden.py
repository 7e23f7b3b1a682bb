"""The committed fixtures of tests/golden/ (written by tests/golden/make_fixtures.py): seeded inputs
with the outputs the CPU oracle gave when they were made.

CPU half: the oracle of today reproduces every stored output (bit-exact where the output is bits or
indices, one part in 1e6 where it is a rounded fp32 copy of an fp64 result), so an edit of the oracle
that moves a result is caught here.  GPU half: the HIP kernels, through the C ABI, against the stored
outputs at the bars of the parity tests (bit-exact for moved bytes and indices, 1e-5 relative for
fp32, 2e-2 absolute for bf16, 1 % of the largest entry for the attention gradients).
"""
import os

import numpy as np
import pytest
import torch

from tests.helpers import announce, bits, from_bits

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
NAMES = ["relu_sigmoid_rowsum", "add_rmsnorm_bf16", "col_mean_var_argmax", "gather_rows", "permute4_0213",
         "attention_bf16", "attention_bwd_causal", "ring_forward_update", "ring_forward_update_lse", "add_bf16"]
DEV = "cuda:0"


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        ins = {k[3:]: z[k] for k in z.files if k.startswith("in_")}
        outs = {k[4:]: z[k] for k in z.files if k.startswith("out_")}
    return ins, outs


@pytest.fixture(scope="module")
def O():
    from oracle import oracle

    return oracle


def test_every_fixture_is_present_and_small():
    for name in NAMES:
        path = os.path.join(GOLDEN, name + ".npz")
        assert os.path.exists(path), f"{name}.npz missing: run python tests/golden/make_fixtures.py"
        assert os.path.getsize(path) < 400_000


def test_generator_reproduces_the_committed_fixtures():
    """make_fixtures.py is the script that made the files: running its cases again (nothing written)
    gives the stored inputs bit for bit, so the fixtures are not orphaned from their generator."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    seen = []
    for name, inputs, _ in mod.cases():
        ins, _ = load(name)
        seen.append(name)
        assert set(ins) == set(inputs)
        for k, v in inputs.items():
            assert np.array_equal(np.asarray(v), ins[k]), (name, k)
    assert seen == NAMES


def _same_f32(got, want, name):
    np.testing.assert_allclose(np.asarray(got, dtype=np.float64), want.astype(np.float64), rtol=1e-6, atol=1e-30,
                               err_msg=name)


def test_oracle_reproduces_golden_outputs(O):
    i, o = load("relu_sigmoid_rowsum")
    _same_f32(O.relu_sigmoid_rowsum(i["x"]), o["y"], "rowsum")

    i, o = load("add_rmsnorm_bf16")
    out, s = O.add_rmsnorm_bf16(i["h"], i["r"], i["w"], float(i["eps"]))
    assert np.array_equal(out, o["out"]) and np.array_equal(s, o["h_plus_r"])

    i, o = load("col_mean_var_argmax")
    m0, v0, a0 = O.col_mean_var_argmax(i["x"], 0.0)
    _, v1, _ = O.col_mean_var_argmax(i["x"], 1.0)
    _same_f32(m0, o["mean"], "mean")
    _same_f32(v0, o["var_c0"], "var c0")
    _same_f32(v1, o["var_c1"], "var c1")
    assert np.array_equal(a0, o["argmax"])
    assert o["var_c0"][3] == 0.0 and o["argmax"][3] == 0 and o["argmax"][7] == 4  # the planted column cases

    i, o = load("gather_rows")
    assert np.array_equal(O.gather_rows(i["table"], i["idx"]), o["out"])
    i, o = load("permute4_0213")
    assert np.array_equal(O.permute4(i["t"], (0, 2, 1, 3)), o["out"])

    i, o = load("attention_bf16")
    for tag, causal in (("causal", True), ("full", False)):
        out, mx, sm = O.attention_bf16(i["q"], i["k"], i["v"], float(i["scale"]), causal)
        assert np.array_equal(out, o["out_" + tag])
        _same_f32(mx[..., 0], o["max_" + tag], "max " + tag)
        _same_f32(sm[..., 0], o["sum_" + tag], "sum " + tag)

    i, o = load("attention_bwd_causal")
    got = O.attention_bwd(i["q"], i["k"], i["v"], i["dout"], float(i["scale"]), True)
    for g, k in zip(got, ("dq", "dk", "dv")):
        np.testing.assert_allclose(g, o[k].astype(np.float64), rtol=1e-6, atol=1e-9, err_msg=k)

    i, o = load("ring_forward_update")
    got = O.forward_update(i["prev_out"], i["prev_max"], i["prev_sum"], i["cur_out"], i["cur_max"], i["cur_sum"])
    for g, k in zip(got, ("out", "max", "sum")):
        np.testing.assert_allclose(g, o[k].astype(np.float64), rtol=1e-6, atol=1e-9, err_msg=k)

    i, o = load("ring_forward_update_lse")
    got = O.forward_update_lse(i["prev_out"], i["prev_lse"], i["cur_out"], i["cur_lse"])
    for g, k in zip(got, ("out", "lse")):
        np.testing.assert_allclose(g, o[k].astype(np.float64), rtol=1e-6, atol=1e-9, err_msg=k)

    i, o = load("add_bf16")
    assert np.array_equal(O.add_bf16(i["dst"], i["src"]), o["out"])


@pytest.mark.gpu
def test_hip_kernels_reproduce_golden_outputs(O):
    from inductor_x_amd import kernels as K

    f32 = O.bf16_bits_to_f32
    announce("golden rowsum")
    i, o = load("relu_sigmoid_rowsum")
    y = K.fused_relu_sigmoid_rowsum(torch.from_numpy(i["x"]).to(DEV)).cpu().numpy()
    np.testing.assert_allclose(y, o["y"], rtol=1e-5, atol=1e-6)

    announce("golden add_rmsnorm")
    i, o = load("add_rmsnorm_bf16")
    out, s = K.add_rmsnorm(from_bits(i["h"]).to(DEV), from_bits(i["r"]).to(DEV), from_bits(i["w"]).to(DEV),
                           float(i["eps"]))
    assert np.array_equal(bits(s), o["h_plus_r"])
    assert np.abs(f32(bits(out)) - f32(o["out"])).max() <= 2e-2

    announce("golden col_mean_var_argmax")
    i, o = load("col_mean_var_argmax")
    x = torch.from_numpy(i["x"]).to(DEV)
    for corr, key in ((0.0, "var_c0"), (1.0, "var_c1")):
        mean, var, arg = K.col_mean_var_argmax(x, corr)
        np.testing.assert_allclose(mean.cpu().numpy(), o["mean"], rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(var.cpu().numpy(), o[key], rtol=1e-5, atol=1e-6)
        assert np.array_equal(arg.cpu().numpy(), o["argmax"])

    announce("golden gather_rows / permute")
    i, o = load("gather_rows")
    got = K.gather_rows(from_bits(i["table"]).to(DEV), torch.from_numpy(i["idx"]).to(DEV))
    assert np.array_equal(bits(got), o["out"])
    i, o = load("permute4_0213")
    got = K.permute_0213_contiguous(from_bits(i["t"]).to(DEV))
    assert np.array_equal(bits(got), o["out"])

    announce("golden attention forward")
    i, o = load("attention_bf16")
    q, k, v = (from_bits(i[n]).to(DEV) for n in ("q", "k", "v"))
    for tag, causal in (("causal", True), ("full", False)):
        out, mx, sm = K.fused_attention(q, k, v, float(i["scale"]), causal)
        assert np.abs(f32(bits(out)) - f32(o["out_" + tag])).max() <= 2e-2
        np.testing.assert_allclose(mx[..., 0].cpu().numpy(), o["max_" + tag], rtol=1e-3, atol=1e-3)
        np.testing.assert_allclose(sm[..., 0].cpu().numpy(), o["sum_" + tag], rtol=2e-3)

    announce("golden attention backward")
    i, o = load("attention_bwd_causal")
    q, k, v, do = (from_bits(i[n]).to(DEV) for n in ("q", "k", "v", "dout"))
    out, mx, sm = K.fused_attention(q, k, v, float(i["scale"]), True)
    for g, key in zip(K.fused_attention_backward(q, k, v, out, do, mx, sm, float(i["scale"]), True), ("dq", "dk", "dv")):
        want = o[key]
        assert np.abs(g.float().cpu().numpy() - want).max() <= 1e-2 * np.abs(want).max() + 1e-3, key
