"""The accuracy bisect tool (counterpart of the reference's dump rewriters, reference
test/npu_indexing/accuracy_check/fx_graph_gen.py:19-142): it must name the first wrong node of a
graph whose compiled form carries a planted fault, say whether the fault survives compiling the node
alone, and report nothing for a correct compilation.  The CPU tests plant the fault in a stand-in
compiler (an interpreter), so they pin the search itself; the GPU tests run the real backend."""
import pytest
import torch
import torch.fx as fx

from inductor_x_amd import accuracy_check as ac
from tests.helpers import announce


def _norm_graph(x, w):
    h = torch.tanh(x * 2 + 1)
    v, m = torch.var_mean(h, dim=-1, keepdim=True)
    y = (h - m) * torch.rsqrt(v + 1e-5) * w
    return y.sum(-1), y.argmax(-1)


def _faulty(target, delta, only_fused):
    """A compiler that evaluates the graph eagerly and adds `delta` to the result of `target`."""

    def compiler(sub, inputs):
        fused = sum(1 for n in sub.graph.nodes if n.op == "call_function") > 1

        class Run(fx.Interpreter):
            def run_node(self, n):
                out = super().run_node(n)
                if n.op == "call_function" and n.target is target and (fused or not only_fused):
                    out = out + delta
                return out

        return lambda *a: Run(sub).run(*a)

    return compiler


def _inputs(device="cpu"):
    g = torch.Generator().manual_seed(0)
    return torch.randn(32, 64, generator=g).to(device), torch.randn(64, generator=g).to(device)


def test_capture_returns_aten_graph_and_real_inputs():
    x, w = _inputs()
    gm, flat = ac.capture(_norm_graph, x, w)
    targets = [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]
    assert "aten.var_mean.correction" in targets and "aten.argmax.default" in targets
    assert len(flat) == 2 and torch.equal(flat[0], x) and torch.equal(flat[1], w)
    vals = ac.node_values(gm, flat)
    out = [n for n in gm.graph.nodes if n.op == "output"][0].args[0]
    want = _norm_graph(x, w)
    assert torch.equal(vals[out[0].name], want[0]) and torch.equal(vals[out[1].name], want[1])


def test_digest_is_md5_of_fp64_bytes():
    import hashlib

    t = torch.tensor([1.0, 2.5, -3.0], dtype=torch.bfloat16)
    want = hashlib.md5(torch.tensor([1.0, 2.5, -3.0], dtype=torch.float64).numpy().tobytes()).hexdigest()
    assert ac.tensor_digest(t) == want


@pytest.mark.parametrize("target,name", [
    (torch.ops.aten.tanh.default, "tanh"),
    (torch.ops.aten.rsqrt.default, "rsqrt"),
    (torch.ops.aten.sum.dim_IntList, "sum_1"),
    (torch.ops.aten.mul.Tensor, "mul"),  # three mul nodes: the first in graph order must be named
])
def test_bisect_names_first_planted_fault(target, name):
    x, w = _inputs()
    gm, flat = ac.capture(_norm_graph, x, w)
    rep = ac.bisect(gm, flat, compiler=_faulty(target, 0.05, only_fused=False))
    assert not rep.ok and rep.first_bad.node == name, str(rep)
    assert rep.isolated_ok is False
    assert rep.first_bad.max_abs == pytest.approx(0.05, rel=1e-3)
    # binary search: far fewer compilations than nodes (12 tensor nodes here)
    assert rep.compilations <= 2 + rep.nodes.bit_length() + 1


def test_bisect_tells_fusion_faults_from_single_op_faults():
    x, w = _inputs()
    gm, flat = ac.capture(_norm_graph, x, w)
    rep = ac.bisect(gm, flat, compiler=_faulty(torch.ops.aten.rsqrt.default, 0.01, only_fused=True))
    assert not rep.ok and rep.first_bad.node == "rsqrt" and rep.isolated_ok is True
    assert "fusion" in str(rep)


def test_integer_nodes_must_match_exactly_and_multi_output_producers_are_isolated():
    x, w = _inputs()
    gm, flat = ac.capture(_norm_graph, x, w)
    rep = ac.bisect(gm, flat, compiler=_faulty(torch.ops.aten.argmax.default, 1, only_fused=False))
    assert not rep.ok and rep.first_bad.node == "argmax" and rep.first_bad.max_abs == 32  # all 32 rows differ

    # var_mean returns a tuple; the wrong tensor is its getitem, isolated together with its producer
    def bad_var(sub, inputs):
        class Run(fx.Interpreter):
            def run_node(self, n):
                out = super().run_node(n)
                if n.op == "call_function" and n.target is torch.ops.aten.var_mean.correction:
                    out = (out[0] * 1.1, out[1])
                return out

        return lambda *a: Run(sub).run(*a)

    rep = ac.bisect(gm, flat, compiler=bad_var)
    assert not rep.ok and rep.first_bad.node == "getitem" and rep.isolated_ok is False


def test_clean_compilation_reports_ok_with_digests():
    x, w = _inputs()
    rep = ac.check(_norm_graph, x, w, compiler=_faulty(None, 0.0, only_fused=False), digests=True)
    assert rep.ok and rep.compilations == 1 and rep.first_bad is None
    assert set(rep.digests) >= {"tanh", "rsqrt", "sum_1", "argmax"} and all(len(d) == 32 for d in rep.digests.values())


def test_inductor_cpu_codegen_passes_the_check():
    x, w = _inputs()
    rep = ac.check(_norm_graph, x, w, rtol=1e-4, atol=1e-5)
    assert rep.ok, str(rep)


@pytest.mark.gpu
def test_generated_hip_kernels_pass_the_check():
    import inductor_x_amd  # noqa: F401  registration side effects

    x, w = _inputs("cuda:0")
    announce("accuracy_check: norm graph through the HIP backend")
    rep = ac.check(_norm_graph, x, w, rtol=1e-4, atol=1e-5)
    assert rep.ok, str(rep)

    def block(h, r, wt):
        s = h + r
        n = s.float() * torch.rsqrt(s.float().pow(2).mean(-1, keepdim=True) + 1e-6) * wt.float()
        return n.to(torch.bfloat16), s

    g = torch.Generator().manual_seed(1)
    h = torch.randn(256, 4096, generator=g).bfloat16().cuda()
    r = torch.randn(256, 4096, generator=g).bfloat16().cuda()
    wt = (1 + 0.02 * torch.randn(4096, generator=g)).bfloat16().cuda()
    announce("accuracy_check: add+rmsnorm bf16 through the HIP backend")
    rep = ac.check(block, h, r, wt, rtol=2e-2, atol=2e-2)
    assert rep.ok, str(rep)


@pytest.mark.gpu
def test_planted_fault_is_found_behind_the_real_backend():
    """The real compilation with one output corrupted afterwards: the search runs real kernels."""
    import inductor_x_amd  # noqa: F401

    x, w = _inputs("cuda:0")
    gm, flat = ac.capture(_norm_graph, x, w)
    names = [n.name for n in gm.graph.nodes if n.op == "call_function" and n.target is not __import__("operator").getitem]

    def corrupting(sub, inputs):
        real = ac.default_compiler(sub, inputs)
        outs_nodes = [n for n in sub.graph.nodes if n.op == "output"][0].args[0]
        idx = [i for i, n in enumerate(outs_nodes) if n.name == "sub"]

        def run(*a):
            out = list(real(*a))
            for i in idx:
                out[i] = out[i] + 0.5
            return out

        return run

    announce("accuracy_check: planted fault at node 'sub' behind the HIP backend")
    rep = ac.bisect(gm, flat, compiler=corrupting)
    assert "sub" in names and not rep.ok and rep.first_bad.node == "sub", str(rep)
