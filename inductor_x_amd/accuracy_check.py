"""Find the first ATen node of a compiled graph whose value differs from eager.

Counterpart of the reference's accuracy-check scripts (reference
test/npu_indexing/accuracy_check/fx_graph_gen.py:19-142 and gen_output_code.py): those rewrite the
text of Inductor's debug dumps (`fx_graph_readable.py`, `output_code.py`) so that every
intermediate prints an md5 of its fp64 bytes, or is saved to disk, and a person then compares the
two listings.  Here the same question is answered in-process, without debug dumps:

  1. `capture` traces the function to the ATen graph Inductor would receive (after AOTAutograd);
  2. the graph is evaluated node by node in eager mode, which gives every intermediate
     (`node_values`, with the same md5-of-fp64-bytes digest the reference prints);
  3. `bisect` compiles *prefixes* of the graph that return every tensor computed so far and
     compares them with the eager values.  A prefix that contains a wrong node stays wrong when it
     grows, so a binary search over the prefix length finds the first wrong node in
     O(log n) compilations;
  4. the node found is compiled once more on its own, fed with the eager values of its operands:
     `isolated_ok` tells a wrong single-op lowering from an error that only appears in fusion.

Works on any device Inductor compiles for; on a GPU the graphs go through this package's backend.
"""
from __future__ import annotations

import dataclasses
import hashlib
from typing import Any, Callable, Optional, Sequence

import torch
import torch.fx as fx

Compiler = Callable[[fx.GraphModule, Sequence[torch.Tensor]], Callable]


def tensor_digest(t: torch.Tensor) -> str:
    """md5 of the tensor's values as fp64 bytes (the digest the reference's rewritten graphs
    print, reference test/npu_indexing/accuracy_check/fx_graph_gen.py:57,72)."""
    return hashlib.md5(t.detach().to(torch.float64).cpu().contiguous().numpy().tobytes()).hexdigest()


def capture(fn: Callable, *args: Any) -> tuple[fx.GraphModule, list[torch.Tensor]]:
    """The forward ATen graph of `fn(*args)` as Inductor receives it, and its flat inputs."""
    from torch._dynamo.backends.common import aot_autograd

    graphs: list[fx.GraphModule] = []
    flat: list[list[Any]] = []

    def fw_compiler(gm: fx.GraphModule, example_inputs: Sequence[torch.Tensor]) -> Callable:
        # the example inputs are fake tensors; the real ones are seen when the graph is called
        graphs.append(gm)

        def run(args: list[Any]) -> Any:
            if len(flat) < len(graphs):
                flat.append([a.detach().clone() if isinstance(a, torch.Tensor) else a for a in args])
            return gm.forward(*args)

        run._boxed_call = True  # type: ignore[attr-defined]
        return run

    torch._dynamo.reset()
    with torch.no_grad():
        torch.compile(fn, backend=aot_autograd(fw_compiler=fw_compiler), fullgraph=True)(*args)
    torch._dynamo.reset()
    if not graphs or not flat:
        raise RuntimeError("accuracy_check.capture: the function produced no graph (no tensor computation traced)")
    return graphs[0], flat[0]


class _Recorder(fx.Interpreter):
    def __init__(self, gm: fx.GraphModule):
        super().__init__(gm, garbage_collect_values=False)
        self.values: dict[str, Any] = {}

    def run_node(self, n: fx.Node) -> Any:
        out = super().run_node(n)
        self.values[n.name] = out
        return out


def node_values(gm: fx.GraphModule, inputs: Sequence[torch.Tensor]) -> dict[str, Any]:
    """Eager value of every node of the graph, keyed by node name."""
    rec = _Recorder(gm)
    with torch.no_grad():
        rec.run(*inputs)
    return rec.values


def _tensor_nodes(gm: fx.GraphModule, values: dict[str, Any]) -> list[fx.Node]:
    return [
        n for n in gm.graph.nodes
        if n.op in ("call_function", "call_method", "call_module") and isinstance(values.get(n.name), torch.Tensor)
    ]


def _prefix_module(gm: fx.GraphModule, upto: fx.Node, returned: Sequence[fx.Node]) -> fx.GraphModule:
    """Copy of the graph cut after `upto`, returning the nodes in `returned`."""
    g = fx.Graph()
    env: dict[fx.Node, fx.Node] = {}
    for n in gm.graph.nodes:
        if n.op == "output":
            break
        env[n] = g.node_copy(n, lambda x: env[x])
        if n is upto:
            break
    g.output(tuple(env[n] for n in returned))
    return fx.GraphModule(gm, g)


def _single_node_module(gm: fx.GraphModule, node: fx.Node, values: dict[str, Any]) -> tuple[fx.GraphModule, list[fx.Node]]:
    """A graph of `node` alone; its tensor operands become placeholders (returned in order).
    Operands that are not tensors (the tuple a multi-output operator returns, sizes) are
    recomputed inside the graph from their own operands."""
    g = fx.Graph()
    operands: list[fx.Node] = []
    env: dict[fx.Node, fx.Node] = {}

    def lift(x: fx.Node) -> fx.Node:
        if x not in env:
            if isinstance(values.get(x.name), torch.Tensor) or x.op == "placeholder":
                env[x] = g.placeholder(x.name)
                env[x].meta = dict(x.meta)
                operands.append(x)
            else:
                env[x] = g.node_copy(x, lift)
        return env[x]

    out = g.node_copy(node, lift)
    g.output((out,))
    return fx.GraphModule(gm, g), operands


def default_compiler(gm: fx.GraphModule, inputs: Sequence[torch.Tensor]) -> Callable:
    from torch._inductor.compile_fx import compile_fx

    return compile_fx(gm, list(inputs))


def _call(compiled: Callable, inputs: Sequence[torch.Tensor]) -> list[Any]:
    out = compiled(*inputs)
    return list(out) if isinstance(out, (tuple, list)) else [out]


@dataclasses.dataclass
class Mismatch:
    node: str
    target: str
    max_abs: float
    max_rel: float
    eager_digest: str
    compiled_digest: str


@dataclasses.dataclass
class Report:
    ok: bool
    nodes: int
    compilations: int
    first_bad: Optional[Mismatch] = None
    isolated_ok: Optional[bool] = None
    digests: dict[str, str] = dataclasses.field(default_factory=dict)

    def __str__(self) -> str:
        if self.ok:
            return f"accuracy_check: {self.nodes} tensor nodes agree with eager ({self.compilations} compilations)"
        m = self.first_bad
        where = "also wrong when compiled alone" if self.isolated_ok is False else "correct when compiled alone: a fusion effect"
        return (f"accuracy_check: first wrong node {m.node} = {m.target}: max abs err {m.max_abs:.3e}, "
                f"max rel err {m.max_rel:.3e}; {where} ({self.compilations} compilations)")


def _compare(name: str, target: str, want: torch.Tensor, got: Any, rtol: float, atol: float) -> Optional[Mismatch]:
    if not isinstance(got, torch.Tensor) or got.shape != want.shape or got.dtype != want.dtype:
        return Mismatch(name, target, float("inf"), float("inf"), tensor_digest(want), "shape or dtype differs")
    if want.numel() == 0:
        return None
    if not (want.is_floating_point() or want.is_complex()):
        if torch.equal(want, got):
            return None
        bad = float((want != got).sum())
        return Mismatch(name, target, bad, bad, tensor_digest(want), tensor_digest(got))
    w, g = want.to(torch.float64), got.to(torch.float64)
    same = (w == g) | (w.isnan() & g.isnan())
    err = torch.where(same, torch.zeros_like(w), (w - g).abs())
    if bool((err.nan_to_num(nan=float("inf")) <= atol + rtol * w.abs()).all()):
        return None
    err = err.nan_to_num(nan=float("inf"))
    rel = err / w.abs().clamp_min(1e-300)
    return Mismatch(name, target, float(err.max()), float(rel.max()), tensor_digest(want), tensor_digest(got))


def bisect(
    gm: fx.GraphModule,
    inputs: Sequence[torch.Tensor],
    rtol: float = 1e-3,
    atol: float = 1e-3,
    compiler: Optional[Compiler] = None,
    digests: bool = False,
) -> Report:
    """First node (in graph order) whose compiled value leaves eager's by more than
    atol + rtol * |eager| (the reference's tests use 1e-3 for both, reference
    test/npu_indexing/reduction_test.py:28-30); integer and boolean nodes must be equal."""
    compiler = compiler or default_compiler
    values = node_values(gm, inputs)
    nodes = _tensor_nodes(gm, values)
    report = Report(ok=True, nodes=len(nodes), compilations=0)
    if digests:
        report.digests = {n.name: tensor_digest(values[n.name]) for n in nodes}
    if not nodes:
        return report

    def first_mismatch(k: int) -> Optional[Mismatch]:
        sub = _prefix_module(gm, nodes[k], nodes[: k + 1])
        report.compilations += 1
        torch._dynamo.reset()
        with torch.no_grad():
            outs = _call(compiler(sub, inputs), inputs)
        for n, got in zip(nodes[: k + 1], outs):
            m = _compare(n.name, str(n.target), values[n.name], got, rtol, atol)
            if m is not None:
                return m
        return None

    worst = first_mismatch(len(nodes) - 1)
    if worst is None:
        return report
    # invariant: prefix `lo - 1` is clean (or empty), prefix `hi` is not
    lo, hi, found = 0, len(nodes) - 1, worst
    while lo < hi:
        mid = (lo + hi) // 2
        m = first_mismatch(mid)
        if m is None:
            lo = mid + 1
        else:
            hi, found = mid, m
    # a prefix reports its earliest wrong node, which may precede its last one
    report.ok = False
    report.first_bad = found
    bad = next(n for n in nodes if n.name == found.node)
    single, operands = _single_node_module(gm, bad, values)
    single_inputs = [values[o.name] for o in operands]
    report.compilations += 1
    torch._dynamo.reset()
    with torch.no_grad():
        got = _call(compiler(single, single_inputs), single_inputs)[0]
    report.isolated_ok = _compare(bad.name, str(bad.target), values[bad.name], got, rtol, atol) is None
    return report


def check(fn: Callable, *args: Any, rtol: float = 1e-3, atol: float = 1e-3,
          compiler: Optional[Compiler] = None, digests: bool = False) -> Report:
    """capture + bisect for a Python function and its example arguments."""
    gm, flat = capture(fn, *args)
    return bisect(gm, flat, rtol=rtol, atol=atol, compiler=compiler, digests=digests)
