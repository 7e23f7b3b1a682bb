"""Top-2 expert gating through torch.compile, forward and backward, against eager: the routing
graph the reference runs as its mixture-of-experts scenario (reference
test/npu_indexing/moe/run_moe.py:24-115 driven by moe/main.py:37-49 at 4096 tokens x 8 experts).
It mixes what the generator handles (softmax over a short row, column sums and means, masked
row maxima with their indices, integer arithmetic, concatenation) with what stays a library
call (top-k, cumulative sums)."""
import math

import pytest
import torch
import torch.nn.functional as F

from tests.helpers import announce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _slots(tokens: int, experts: int, factor: float, floor: int) -> int:
    return max(int(math.ceil(tokens / experts * factor)), floor)


def route_top2(logits: torch.Tensor, factor: float = 1.1, floor: int = 4):
    """Two experts per token with a per-expert slot budget; returns the balance loss, the slot
    of each (token, choice), the renormalised gate weights and, per expert, the tokens it keeps."""
    tokens, experts = logits.shape
    slots = _slots(tokens, experts, 2 * factor, floor)
    gates = F.softmax(logits, dim=1)
    choice = torch.topk(gates, 2, dim=-1).indices
    picked = F.one_hot(choice, num_classes=experts)
    first, second = picked[:, 0, :], picked[:, 1, :]
    # position of every token in the queue of its expert; second choices queue behind all firsts
    pos1 = torch.cumsum(first, dim=0) - 1
    pos2 = torch.cumsum(second, dim=0) - 1 + first.sum(dim=0, keepdim=True)
    balance = (gates.mean(dim=0) * first.float().mean(dim=0)).mean() * experts * experts
    first = first * (pos1 < slots)
    second = second * (pos2 < slots)
    slot1 = (pos1 * first).sum(dim=1)
    slot2 = (pos2 * second).sum(dim=1)
    w1, e1 = (gates * first.float()).max(dim=1)
    w2, e2 = (gates * second.float()).max(dim=1)
    total = torch.clamp(w1 + w2, min=torch.finfo(gates.dtype).eps)
    w1, w2 = w1 / total, w2 / total
    where1 = e1.int() * slots + slot1.int()
    where2 = e2.int() * slots + slot2.int()
    kept = torch.topk(first * 2 + second, k=slots, dim=0, sorted=True).indices.t()
    return balance, torch.cat([where1, where2]), torch.cat([w1, w2]), kept


@pytest.mark.parametrize("tokens,experts", [(4096, 8), (1000, 16), (257, 4)])
def test_top2_routing_forward_and_backward(tokens, experts):
    announce(f"compile top-2 routing {tokens}x{experts}")
    import inductor_x_amd  # noqa: F401

    g = torch.Generator(device="cpu").manual_seed(tokens + experts)
    base = torch.randn(tokens, experts, generator=g).to(DEV)
    torch._dynamo.reset()
    compiled = torch.compile(route_top2, dynamic=False)
    outs = []
    for fn in (route_top2, compiled):
        logits = base.clone().requires_grad_()
        balance, where, weights, kept = fn(logits)
        (weights.sum() + balance).backward()
        outs.append((balance.detach(), where, weights.detach(), kept, logits.grad))
    (rb, rw, rg, rk, rgrad), (cb, cw, cg, ck, cgrad) = outs
    torch.testing.assert_close(cb, rb, rtol=1e-5, atol=1e-6)
    assert torch.equal(cw, rw)
    torch.testing.assert_close(cg, rg, rtol=1e-5, atol=1e-6)
    # top-k of a three-valued key is full of ties, but both sides hand the library kernel the
    # same integer input, so the kept tokens agree exactly
    assert torch.equal(ck, rk)
    torch.testing.assert_close(cgrad, rgrad, rtol=1e-4, atol=1e-6)
