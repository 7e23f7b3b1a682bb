"""A small transformer block trained one step through torch.compile: forward and backward graphs
(layer norm, GELU, bias and weight gradients, residuals, the fused attention pattern) run on
generated HIP kernels plus library GEMMs, and every gradient is compared with eager autograd.
The reference registers its attention pattern for training traces as well
(reference inductor_x/npu_fusion_attention_graph.py:196-230)."""
import math

import pytest
import torch
import torch.nn.functional as F

from tests.helpers import announce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def backend():
    import inductor_x_amd  # noqa: F401  registration side effects

    return inductor_x_amd


class Block(torch.nn.Module):
    def __init__(self, dim: int, heads: int, hidden: int):
        super().__init__()
        self.heads = heads
        self.ln1 = torch.nn.LayerNorm(dim)
        self.q = torch.nn.Linear(dim, dim)
        self.k = torch.nn.Linear(dim, dim)
        self.v = torch.nn.Linear(dim, dim)
        self.proj = torch.nn.Linear(dim, dim)
        self.ln2 = torch.nn.LayerNorm(dim)
        self.up = torch.nn.Linear(dim, hidden)
        self.down = torch.nn.Linear(hidden, dim)

    def forward(self, x):
        B, S, D = x.shape
        h = self.ln1(x)
        hd = D // self.heads
        # heads split as [B, S, N, D] then permuted to [B, N, S, D]: the form of the registered pattern
        q = self.q(h).view(B, S, self.heads, hd).permute(0, 2, 1, 3)
        k = self.k(h).view(B, S, self.heads, hd).permute(0, 2, 1, 3)
        v = self.v(h).view(B, S, self.heads, hd).permute(0, 2, 1, 3)
        att = torch.matmul(q, k.transpose(-2, -1)).div(math.sqrt(hd)).softmax(dim=-1).matmul(v)
        x = x + self.proj(att.permute(0, 2, 1, 3).reshape(B, S, D))
        return x + self.down(F.gelu(self.up(self.ln2(x))))


@pytest.mark.parametrize("dtype,dim", [(torch.float32, 256), (torch.bfloat16, 256), (torch.bfloat16, 512)])
def test_transformer_block_training_step(dtype, dim):
    from torch._inductor.utils import run_and_get_code

    announce(f"compile transformer block forward+backward {dtype} dim={dim}")
    torch.manual_seed(0)
    heads, hidden, B, S = 4, 1024, 4, 128
    ref_model = Block(dim, heads, hidden).to(DEV).to(dtype)
    model = Block(dim, heads, hidden).to(DEV).to(dtype)
    model.load_state_dict(ref_model.state_dict())
    x = torch.randn(B, S, dim, device=DEV).to(dtype)
    target = torch.randn(B, S, dim, device=DEV).to(dtype)

    def step(m, x):
        loss = F.mse_loss(m(x).float(), target.float())
        loss.backward()
        return loss

    loss_ref = step(ref_model, x)
    torch._dynamo.reset()
    # dynamic=False: the cases differ in width only, which would otherwise be taken for a dynamic
    # dimension from the second case on (and the fused attention op needs a static head dimension)
    compiled = torch.compile(model, dynamic=False)

    def run():
        return step(compiled, x)

    loss, codes = run_and_get_code(run)
    code = "\n".join(codes)
    assert code.count("generated_kernel(") >= 4, "forward and backward should both run generated kernels"
    assert "triton.jit" not in code and "@triton" not in code
    if dtype == torch.bfloat16 and dim // heads == 128:
        # head dimension 128 in bf16: the attention pattern is replaced by the fused op, forward and backward
        assert "npu_fa" in code and "npu_fa_backward" in code
    tol = dict(rtol=2e-3, atol=2e-4) if dtype == torch.float32 else dict(rtol=5e-2, atol=5e-2)
    torch.testing.assert_close(loss.float(), loss_ref.float(), **tol)
    for (name, p), (_, q) in zip(model.named_parameters(), ref_model.named_parameters()):
        assert p.grad is not None, name
        scale = max(q.grad.float().abs().max().item(), 1e-6)
        err = (p.grad.float() - q.grad.float()).abs().max().item()
        assert err <= (2e-3 if dtype == torch.float32 else 5e-2) * scale + 1e-6, f"{name}: {err} vs scale {scale}"


def test_layernorm_training_at_a_size_where_inductor_would_mix_reduction_orders():
    """From 5 M elements on, Inductor fuses a row reduction and a column reduction over the same
    tile into one Triton-shaped kernel (torch/_inductor/scheduler.py MixOrderReduction.can_fuse);
    this backend keeps them as a row kernel and a column sweep, and the step must compile and
    agree with eager (input, weight and bias gradients of LayerNorm on [8192, 1024])."""
    announce("compile layernorm forward+backward [8192,1024]")
    torch.manual_seed(0)
    x = torch.randn(8192, 1024, device=DEV, requires_grad=True)
    w = torch.randn(1024, device=DEV, requires_grad=True)
    b = torch.randn(1024, device=DEV, requires_grad=True)
    dy = torch.randn(8192, 1024, device=DEV)

    def step(x, w, b):
        for t_ in (x, w, b):
            t_.grad = None
        y = F.layer_norm(x, (1024,), w, b)
        y.backward(dy)
        return y.detach(), x.grad.clone(), w.grad.clone(), b.grad.clone()

    ref = step(x, w, b)
    torch._dynamo.reset()
    got = torch.compile(step, dynamic=False)(x, w, b)
    for g, r in zip(got, ref):
        torch.testing.assert_close(g, r, rtol=1e-4, atol=1e-4 * float(r.abs().max()))
