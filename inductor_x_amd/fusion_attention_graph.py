"""Fused-attention custom op and graph pattern.

Counterpart of reference inductor_x/npu_fusion_attention_graph.py: the same
operator library and schemas (`npu_graph::npu_fa`, `npu_graph::npu_fa_backward`,
:13-18), a device implementation (:20-42), Meta implementations giving the
output shapes (:45-86), an autograd.Function wrapper (:88-123), the public
npu_fusion_attention_graph() (:125-132) and the replacement of
    matmul(q, k^T).div(inv_scale).softmax(-1)[.dropout].matmul(v)
with q, k, v given as [B, S, N, D] and permuted (0, 2, 1, 3) (:134-230).

The device implementation runs the MFMA kernel of this package.  As in the
reference the op receives the *inverse* scale from the pattern and inverts it
(:20-35, :162).  The reference's pattern carries no mask; a causal mask enters
through the op's own arguments: sparse_mode 2 or 3, or next_tockens == 0 with
pre_tockens covering the sequence.  Supported: layouts "BNSD", "BSH", "SBH" ("BSH" and "SBH" are
viewed as [B, N, S, D], copied once into that order for the kernels and copied back).  The fused
kernel takes bf16 and fp16 operands with a head dimension that is a multiple of 8 up to 128
(smaller heads are zero-padded to 128) at any query and key lengths, also with a general mask (any
type, non-zero = hidden); a positional bias (pse), fp32 operands, other
head dimensions and dropout (keep_prob < 1) run the same mathematics over library GEMMs.  pre_tockens / next_tockens
short of the sequence (sparse_mode 0) describe a sliding window, key j visible to query i when
-pre_tockens <= j - i <= next_tockens: it becomes a mask for the fused kernels, joined with atten_mask if one is
given.  Padding masks, prefixes, variable sequence lengths and the other sparse modes raise.
The backward op recomputes the probabilities from the saved row statistics inside fused gradient
kernels (bf16 or fp16, head dimension up to 128, one shape for q, k, v;
kernels.fused_attention_backward) and falls back to the GEMM formulation otherwise
(attention_backward.py), which also returns the gradient of pse; a general mask runs the fused
gradient kernels too; the training variant of the
pattern is registered beside the inference one.
"""
from __future__ import annotations

import functools

import torch
from torch.autograd import Function
from torch.library import Library

TOKEN_MAX = 2147483647

npu_def = Library("npu_graph", "DEF")
gpu_lib = Library("npu_graph", "IMPL", "CUDA")
meta_lib = Library("npu_graph", "IMPL", "Meta")

npu_def.define(
    "npu_fa(Tensor query, Tensor key, Tensor value, int head_num, str input_layout, Tensor? pse=None, "
    "Tensor? padding_mask=None, Tensor? atten_mask=None, float scale=1., float keep_prob=1., "
    "int pre_tockens=2147483647, int next_tockens=2147483647, int inner_precise=0, int[]? prefix=None, "
    "int[]? actual_seq_qlen=None, int[]? actual_seq_kvlen=None, int sparse_mode=0, bool gen_mask_parallel=True, "
    "bool sync=False) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)"
)
npu_def.define(
    "npu_fa_backward(Tensor query, Tensor key, Tensor value, Tensor dy, int head_num, str input_layout, *, "
    "Tensor? pse=None, Tensor? padding_mask=None, Tensor? atten_mask=None, Tensor? softmax_max=None, "
    "Tensor? softmax_sum=None, Tensor? softmax_in=None, Tensor? attention_in=None, float scale_value=1., "
    "float keep_prob=1., int pre_tockens=2147483647, int next_tockens=2147483647, int inner_precise=0, "
    "Tensor? seed=None, Tensor? offset=None, Tensor? numels=None, int[]? prefix=None, int[]? actual_seq_qlen=None, "
    "int[]? actual_seq_kvlen=None, int sparse_mode=0, bool gen_mask_parallel=True, bool sync=False) "
    "-> (Tensor, Tensor, Tensor, Tensor)"
)


LAYOUTS = ("BNSD", "BSH", "SBH")


def _to_bnsd(t, head_num: int, layout: str):
    """View a tensor given in `layout` as [B, N, S, D] (reference
    inductor_x/npu_fusion_attention_graph.py:49-61 reads B and S out of the same three layouts)."""
    if layout == "BNSD":
        return t
    if t.dim() != 3 or t.size(2) % head_num:
        raise ValueError(f"npu_fa: layout {layout} needs a 3-d tensor whose hidden size is a multiple of "
                         f"head_num {head_num}, got {tuple(t.shape)}")
    d = t.size(2) // head_num
    if layout == "BSH":
        return t.view(t.size(0), t.size(1), head_num, d).permute(0, 2, 1, 3)
    return t.view(t.size(0), t.size(1), head_num, d).permute(1, 2, 0, 3)  # SBH


def _from_bnsd(t, layout: str):
    """[B, N, S, D] back to `layout`, contiguous."""
    if layout == "BNSD":
        return t
    b, n, s, d = t.shape
    if layout == "BSH":
        return t.permute(0, 2, 1, 3).reshape(b, s, n * d)
    return t.permute(2, 0, 1, 3).reshape(s, b, n * d)  # SBH


def _check_layout(op: str, layout: str):
    if layout not in LAYOUTS:
        raise NotImplementedError(f"{op}: layout {layout!r} (supported: {', '.join(LAYOUTS)})")


@functools.lru_cache(maxsize=4)
def _band_mask(sq: int, sk: int, pre_tockens: int, next_tockens: int, device: str) -> torch.Tensor:
    """[sq, sk] bool, True = hidden: key j is visible to query i when -pre_tockens <= j - i <= next_tockens."""
    dist = torch.arange(sk, device=device).view(1, sk) - torch.arange(sq, device=device).view(sq, 1)
    return (dist > next_tockens) | (dist < -pre_tockens)


def _mask_plan(query, key, atten_mask, pre_tockens: int, next_tockens: int, sparse_mode: int):
    """(causal, mask) for the op's mask arguments.  causal: the plain causal mask, which the kernels apply
    themselves (sparse_mode 2 or 3, or next_tockens == 0 with pre_tockens covering the sequence; a mask tensor,
    if given, is then the compressed triangle of the reference's device library and is not read).  Otherwise
    mask is what hides keys: a given atten_mask as it stands, a band when pre_tockens / next_tockens are short
    of the sequence (a sliding window: key j visible to query i when -pre_tockens <= j - i <= next_tockens),
    or both."""
    sq, sk = query.size(2), key.size(2)
    if sparse_mode in (2, 3):
        return True, None
    if sparse_mode != 0:
        raise NotImplementedError("npu_fa: sparse modes other than 0, 2 and 3 are not supported")
    if next_tockens == 0 and pre_tockens >= sq:
        return True, None
    mask = atten_mask
    if next_tockens < sk - 1 or pre_tockens < sq - 1:
        band = _band_mask(sq, sk, max(int(pre_tockens), -TOKEN_MAX), max(int(next_tockens), -TOKEN_MAX), str(query.device))
        if mask is None:
            mask = band
        else:
            hide = mask if mask.dtype == torch.bool else mask != 0
            mask = hide | (band if hide.dim() == 2 else band.view(1, 1, sq, sk))
    return False, mask


def npu_fa_gpu(query, key, value, head_num, input_layout, pse=None, padding_mask=None, atten_mask=None, scale=1.0,
               keep_prob=1.0, pre_tockens=TOKEN_MAX, next_tockens=TOKEN_MAX, inner_precise=0, prefix=None,
               actual_seq_qlen=None, actual_seq_kvlen=None, sparse_mode=0, gen_mask_parallel=True, sync=False):
    from . import kernels

    _check_layout("npu_fa", input_layout)
    layout = input_layout
    query, key, value = (_to_bnsd(t, head_num, layout) for t in (query, key, value))
    if padding_mask is not None or prefix or actual_seq_qlen or actual_seq_kvlen:
        raise NotImplementedError("npu_fa: padding_mask / prefix / variable sequence lengths")
    if not (0.0 <= keep_prob <= 1.0):
        raise ValueError(f"npu_fa: keep_prob {keep_prob} outside [0, 1]")
    if query.size(1) != head_num:
        raise ValueError(f"npu_fa: head_num {head_num} does not match query of shape {tuple(query.shape)}")
    if scale == 0:
        raise ZeroDivisionError("npu_fa: the inverse scale factor is zero")
    # the graph pattern passes the divisor of the scores; the kernel multiplies
    real_scale = 1.0 / scale
    causal, mask = _mask_plan(query, key, atten_mask, pre_tockens, next_tockens, sparse_mode)
    seed = numels = 0
    head_dim = query.size(3)
    mask_fits = mask is None or (mask.is_cuda and mask.dim() in (2, 4))
    if (pse is None and mask_fits and keep_prob == 1.0 and query.dtype in (torch.bfloat16, torch.float16) and head_dim <= 128 and head_dim % 8 == 0
            and head_dim > 0 and query.size(2) > 0 and key.size(2) > 0 and (not causal or query.size(2) == key.size(2))):
        # the MFMA kernel: bf16 or fp16, head dimension 128, any sequence lengths.  A smaller head
        # dimension is padded with zero columns (scores and statistics do not change, the extra output
        # columns are dropped); up to 64 columns the kernel skips the matrix work on the zero half
        pad = 128 - head_dim
        widen = (lambda t: torch.nn.functional.pad(t, (0, pad))) if pad else (lambda t: t.contiguous())  # noqa: E731
        out, smax, ssum = kernels.fused_attention(widen(query), widen(key), widen(value), real_scale, causal,
                                                  data_columns=64 if head_dim <= 64 else 128, mask=mask)
        if pad:
            out = out[..., :head_dim].contiguous()
    else:
        # head dimensions above 128 or not a multiple of 8, fp32, dropout, a positional bias: the same
        # mathematics over library GEMMs.  The dropout seed comes from torch's CPU generator (torch.manual_seed makes a
        # run repeatable) and travels to the backward in the op's seed output, as in the reference's op.
        from .attention_backward import attention_forward_over_gemms

        if keep_prob < 1.0:
            seed = int(torch.randint(0, 1 << 62, (1,), dtype=torch.int64).item())
            numels = query.size(0) * query.size(1) * query.size(2) * key.size(2)
        out, smax, ssum = attention_forward_over_gemms(query, key, value, real_scale, causal, keep_prob, seed,
                                                       pse=pse, atten_mask=mask)
    softmax_out = torch.empty([0], dtype=query.dtype, device=query.device)
    word = lambda v: torch.tensor([v], dtype=torch.int64)  # noqa: E731  seed / offset / numels live on the host
    return _from_bnsd(out, layout), smax, ssum, softmax_out, word(seed), word(0), word(numels)


gpu_lib.impl("npu_fa", npu_fa_gpu)


def npu_fa_backward_gpu(query, key, value, dy, head_num, input_layout, *, pse=None, padding_mask=None,
                        atten_mask=None, softmax_max=None, softmax_sum=None, softmax_in=None, attention_in=None,
                        scale_value=1.0, keep_prob=1.0, pre_tockens=TOKEN_MAX, next_tockens=TOKEN_MAX,
                        inner_precise=0, seed=None, offset=None, numels=None, prefix=None, actual_seq_qlen=None,
                        actual_seq_kvlen=None, sparse_mode=0, gen_mask_parallel=True, sync=False):
    """Gradients of npu_fa (reference inductor_x/npu_fusion_attention_graph.py:38-42: like the forward,
    the op receives the inverse scale and inverts it)."""
    from .attention_backward import fused_attention_backward

    _check_layout("npu_fa_backward", input_layout)
    layout = input_layout
    if padding_mask is not None or prefix or actual_seq_qlen or actual_seq_kvlen:
        raise NotImplementedError("npu_fa_backward: padding_mask / prefix / variable sequence lengths")
    if not (0.0 <= keep_prob <= 1.0):
        raise ValueError(f"npu_fa_backward: keep_prob {keep_prob} outside [0, 1]")
    if keep_prob < 1.0 and seed is None:
        raise ValueError("npu_fa_backward: dropout needs the forward's seed")
    if softmax_max is None or softmax_sum is None or attention_in is None:
        raise ValueError("npu_fa_backward: needs softmax_max, softmax_sum and attention_in from the forward")
    if scale_value == 0:
        raise ZeroDivisionError("npu_fa_backward: the inverse scale factor is zero")
    query, key, value, attention_in, dy = (
        _to_bnsd(t, head_num, layout).contiguous() for t in (query, key, value, attention_in, dy)
    )
    causal, mask = _mask_plan(query, key, atten_mask, pre_tockens, next_tockens, sparse_mode)
    grads = fused_attention_backward(
        query, key, value, attention_in, dy, softmax_max, softmax_sum, 1.0 / scale_value, causal,
        keep_prob=keep_prob, seed=int(seed.item()) if keep_prob < 1.0 else 0, pse=pse, atten_mask=mask,
    )
    dq, dk, dv = (_from_bnsd(t, layout) for t in grads[:3])
    dpse = grads[3] if len(grads) > 3 and grads[3] is not None else torch.empty([0], dtype=query.dtype, device=query.device)
    return dq, dk, dv, dpse


gpu_lib.impl("npu_fa_backward", npu_fa_backward_gpu)


def npu_fa_meta(query, key, value, head_num, input_layout, pse=None, padding_mask=None, atten_mask=None, scale=1.0,
                keep_prob=1.0, pre_tockens=TOKEN_MAX, next_tockens=TOKEN_MAX, inner_precise=0, prefix=None,
                actual_seq_qlen=None, actual_seq_kvlen=None, sparse_mode=0, gen_mask_parallel=True, sync=False):
    B, S1 = query.size(0), query.size(2)
    if input_layout == "BSH":
        B, S1 = query.size(0), query.size(1)
    if input_layout == "SBH":
        B, S1 = query.size(1), query.size(0)
    dev = query.device
    return (
        torch.empty_like(query).contiguous(),
        torch.empty([B, head_num, S1, 8], dtype=torch.float32, device=dev),
        torch.empty([B, head_num, S1, 8], dtype=torch.float32, device=dev),
        torch.empty([0], dtype=query.dtype, device=dev),
        torch.empty([1], dtype=torch.int64, device="meta"),
        torch.empty([1], dtype=torch.int64, device="meta"),
        torch.empty([1], dtype=torch.int64, device="meta"),
    )


meta_lib.impl("npu_fa", npu_fa_meta)


def npu_fa_backward_meta(query, key, value, dy, head_num, input_layout, *, pse=None, padding_mask=None,
                         atten_mask=None, softmax_max=None, softmax_sum=None, softmax_in=None, attention_in=None,
                         scale_value=1.0, keep_prob=1.0, pre_tockens=TOKEN_MAX, next_tockens=TOKEN_MAX,
                         inner_precise=0, seed=None, offset=None, numels=None, prefix=None, actual_seq_qlen=None,
                         actual_seq_kvlen=None, sparse_mode=0, gen_mask_parallel=True, sync=False):
    return (
        torch.empty_like(query).contiguous(),
        torch.empty_like(key).contiguous(),
        torch.empty_like(value).contiguous(),
        torch.empty_like(pse).contiguous() if pse is not None else torch.empty([0], dtype=query.dtype, device=query.device),
    )


meta_lib.impl("npu_fa_backward", npu_fa_backward_meta)


class GraphAttentionFunction(Function):
    """autograd wrapper of npu_graph::npu_fa (reference
    inductor_x/npu_fusion_attention_graph.py:88-123)."""

    @staticmethod
    def forward(ctx, query, key, value, head_num, input_layout, pse=None, padding_mask=None, atten_mask=None,
                scale=1.0, keep_prob=1.0, pre_tockens=TOKEN_MAX, next_tockens=TOKEN_MAX, inner_precise=0,
                prefix=None, actual_seq_qlen=None, actual_seq_kvlen=None, sparse_mode=0, gen_mask_parallel=True,
                sync=False):
        res = torch.ops.npu_graph.npu_fa(
            query, key, value, head_num, input_layout, pse=pse, padding_mask=padding_mask, atten_mask=atten_mask,
            scale=scale, keep_prob=keep_prob, pre_tockens=pre_tockens, next_tockens=next_tockens,
            inner_precise=inner_precise, prefix=prefix, actual_seq_qlen=actual_seq_qlen,
            actual_seq_kvlen=actual_seq_kvlen, sparse_mode=sparse_mode, gen_mask_parallel=gen_mask_parallel, sync=sync,
        )
        ctx.save_for_backward(query, key, value, pse, padding_mask, atten_mask, res[1], res[2], res[3], res[0],
                              res[4], res[5], res[6])
        ctx.attrs = dict(head_num=head_num, input_layout=input_layout, scale=scale, keep_prob=keep_prob,
                         pre_tockens=pre_tockens, next_tockens=next_tockens, inner_precise=inner_precise,
                         prefix=prefix, actual_seq_qlen=actual_seq_qlen, actual_seq_kvlen=actual_seq_kvlen,
                         sparse_mode=sparse_mode, gen_mask_parallel=gen_mask_parallel, sync=sync)
        return res

    @staticmethod
    def backward(ctx, grad0, *unused):
        (query, key, value, pse, padding_mask, atten_mask, smax, ssum, sout, out, seed, offset, numels) = ctx.saved_tensors
        a = ctx.attrs
        dq, dk, dv, dpse = torch.ops.npu_graph.npu_fa_backward(
            query, key, value, grad0, a["head_num"], a["input_layout"], pse=pse, padding_mask=padding_mask,
            atten_mask=atten_mask, softmax_max=smax, softmax_sum=ssum, softmax_in=sout, attention_in=out,
            scale_value=a["scale"], keep_prob=a["keep_prob"], pre_tockens=a["pre_tockens"],
            next_tockens=a["next_tockens"], inner_precise=a["inner_precise"], seed=seed, offset=offset, numels=numels,
            prefix=a["prefix"], actual_seq_qlen=a["actual_seq_qlen"], actual_seq_kvlen=a["actual_seq_kvlen"],
            sparse_mode=a["sparse_mode"], gen_mask_parallel=a["gen_mask_parallel"], sync=a["sync"],
        )
        return (dq, dk, dv, None, None, dpse if pse is not None else None) + (None,) * 13


def npu_fusion_attention_graph(query, key, value, head_num, input_layout, pse=None, padding_mask=None,
                               atten_mask=None, scale=1.0, keep_prob=1.0, pre_tockens=TOKEN_MAX,
                               next_tockens=TOKEN_MAX, inner_precise=0, prefix=None, actual_seq_qlen=None,
                               actual_seq_kvlen=None, sparse_mode=0, gen_mask_parallel=True, sync=False):
    """Public entry (reference inductor_x/npu_fusion_attention_graph.py:125-132).
    `scale` is the divisor applied to the scores, as the graph pattern passes it."""
    return GraphAttentionFunction.apply(
        query, key, value, head_num, input_layout, pse, padding_mask, atten_mask, scale, keep_prob, pre_tockens,
        next_tockens, inner_precise, prefix, actual_seq_qlen, actual_seq_kvlen, sparse_mode, gen_mask_parallel, sync,
    )


# ---------------------------------------------------------------------------
# graph pattern
# ---------------------------------------------------------------------------
def _attention_pattern_1(query, key, value, inv_scale_factor, dropout_p):
    q = query.permute(0, 2, 1, 3)
    k = key.permute(0, 2, 1, 3)
    v = value.permute(0, 2, 1, 3)
    return torch.nn.functional.dropout(
        torch.matmul(q, k.transpose(-2, -1)).div(inv_scale_factor).softmax(dim=-1), p=dropout_p
    ).matmul(v)


def _attention_replacement_1(query, key, value, inv_scale_factor, dropout_p):
    from torch._dynamo.utils import counters

    counters["inductor"]["fuse_attention"] += 1
    head_num = query.size(2)
    return npu_fusion_attention_graph(
        query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2), head_num, "BNSD", None,
        atten_mask=None, scale=inv_scale_factor, keep_prob=1.0 - dropout_p,
    )[0]


def _extra_check(match, training: bool = False) -> bool:
    """Only rewrite what the fused kernels run; anything else stays on Inductor's own path.
    Inference graphs: bf16 or fp16 GPU tensors [B, S, N, 128], any sequence lengths, key and value of
    one shape that may differ from the query's in its length (cross attention).  Training graphs,
    whose backward runs the fused gradient kernels: query, key and value of one shape.  Either way the divisor of the scores, when it is a
    constant, must be positive and finite."""
    try:
        q = match.kwargs["query"].meta["val"]
        k = match.kwargs["key"].meta["val"]
        v = match.kwargs["value"].meta["val"]
    except Exception:
        return False
    if not (q.device.type == "cuda" and q.dim() == 4 and q.size(3) == 128 and q.size(1) > 0):
        return False
    if q.dtype not in (torch.bfloat16, torch.float16):
        return False
    if training and tuple(k.shape) != tuple(q.shape):
        return False
    if k.dim() != 4 or k.size(1) <= 0 or (k.size(0), k.size(2), k.size(3)) != (q.size(0), q.size(2), q.size(3)):
        return False
    if tuple(v.shape) != tuple(k.shape):
        return False
    for t in (k, v):
        if t.dtype != q.dtype or t.device != q.device:
            return False
    # the divisor of the scores: a keyword of the match when the pattern captured it, otherwise the
    # second operand of the division node that was matched
    divisors = [match.kwargs.get("inv_scale_factor")]
    for node in getattr(match, "nodes", ()):
        if getattr(node, "target", None) in (torch.ops.aten.div.Tensor, torch.ops.aten.div.Scalar) and len(node.args) > 1:
            divisors.append(node.args[1])
    for divisor in divisors:
        if isinstance(divisor, (int, float)) and not (divisor > 0 and divisor != float("inf")):
            return False
    return True


_registered = False


def register_fx_pass() -> None:
    """Register the replacement with Inductor's joint-graph pattern pass
    (reference inductor_x/npu_fusion_attention_graph.py:134-230), for inference and for
    training graphs.  Patterns with dropout are not rewritten: the op would serve them over library
    GEMMs with O(S^2) traffic, slower than the attention Inductor picks for them itself."""
    global _registered
    if _registered:
        return
    _registered = True
    from torch._inductor.fx_passes import joint_graph
    from torch._inductor.fx_passes.fuse_attention import partialize_and_update_signature
    from torch._inductor.pattern_matcher import fwd_only, init_once_fakemode, joint_fwd_bwd, register_replacement

    @init_once_fakemode
    def _init():
        device = "cuda" if torch.cuda.is_available() else "cpu"
        c = functools.partial(torch.tensor, 2.0, device=device, dtype=torch.float)
        pattern = partialize_and_update_signature(_attention_pattern_1, dropout_p=0.0)
        replacement = partialize_and_update_signature(_attention_replacement_1, dropout_p=0.0)
        # The search function is traced once per element type: a softmax of 16-bit tensors
        # decomposes with conversions to fp32 and back that the fp32 trace does not contain, and
        # bf16 is the type the kernels run (the reference traces fp32 only, :218-224); and once more
        # with a batch of one, for which the batched products trace to different view operations
        # (Inductor's own attention patterns carry the same second variant).
        for dtype in (torch.float, torch.bfloat16, torch.half):
            for batch in (2, 1):
                g = functools.partial(torch.empty, (batch, 4, 8, 16), device=device, dtype=dtype)
                register_replacement(
                    pattern, replacement, [g(), g(), g(), c()], fwd_only, joint_graph.patterns,
                    extra_check=_extra_check, scalar_workaround={}, skip_duplicates=True,
                )
                # training: the same search function traced with its backward; the replacement's
                # autograd.Function supplies npu_fa_backward (reference :196-204, without dropout)
                gr = functools.partial(torch.empty, (batch, 4, 8, 16), device=device, dtype=dtype, requires_grad=True)
                register_replacement(
                    pattern, replacement, [gr(), gr(), gr(), c()], joint_fwd_bwd, joint_graph.patterns,
                    extra_check=functools.partial(_extra_check, training=True), scalar_workaround={},
                    skip_duplicates=True,
                )

    original_lazy_init = joint_graph.lazy_init

    @functools.wraps(original_lazy_init)
    def lazy_init_with_attention():
        # before Inductor's own attention patterns: a pattern pass tries the entries for a node in
        # the order of their registration, and Inductor's first pattern (the same products without
        # the permutes) would otherwise claim the match for scaled_dot_product_attention.  The
        # reference gets the same order by registering at import time (:233).
        _init()
        original_lazy_init()

    joint_graph.lazy_init = lazy_init_with_attention
