"""Backward of the fused attention forward (npu_graph::npu_fa_backward).

Two paths.  bf16 or fp16 with a head dimension up to 128 (a multiple of 8; smaller ones are padded with zero columns)
runs the fused MFMA
kernels (kernels.fused_attention_backward, csrc/mi/attention_bwd_w8.h).  Other shapes run the matrix
products as library GEMMs (torch.bmm, hipBLASLt underneath) on a bounded number of heads at a time
and move O(S^2) intermediates through HBM.  Both recompute the probabilities from the forward's
saved row statistics.  Definitions (per head, scores scaled by `scale`, causal mask optional), with m = softmax_max and
l = softmax_sum as saved by the forward:

    S  = Q K^T * scale                      P  = exp(S - m) / l          (masked entries: 0)
    dV = P^T dO                             dP = dO V^T
    D  = rowsum(dO * O)                     dS = P * (dP - D) * scale
    dQ = dS K                               dK = dS^T Q

The probabilities and dS are rounded to the operand type before they enter a GEMM, as a fused kernel would do;
all reductions and the softmax algebra are fp32.  Counterpart of the reference's call into
torch_npu.npu_fusion_attention_grad (reference inductor_x/npu_fusion_attention_graph.py:38-42).
"""
from __future__ import annotations

import torch

# heads processed per round: bounds the fp32 [heads, S, S] intermediates (two live at a time)
_SCORE_BYTES_BUDGET = 2 << 30
_GEMM_DTYPES = (torch.bfloat16, torch.float16, torch.float32)


def _bmm_f32(a, b):
    """Batched product with an fp32 result: fp32 accumulation output for 16-bit operands."""
    if a.dtype == torch.float32:
        return torch.bmm(a, b)
    return torch.bmm(a, b, out_dtype=torch.float32)


def _heads_per_round(heads: int, Sq: int, Sk: int = None) -> int:
    Sk = Sq if Sk is None else Sk
    return max(1, min(heads, _SCORE_BYTES_BUDGET // max(2 * Sq * Sk * 4, 1)))


def dropout_keep_mask(seed: int, first_head: int, heads: int, Sq: int, keep_prob: float, device, Sk: int = None):
    """The [heads, Sq, Sk] mask of kept probabilities for heads first_head .. first_head + heads - 1 of
    a call whose dropout seed is `seed`: a uniform draw per entry from a generator seeded with
    seed + first_head, kept where it is below keep_prob.  Forward and backward walk the heads in the
    same rounds (_heads_per_round) and so regenerate identical masks from the seed alone."""
    gen = torch.Generator(device=device)
    gen.manual_seed((int(seed) + int(first_head)) & ((1 << 63) - 1))
    return torch.rand(heads, Sq, Sq if Sk is None else Sk, device=device, generator=gen) < keep_prob


def _check_shapes(what: str, q, k, v, causal: bool):
    """q [B, N, Sq, D]; k and v [B, N, Sk, D]; a causal mask needs Sq == Sk."""
    if not (k.shape == v.shape and q.shape[:2] == k.shape[:2] and q.shape[3] == k.shape[3]):
        raise ValueError(f"attention {what}: q [B, N, Sq, D] and k, v [B, N, Sk, D] must agree in B, N and D")
    if causal and q.shape[2] != k.shape[2]:
        raise ValueError(f"attention {what}: a causal mask needs equal query and key lengths")


def _check_keep_prob(keep_prob: float) -> float:
    if not (0.0 <= keep_prob <= 1.0):
        raise ValueError(f"attention: keep_prob must lie in [0, 1], got {keep_prob}")
    return 0.0 if keep_prob == 0.0 else 1.0 / keep_prob


def _per_head(t, B: int, N: int, Sq: int, Sk: int, what: str):
    """A bias or mask given as [Sq, Sk] or broadcastable to [B, N, Sq, Sk], as a [B * N or 1, Sq, Sk] view
    (no copy when it broadcasts over batch and heads)."""
    if t.dim() == 2:
        t = t.view(1, 1, *t.shape)
    if t.dim() != 4 or t.shape[2:] != (Sq, Sk) or t.shape[0] not in (1, B) or t.shape[1] not in (1, N):
        raise ValueError(f"attention: {what} of shape {tuple(t.shape)} does not broadcast to [{B}, {N}, {Sq}, {Sk}]")
    if t.shape[0] == 1 and t.shape[1] == 1:
        return t.view(1, Sq, Sk)
    return t.expand(B, N, Sq, Sk).reshape(B * N, Sq, Sk)


def attention_forward_over_gemms(q, k, v, scale: float, causal: bool, keep_prob: float = 1.0, seed: int = 0,
                                 pse=None, atten_mask=None):
    """softmax(q k^T * scale [+ causal mask]) v with library GEMMs for shapes and element types the
    fused forward kernels do not cover (q [B, N, Sq, D], k and v [B, N, Sk, D]: any head dimension
    and sequence lengths, a causal mask needs Sq == Sk; bf16, fp16, fp32).
    Returns (out, softmax_max, softmax_sum) like kernels.fused_attention: the row statistics are
    fp32 [B, N, S, 8], the probabilities are rounded to the operand type before the second product
    and O(S^2) intermediates move through HBM, a bounded number of heads at a time.
    keep_prob < 1 drops probabilities after the softmax (dropout_keep_mask) and scales the kept ones
    by 1 / keep_prob; the row statistics are those of the undropped softmax.
    pse (a positional bias, [Sq, Sk] or broadcastable to [B, N, Sq, Sk]) is added to q k^T before the
    scaling and atten_mask (boolean or integer, non-zero = the key is hidden from the query) is
    applied after it -- softmax(mask(scale * (pse + q k^T))) as the fused op of the reference's
    device library documents it (call site: reference inductor_x/npu_fusion_attention_graph.py:31);
    a row with every key hidden gives zeros."""
    inv_keep = _check_keep_prob(keep_prob)
    for t in (q, k, v):
        if not (t.is_cuda and t.dtype in _GEMM_DTYPES and t.dtype == q.dtype and t.dim() == 4):
            raise ValueError("attention forward: q, k, v must be 4-D GPU tensors of one floating-point type")
    _check_shapes("forward", q, k, v, causal)
    B, N, S, D = q.shape
    Sk = k.shape[2]
    heads = B * N
    qh = q.contiguous().view(heads, S, D)
    kh, vh = (t.contiguous().view(heads, Sk, D) for t in (k, v))
    out = torch.empty_like(qh)
    smax = torch.empty(heads, S, dtype=torch.float32, device=q.device)
    ssum = torch.empty(heads, S, dtype=torch.float32, device=q.device)
    if heads and S and Sk == 0:
        raise ValueError("attention forward: no keys")
    if heads and S:
        chunk = _heads_per_round(heads, S, Sk)
        mask = torch.ones(S, S, dtype=torch.bool, device=q.device).triu_(1) if causal else None
        bias = _per_head(pse, B, N, S, Sk, "pse") if pse is not None else None
        hide = _per_head(atten_mask != 0, B, N, S, Sk, "atten_mask") if atten_mask is not None else None
        for h0 in range(0, heads, chunk):
            sl = slice(h0, min(h0 + chunk, heads))
            s = _bmm_f32(qh[sl], kh[sl].transpose(1, 2))
            if bias is not None:
                s.add_(bias if bias.shape[0] == 1 else bias[sl])
            s.mul_(scale)
            if mask is not None:
                s.masked_fill_(mask, float("-inf"))
            if hide is not None:
                s.masked_fill_(hide if hide.shape[0] == 1 else hide[sl], float("-inf"))
            m = s.amax(-1)
            if hide is not None:
                m = torch.where(torch.isinf(m), torch.zeros_like(m), m)  # rows with every key hidden
            p = s.sub_(m.unsqueeze(-1)).exp_()
            l = p.sum(-1)
            if hide is not None:
                l = torch.where(l == 0, torch.ones_like(l), l)
            smax[sl], ssum[sl] = m, l
            if keep_prob < 1.0:
                p.mul_(dropout_keep_mask(seed, h0, sl.stop - h0, S, keep_prob, q.device, Sk)).mul_(inv_keep)
            out[sl] = (_bmm_f32(p.to(q.dtype), vh[sl]) / l.unsqueeze(-1)).to(q.dtype)
    stats = lambda t: t.view(B, N, S, 1).expand(B, N, S, 8).contiguous()  # noqa: E731
    return out.view(B, N, S, D), stats(smax), stats(ssum)


def fused_attention_backward(q, k, v, out, dout, softmax_max, softmax_sum, scale: float, causal: bool,
                             use_kernels=None, keep_prob: float = 1.0, seed: int = 0, pse=None, atten_mask=None):
    """q, out, dout: [B, N, Sq, D] and k, v: [B, N, Sk, D] of one floating-point type; softmax_max /
    softmax_sum: [B, N, Sq, 8] fp32 from the forward.  Returns (dq, dk, dv) in that type.  use_kernels: None = fused
    kernels where they apply (bf16 or fp16, head dimension up to 128, one shape for q, k and v, no dropout, a
    sequence length that is a multiple of 64 or, under a causal mask, any; smaller head dimensions and causal
    lengths in between are zero-padded).
    keep_prob < 1 with the forward's seed regenerates the forward's dropout mask (GEMM path only).
    With pse or atten_mask the result has a fourth member, the gradient of pse in pse's own shape (None
    without pse); a mask alone runs on the fused kernels under the same shape limits, pse over GEMMs."""
    kernel_shape = (q.dim() == 4 and q.shape == k.shape and q.dtype in (torch.bfloat16, torch.float16)
                    and 0 < q.size(3) <= 128 and q.size(3) % 8 == 0 and q.size(2) > 0 and keep_prob == 1.0)
    masked_fit = (kernel_shape and pse is None and atten_mask is not None and atten_mask.is_cuda and atten_mask.dim() in (2, 4))
    # without a causal mask a length that is no multiple of 64 needs the padded keys hidden exactly: a bit mask
    ragged_fit = kernel_shape and pse is None and atten_mask is None and not causal and q.size(2) % 64 != 0
    if (masked_fit or ragged_fit) and use_kernels is not False:
        # The gradient kernels with a bit mask (one shape for q, k, v).  The length is padded to a multiple
        # of 64 with zero rows (statistics m = 0, l = 1); the mask hides the padded keys from every query
        # and, where the caller gave a mask, is that mask padded with "hidden".
        from . import kernels

        d, S = q.size(3), q.size(2)
        pad_d, pad_s = 128 - d, -S % 64
        Sp = S + pad_s
        widen = (lambda t: torch.nn.functional.pad(t, (0, pad_d, 0, pad_s))) if (pad_d or pad_s) else (lambda t: t.contiguous())  # noqa: E731
        smax, ssum = softmax_max.contiguous(), softmax_sum.contiguous()
        if pad_s:
            smax = torch.nn.functional.pad(smax, (0, 0, 0, pad_s), value=0.0)
            ssum = torch.nn.functional.pad(ssum, (0, 0, 0, pad_s), value=1.0)
        if atten_mask is not None:
            m4 = atten_mask.view(1, 1, *atten_mask.shape) if atten_mask.dim() == 2 else atten_mask
            hide = m4 if m4.dtype == torch.bool else m4 != 0
            if pad_s:
                hide = torch.nn.functional.pad(hide, (0, pad_s, 0, pad_s), value=True)
            packed = (kernels.attention_mask_bits(hide, q.size(0), q.size(1), Sp, Sp),
                      kernels.attention_mask_bits(hide.transpose(-1, -2), q.size(0), q.size(1), Sp, Sp))
            # the tiles of the other axis each block of 256 rows has to visit (a sliding window visits few)
            ranges = (kernels.attention_mask_tile_ranges(packed[0], Sp, Sp, causal),
                      kernels.attention_mask_tile_ranges(packed[1], Sp, Sp, causal, transposed=True))
        else:
            ranges = None
            # keys S .. Sp - 1 hidden from everybody: the same word row for every query (only the last key
            # tile has bits set); transposed, a padded key hides every query and a real key none
            tiles = Sp // 64
            words = torch.zeros(tiles, dtype=torch.int64, device=q.device)
            words[tiles - 1] = -1 << (S % 64)
            rows = words.view(1, 1, 1, tiles).expand(1, 1, Sp, tiles).contiguous().view(torch.uint8)
            cols = torch.zeros(Sp, tiles, dtype=torch.int64, device=q.device)
            cols[S:] = -1
            packed = (rows, cols.view(1, 1, Sp, tiles).view(torch.uint8))
        grads = kernels.fused_attention_backward(widen(q), widen(k), widen(v), widen(out), widen(dout), smax, ssum, scale, causal,
                                                 packed_masks=packed, tile_ranges=ranges)
        grads = tuple(g[:, :, :S, :d].contiguous() for g in grads) if (pad_d or pad_s) else grads
        return grads + (None,) if atten_mask is not None else grads
    if pse is not None or atten_mask is not None:
        if use_kernels:
            raise NotImplementedError("attention backward: the fused kernels take no bias, and a mask only for one shape of q, k, v")
        return _backward_over_gemms(q, k, v, out, dout, softmax_max, softmax_sum, scale, causal, keep_prob, seed,
                                    pse=pse, atten_mask=atten_mask)
    fits = kernel_shape  # (without a causal mask, lengths that are no multiple of 64 took the masked kernels above)
    if use_kernels is None:
        use_kernels = fits
    if use_kernels:
        if keep_prob != 1.0:
            raise NotImplementedError("attention backward: the fused kernels have no dropout")
        from . import kernels

        # A head dimension below 128 is padded with zero columns: scores, probabilities and
        # rowsum(dO * O) do not change, the extra gradient columns are zero and dropped.
        # Under a causal mask a sequence length that is no multiple of 64 is padded with zero rows
        # (statistics m = 0, l = 1): the mask hides every padded key from every real query, so its
        # probability is exactly zero, and a padded query has dO = 0 and Q = 0, so it adds nothing to
        # dV or dK; the padded rows of the results are dropped.  Without the mask a padded key would
        # get the probability exp(-logsumexp of the row), which times K = 0 is zero only while it
        # stays finite in the operand type: those lengths took the kernels with a bit mask above.
        d, S = q.size(3), q.size(2)
        pad_d, pad_s = 128 - d, -S % 64
        if pad_s and not causal:
            raise NotImplementedError("attention backward: without a causal mask a sequence length that is no multiple "
                                      "of 64 needs the masked kernels")
        if pad_d or pad_s:
            widen = lambda t: torch.nn.functional.pad(t, (0, pad_d, 0, pad_s))  # noqa: E731
        else:
            widen = lambda t: t.contiguous()  # noqa: E731
        smax, ssum = softmax_max.contiguous(), softmax_sum.contiguous()
        if pad_s:
            smax = torch.nn.functional.pad(smax, (0, 0, 0, pad_s), value=0.0)
            ssum = torch.nn.functional.pad(ssum, (0, 0, 0, pad_s), value=1.0)
        # up to 64 columns the kernels skip the matrix work on the zero half of the padded heads
        grads = kernels.fused_attention_backward(widen(q), widen(k), widen(v), widen(out), widen(dout), smax, ssum, scale, causal,
                                                 data_columns=64 if d <= 64 else 128)
        return tuple(g[:, :, :S, :d].contiguous() for g in grads) if (pad_d or pad_s) else grads
    return _backward_over_gemms(q, k, v, out, dout, softmax_max, softmax_sum, scale, causal, keep_prob, seed)


def _backward_over_gemms(q, k, v, out, dout, softmax_max, softmax_sum, scale: float, causal: bool,
                         keep_prob: float = 1.0, seed: int = 0, pse=None, atten_mask=None):
    # With dropout, Pd = P * keep / keep_prob takes P's place in dV = Pd^T dO, and dP = (dO V^T) * keep /
    # keep_prob; D = rowsum(dO * O) = rowsum(P * dP) still holds because O = Pd V.
    inv_keep = _check_keep_prob(keep_prob)
    for t in (q, k, v, out, dout):
        if not (t.is_cuda and t.dtype in _GEMM_DTYPES and t.dtype == q.dtype and t.dim() == 4):
            raise ValueError("attention backward: q, k, v, out, dout must be 4-D GPU tensors of one floating-point type")
    _check_shapes("backward", q, k, v, causal)
    if not (q.shape == out.shape == dout.shape):
        raise ValueError("attention backward: q, out and dout must share one [B, N, Sq, D] shape")
    B, N, S, D = q.shape
    Sk = k.shape[2]
    if softmax_max.shape != (B, N, S, 8) or softmax_sum.shape != (B, N, S, 8):
        raise ValueError("attention backward: softmax statistics must be [B, N, S, 8]")
    heads = B * N
    qh, oh, doh = (t.contiguous().view(heads, S, D) for t in (q, out, dout))
    kh, vh = (t.contiguous().view(heads, Sk, D) for t in (k, v))
    m = softmax_max.reshape(heads, S, 8)[..., 0].contiguous()
    l = softmax_sum.reshape(heads, S, 8)[..., 0].contiguous()
    dq = torch.empty_like(qh)
    dk = torch.empty_like(kh)
    dv = torch.empty_like(vh)
    if heads == 0 or S == 0 or Sk == 0:
        return dq.view(B, N, S, D), dk.zero_().view(B, N, Sk, D), dv.zero_().view(B, N, Sk, D)
    chunk = _heads_per_round(heads, S, Sk)
    mask = None
    if causal:
        mask = torch.ones(S, S, dtype=torch.bool, device=q.device).triu_(1)
    extras = pse is not None or atten_mask is not None
    bias = _per_head(pse, B, N, S, Sk, "pse") if pse is not None else None
    hide = _per_head(atten_mask != 0, B, N, S, Sk, "atten_mask") if atten_mask is not None else None
    dpse = torch.zeros(heads, S, Sk, dtype=torch.float32, device=q.device) if pse is not None else None
    for h0 in range(0, heads, chunk):
        sl = slice(h0, min(h0 + chunk, heads))
        qc, kc, vc, oc, doc = qh[sl], kh[sl], vh[sl], oh[sl], doh[sl]
        s = _bmm_f32(qc, kc.transpose(1, 2))
        if bias is not None:
            s.add_(bias if bias.shape[0] == 1 else bias[sl])
        # P = exp(S * scale - m) / l, masked entries exactly zero
        s.mul_(scale).sub_(m[sl].unsqueeze(-1))
        if mask is not None:
            s.masked_fill_(mask, float("-inf"))
        if hide is not None:
            s.masked_fill_(hide if hide.shape[0] == 1 else hide[sl], float("-inf"))
        p = s.exp_().div_(l[sl].unsqueeze(-1))
        dp = _bmm_f32(doc, vc.transpose(1, 2))
        if keep_prob < 1.0:
            keep = dropout_keep_mask(seed, h0, sl.stop - h0, S, keep_prob, q.device, Sk)
            dv[sl] = torch.bmm((p * keep).mul_(inv_keep).to(q.dtype).transpose(1, 2), doc)
            dp.mul_(keep).mul_(inv_keep)
            del keep
        else:
            dv[sl] = torch.bmm(p.to(q.dtype).transpose(1, 2), doc)
        delta = (doc.float() * oc.float()).sum(-1, keepdim=True)
        ds = p.mul_(dp.sub_(delta)).mul_(scale)
        if dpse is not None:
            dpse[sl] = ds  # d loss / d (q k^T) is also d loss / d pse: the bias sits beside the product
        ds16 = ds.to(q.dtype)
        dq[sl] = torch.bmm(ds16, kc)
        dk[sl] = torch.bmm(ds16.transpose(1, 2), qc)
    grads = (dq.view(B, N, S, D), dk.view(B, N, Sk, D), dv.view(B, N, Sk, D))
    if not extras:
        return grads
    if dpse is not None:
        # fold the [B, N, S, S] gradient onto the axes pse broadcast over
        g = dpse.view(B, N, S, Sk)
        shape = pse.shape if pse.dim() == 4 else (1, 1) + tuple(pse.shape)
        for axis in (0, 1):
            if shape[axis] == 1 and g.shape[axis] != 1:
                g = g.sum(axis, keepdim=True)
        dpse = g.reshape(pse.shape).to(pse.dtype)
    return grads + (dpse,)
