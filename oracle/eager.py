"""Eager FlashBias attention oracle (test infrastructure, never shipped).

Restates the reference's eager path ``attention_torch``
(``flash_bias/attention_func.py:16-55``): scores laid out (B, Lq, H, Lk), multiplied
by ``softmax_scale``, dense bias (B, H, Lq, Lk) added, top-left aligned causal fill
with -inf, softmax over keys, weighted sum of V.  The dense bias is the product of the
low-rank factors, ``q_bias @ k_bias^T`` (``flash_bias/benchmark.py:43``), optionally
plus the additive mask of ``flash_bias/flash_bias_triton.py:263-282``.

Tensors use the reference layout: q (B, Lq, H, d); k, v (B, Lk, H, d);
q_bias (B|1, Lq, H|1, r); k_bias (B|1, Lk, H|1, r); mask broadcastable to (B, H, Lq, Lk).
"""
import math

import torch


def default_scale(d):
    """``softmax_scale or 1/sqrt(d)`` -- flash_bias/flash_bias_triton.py:1110."""
    return 1.0 / math.sqrt(d)


def materialize_bias(q_bias, k_bias, batch, nheads):
    """Dense (B, H, Lq, Lk) bias from (B|1, L, H|1, r) factors (benchmark.py:43)."""
    qb = q_bias.expand(batch, q_bias.shape[1], nheads, q_bias.shape[3]).permute(0, 2, 1, 3)
    kb = k_bias.expand(batch, k_bias.shape[1], nheads, k_bias.shape[3]).permute(0, 2, 1, 3)
    return qb @ kb.transpose(-1, -2)


def logits(q, k, softmax_scale, bias=None, causal=False):
    """Pre-softmax scores in (B, Lq, H, Lk) layout (attention_func.py:30-47)."""
    lq, lk = q.shape[1], k.shape[1]
    s = torch.einsum("bqnh,bknh->bqnk", q, k) * softmax_scale
    if bias is not None:
        s = s + bias.permute(0, 2, 1, 3)
    if causal:
        # top-left aligned: key j is visible from query i iff j <= i (attention_func.py:44-47)
        hidden = torch.ones(lq, lk, device=q.device).triu(1).bool()
        s = s.masked_fill(hidden[None, :, None, :], float("-inf"))
    return s


def attention_eager(q, k, v, softmax_scale, bias=None, causal=False):
    """softmax(scale q k^T + bias) v, output (B, Lq, H, d) (attention_func.py:16-55)."""
    p = torch.softmax(logits(q, k, softmax_scale, bias, causal), dim=-1)
    return torch.einsum("bqnk,bknh->bqnh", p, v)


def _dense_bias(q, q_bias, k_bias, mask):
    batch, _, nheads, _ = q.shape
    bias = None
    if q_bias is not None:
        bias = materialize_bias(q_bias, k_bias, batch, nheads)
    if mask is not None:
        m = mask.to(q.dtype).expand(batch, nheads, q.shape[1], -1)
        bias = m if bias is None else bias + m
    return bias


def flashbias_eager(q, k, v, q_bias=None, k_bias=None, mask=None, causal=False,
                    softmax_scale=None, dtype=torch.float32, return_lse=False):
    """The oracle for ``flash_bias_func``: same argument order and meaning
    (flash_bias/flash_bias_triton.py:1347), computed eagerly in ``dtype`` from the given
    (already dtype-rounded) inputs.  LSE is the natural-log row normaliser
    (flash_bias_triton.py:323), shape (B, H, Lq)."""
    scale = softmax_scale or default_scale(q.shape[-1])
    q, k, v = (t.to(dtype) for t in (q, k, v))
    if q_bias is not None:
        q_bias, k_bias = q_bias.to(dtype), k_bias.to(dtype)
    bias = _dense_bias(q, q_bias, k_bias, mask)
    s = logits(q, k, scale, bias, causal)
    o = torch.einsum("bqnk,bknh->bqnh", torch.softmax(s, dim=-1), v)
    if return_lse:
        return o, torch.logsumexp(s, dim=-1).permute(0, 2, 1)
    return o


def flashbias_eager_grads(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, do,
                          dtype=torch.float32):
    """(o, dq, dk, dv, dq_bias, dk_bias) by autograd through the eager path with upstream
    gradient ``do``; factor grads come out already reduced over broadcast dims.  This is
    the recipe of flash_bias/benchmark.py:65-88 with the dense-bias grad folded through
    ``bias = q_bias k_bias^T``."""
    leaves = [t.detach().to(dtype).requires_grad_(True) for t in (q, k, v)]
    has_bias = q_bias is not None
    if has_bias:
        leaves += [t.detach().to(dtype).requires_grad_(True) for t in (q_bias, k_bias)]
    qq, kk, vv = leaves[:3]
    qb, kb = (leaves[3], leaves[4]) if has_bias else (None, None)
    o = flashbias_eager(qq, kk, vv, qb, kb, mask, causal, softmax_scale, dtype=dtype)
    grads = torch.autograd.grad(o, leaves, do.to(dtype))
    if not has_bias:
        grads = tuple(grads) + (None, None)
    return (o.detach(),) + tuple(grads)


def flashbias_eager_sliced(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, do=None,
                           dtype=torch.float32):
    """Same results as the two functions above, one (batch, head) slice at a time so that
    the (Lq, Lk) intermediates stay small at long sequence lengths.  Factors must be
    full-shape (no broadcast dims) when ``do`` is given."""
    batch, lq, nheads, d = q.shape
    o = torch.empty(batch, lq, nheads, d, dtype=dtype)
    outs = None
    if do is not None:
        outs = [torch.zeros_like(t, dtype=dtype) for t in (q, k, v)]
        if q_bias is not None:
            outs += [torch.zeros_like(q_bias, dtype=dtype), torch.zeros_like(k_bias, dtype=dtype)]
    for b in range(batch):
        for h in range(nheads):
            sl = lambda t: None if t is None else t[min(b, t.shape[0] - 1):min(b, t.shape[0] - 1) + 1, :,
                                                    min(h, t.shape[2] - 1):min(h, t.shape[2] - 1) + 1]
            msl = None
            if mask is not None:
                mb, mh = min(b, mask.shape[0] - 1), min(h, mask.shape[1] - 1)
                msl = mask[mb:mb + 1, mh:mh + 1]
            args = (sl(q), sl(k), sl(v), sl(q_bias), sl(k_bias), msl, causal,
                    softmax_scale or default_scale(d))
            if do is None:
                o[b:b + 1, :, h:h + 1] = flashbias_eager(*args, dtype=dtype)
            else:
                res = flashbias_eager_grads(*args, sl(do), dtype=dtype)
                o[b:b + 1, :, h:h + 1] = res[0]
                for dst, g in zip(outs, res[1:]):
                    if g is not None:
                        dst[b:b + 1, :, h:h + 1] = g
    if do is None:
        return o
    while len(outs) < 5:
        outs.append(None)
    return (o,) + tuple(outs)


def flashbias_concat_sdpa(q, k, v, q_bias, k_bias, softmax_scale, causal=False):
    """Library-backed identity used to pin the oracle: attention over the concatenated
    features [q*scale, q_bias] / [k, k_bias] with scale 1
    (flash_bias/attention_func.py:188-237, flash_bias/README.md:38-49)."""
    batch, _, nheads, _ = q.shape
    qb = q_bias.expand(batch, -1, nheads, -1)
    kb = k_bias.expand(batch, -1, nheads, -1)
    qc = torch.cat([q * softmax_scale, qb], dim=-1).transpose(1, 2)
    kc = torch.cat([k, kb], dim=-1).transpose(1, 2)
    out = torch.nn.functional.scaled_dot_product_attention(
        qc, kc, v.transpose(1, 2), attn_mask=None, dropout_p=0.0, is_causal=causal, scale=1.0)
    return out.transpose(1, 2)


def flashbias_backward_stored(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, o, lse, do,
                              round_dtype=None, dtype=torch.float32):
    """Backward from the *stored* forward results, the contract of the reference's
    ``_flash_attn_backward(do, q, k, v, o, ..., lse, ...)`` (flash_bias_triton.py:1197):

        delta = rowsum(o * do)                     (:398, o as stored in the input dtype)
        P     = exp(S - lse)                       (:670)
        dV    = round(P)^T dO                      (:696-697)
        dP    = dO V^T                             (:705)
        dS    = round(P * (dP - delta))            (:714)
        dK = scale dS^T Q, dK_b = dS^T Q_b         (:717-719)
        dQ = scale dS K,   dQ_b = dS K_b           (:728-732)

    ``round_dtype`` (fp16 / bf16) applies the two roundings the reference applies before its
    matmuls; ``None`` keeps everything in ``dtype`` and then this equals autograd through the
    eager path when (o, lse) are the eager ones.  Factor gradients are reduced over broadcast
    dims.  Returns (dq, dk, dv, dq_bias, dk_bias)."""
    scale = softmax_scale or default_scale(q.shape[-1])
    batch, _, nheads, _ = q.shape
    rnd = (lambda t: t.to(round_dtype).to(dtype)) if round_dtype is not None else (lambda t: t)
    qh, kh, vh, doh, oh = (t.to(dtype).permute(0, 2, 1, 3) for t in (q, k, v, do, o))
    bias = _dense_bias(q.to(dtype), None if q_bias is None else q_bias.to(dtype),
                       None if k_bias is None else k_bias.to(dtype), mask)
    s = logits(q.to(dtype), k.to(dtype), scale, bias, causal).permute(0, 2, 1, 3)
    p = torch.exp(s - lse.to(dtype)[..., None])
    delta = (oh * doh).sum(-1, keepdim=True)
    dv = rnd(p).transpose(-1, -2) @ doh
    ds = rnd(p * (doh @ vh.transpose(-1, -2) - delta))
    dq = scale * (ds @ kh)
    dk = scale * (ds.transpose(-1, -2) @ qh)
    out = [t.permute(0, 2, 1, 3) for t in (dq, dk, dv)]
    if q_bias is None:
        return tuple(out) + (None, None)
    qbh = q_bias.to(dtype).expand(batch, -1, nheads, -1).permute(0, 2, 1, 3)
    kbh = k_bias.to(dtype).expand(batch, -1, nheads, -1).permute(0, 2, 1, 3)
    for g, ref in ((ds @ kbh, q_bias), (ds.transpose(-1, -2) @ qbh, k_bias)):
        g = g.permute(0, 2, 1, 3)
        dims = [i for i in (0, 2) if ref.shape[i] == 1 and g.shape[i] != 1]
        out.append(g.sum(dim=dims, keepdim=True) if dims else g)
    return tuple(out)
