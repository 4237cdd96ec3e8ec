"""Builders of the low-rank bias factors that feed ``flash_bias_func``.

Three ways to obtain ``q_bias`` / ``k_bias`` with ``q_bias @ k_bias^T == bias``:
exact closed forms (ALiBi, squared spatial distance), and a truncated SVD of a learned bias
table (Swin-V2 relative position bias).  All factors come back in the operator's layout
(B | 1, L, H | 1, r).
"""
import math

import torch


def alibi_slopes(nheads):
    """Per-head slope m_h = 2^(-8 (h+1) / H) (1_Language_Model/attention_with_alibi_bias.py:8-15)."""
    h = torch.arange(1, nheads + 1, dtype=torch.float64)
    return torch.pow(2.0, -8.0 * h / nheads).float()


def alibi_factors(seqlen_q, seqlen_k, nheads, dtype=torch.float32, device=None, exact=False, reference_sign=False):
    """Factors of the ALiBi bias  -m_h (i - j)  (``reference_sign``: +m_h (i - j), what the
    reference's demo module builds, 1_Language_Model/attention_with_alibi_bias.py:49-52).

    ``exact=False``: the rank-2 closed form  q_bias[i] = [-m_h i, 1],  k_bias[j] = [1, m_h j],
    computed in fp32 and cast once.  In a 16-bit dtype the columns m_h i are rounded to 8 (bf16)
    or 11 (fp16) significant bits, so the product of the cast factors deviates from the closed
    form by up to several units at positions in the thousands.

    ``exact=True``: rank-4 factors whose every column is exactly representable in bf16 and fp16
    for positions below 65536, with i = 256 a_i + b_i and the slope rounded to the dtype once:

        q_bias[i] = [a_i, b_i, 256 m, m],   k_bias[j] = [-256 m, -m, a_j, b_j]

    The four products and their fp32 sum are exact, so the kernels see exactly  -m (i - j)  with
    m = the 16-bit slope: monotone in the distance, relative deviation from the true slope at most
    half an ulp of the dtype.  This is what the module drop-in uses."""
    m = alibi_slopes(nheads).to(device)
    if not exact:
        i = torch.arange(seqlen_q, dtype=torch.float32, device=device)
        j = torch.arange(seqlen_k, dtype=torch.float32, device=device)
        sgn = 1.0 if reference_sign else -1.0
        q_bias = torch.stack([sgn * (i[:, None] * m[None, :]), torch.ones(seqlen_q, nheads, device=device)], dim=-1)
        k_bias = torch.stack([torch.ones(seqlen_k, nheads, device=device), -sgn * (j[:, None] * m[None, :])], dim=-1)
        return q_bias[None].to(dtype), k_bias[None].to(dtype)
    assert max(seqlen_q, seqlen_k) <= 65536, "positions are split into two 8-bit digits"
    m = m.to(dtype).float()  # the slope the kernels will see
    sgn = -1.0 if reference_sign else 1.0

    def digits(n):
        pos = torch.arange(n, device=device)
        return (pos // 256).float()[:, None].expand(n, nheads), (pos % 256).float()[:, None].expand(n, nheads)

    aq, bq = digits(seqlen_q)
    ak, bk = digits(seqlen_k)
    mq, mk = m[None, :].expand(seqlen_q, nheads), m[None, :].expand(seqlen_k, nheads)
    q_bias = torch.stack([aq, bq, 256.0 * mq, mq], dim=-1)
    k_bias = torch.stack([-sgn * 256.0 * mk, -sgn * mk, sgn * ak, sgn * bk], dim=-1)
    return q_bias[None].to(dtype), k_bias[None].to(dtype)


def distance_factors(x_q, x_k, alpha, dtype=torch.float32):
    """Exact rank-(D+2) factors of  -alpha |x_i - x_j|^2  for points x (B, N, D):
    q_bias = [-alpha |x_i|^2, -alpha, 2 alpha x_i],  k_bias = [1, |x_j|^2, x_j]
    (the spatial-distance decomposition of the paper, pic/exact_decompose_pde.png).
    Shapes (B, N, 1, D + 2): shared by all heads."""
    nq = (x_q * x_q).sum(-1, keepdim=True)
    nk = (x_k * x_k).sum(-1, keepdim=True)
    q_bias = torch.cat([-alpha * nq, torch.full_like(nq, -alpha), 2.0 * alpha * x_q], dim=-1)
    k_bias = torch.cat([torch.ones_like(nk), nk, x_k], dim=-1)
    return q_bias[:, :, None, :].to(dtype), k_bias[:, :, None, :].to(dtype)


def pad_rank(q_bias, k_bias, multiple=8):
    """The factors with zero columns appended up to the next multiple of ``multiple`` (the product
    q_bias k_bias^T is unchanged).  ``flash_bias_func`` pads ranks that are not multiples of 8 by
    itself on every call, and ranks below 8 to 16, because the rank-8 kernels fold the softmax scale
    into a 16-bit operand and carry each bias term q_bias[i, c] k_bias[j, c] with a relative error of
    2^-17: harmless for terms up to a few hundred (0.002 in the logits at 256), not for ALiBi's
    closed form (terms in the thousands).  Constant factors with small terms (the distance bias over
    points in a unit box: at most 2 alpha) are padded to 8 here, once, by the caller who knows them;
    the operator then runs the rank-8 kernels and pads nothing per call."""
    rank = q_bias.shape[-1]
    assert k_bias.shape[-1] == rank
    pad = (-rank) % multiple
    if pad == 0:
        return q_bias, k_bias
    return torch.nn.functional.pad(q_bias, (0, pad)), torch.nn.functional.pad(k_bias, (0, pad))


def svd_factors(bias, rank, dtype=torch.float32):
    """Best rank-``rank`` factors (Eckart-Young) of a per-head bias table (H, Lq, Lk).
    Returns q_bias (1, Lq, H, rank), k_bias (1, Lk, H, rank) and the relative Frobenius error
    of the reconstruction, ``|bias - q_bias k_bias^T|_F / |bias|_F``, per head."""
    u, s, vh = torch.linalg.svd(bias.double(), full_matrices=False)
    root = s[:, :rank].sqrt()
    q_bias = u[:, :, :rank] * root[:, None, :]
    k_bias = vh[:, :rank, :].transpose(1, 2) * root[:, None, :]
    tail = (s[:, rank:] ** 2).sum(-1).sqrt()
    rel = tail / (s ** 2).sum(-1).sqrt()
    return (q_bias.permute(1, 0, 2)[None].to(dtype).contiguous(),
            k_bias.permute(1, 0, 2)[None].to(dtype).contiguous(), rel.float())


def swin_v2_bias_table(window, nheads, seed=0, hidden=512):
    """A Swin-V2 style continuous relative position bias (H, N, N) for a ``window`` x ``window``
    token grid with a randomly initialised 2 -> hidden -> H ReLU MLP on log-spaced relative
    coordinates, squashed to (0, 16) (2_Vision_Transformer/swin_transformer_v2.py:98-131)."""
    g = torch.Generator().manual_seed(seed)
    w1 = (torch.rand(hidden, 2, generator=g) * 2 - 1) / math.sqrt(2.0)
    b1 = (torch.rand(hidden, generator=g) * 2 - 1) / math.sqrt(2.0)
    w2 = (torch.rand(nheads, hidden, generator=g) * 2 - 1) / math.sqrt(hidden)
    rel = torch.arange(-(window - 1), window, dtype=torch.float32) / max(window - 1, 1) * 8.0
    rel = torch.sign(rel) * torch.log2(rel.abs() + 1.0) / math.log2(8.0)
    table = torch.stack(torch.meshgrid(rel, rel, indexing="ij"), dim=-1)  # (2W-1, 2W-1, 2)
    table = torch.relu(table @ w1.t() + b1) @ w2.t()  # (2W-1, 2W-1, H)
    pos = torch.stack(torch.meshgrid(torch.arange(window), torch.arange(window), indexing="ij")).flatten(1)
    diff = pos[:, :, None] - pos[:, None, :] + (window - 1)  # (2, N, N), each in [0, 2W-2]
    bias = table[diff[0], diff[1]]  # (N, N, H)
    return 16.0 * torch.sigmoid(bias.permute(2, 0, 1)).contiguous()
