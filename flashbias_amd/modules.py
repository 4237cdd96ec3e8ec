"""Module-level drop-ins that call ``flash_bias_func`` the way the reference's application
code does: an ALiBi causal self-attention block
(1_Language_Model/attention_with_alibi_bias.py:18-64) and the attention core of a Swin-V2
window block with SVD bias factors (2_Vision_Transformer/swin_transformer_v2.py:155-207).
They exist for end-to-end layer timing and as usage examples; parameters are randomly
initialised (no checkpoints ship with either repository)."""
import torch
import torch.nn as nn

from . import factors
from .interface import flash_bias_func


class AttentionWithALiBiBias(nn.Module):
    """Causal multi-head self-attention with ALiBi as an exact rank-2 FlashBias.

    Same constructor arguments and forward contract as the reference module
    (x: (batch, seq, dim) -> (batch, seq, dim)).  Two deliberate differences, both switchable:
    the bias follows the standard ALiBi sign, ``-m_h (i - j)``, unless ``reference_sign=True``
    (the reference builds ``+m_h (i - j)``, attention_with_alibi_bias.py:49-52), and the compute
    dtype defaults to bf16 where the reference casts to fp16 (``dtype=torch.float16`` restores
    that).  The factors are the exact rank-4 form of ``factors.alibi_factors``: the bias the
    kernels see is exactly ``-m (i - j)`` with the slope rounded to the dtype, at every position."""

    def __init__(self, dim, heads, dim_head, dropout=0.0, dtype=torch.bfloat16, reference_sign=False):
        super().__init__()
        self.reference_sign = reference_sign
        inner = dim_head * heads
        self.heads, self.dim_head, self.scale, self.dtype = heads, dim_head, dim_head ** -0.5, dtype
        self.to_q = nn.Linear(dim, inner, bias=False)
        self.to_k = nn.Linear(dim, inner, bias=False)
        self.to_v = nn.Linear(dim, inner, bias=False)
        self.to_out = nn.Sequential(nn.Linear(inner, dim), nn.Dropout(dropout))

    def forward(self, x):
        b, n, _ = x.shape
        split = lambda t: t.view(b, n, self.heads, self.dim_head).to(self.dtype)
        q, k, v = split(self.to_q(x)), split(self.to_k(x)), split(self.to_v(x))
        q_bias, k_bias = factors.alibi_factors(n, n, self.heads, self.dtype, x.device, exact=True,
                                               reference_sign=self.reference_sign)
        o = flash_bias_func(q, k, v, q_bias, k_bias, None, True, self.scale)
        return self.to_out(o.reshape(b, n, -1).to(x.dtype))


class WindowAttentionCore(nn.Module):
    """The attention core of a Swin-V2 window block: cosine attention with a learned per-head
    logit scale, a relative-position bias given by rank-``rank`` SVD factors shared by all
    windows, and an optional shifted-window mask (num_windows, N, N) of 0 / -100 entries.

    x: (num_windows * B, N, C) -> (num_windows * B, N, C), as WindowAttention.forward
    (swin_transformer_v2.py:155-207); scale 1 is passed to the kernel because q is pre-scaled."""

    def __init__(self, dim, window, heads, rank=16, seed=0, dtype=torch.bfloat16):
        super().__init__()
        self.heads, self.dtype = heads, dtype
        self.qkv = nn.Linear(dim, dim * 3, bias=False)
        self.proj = nn.Linear(dim, dim)
        self.logit_scale = nn.Parameter(torch.log(10 * torch.ones(heads, 1, 1)))
        table = factors.swin_v2_bias_table(window, heads, seed)
        q_bias, k_bias, rel = factors.svd_factors(table, rank, dtype)
        self.register_buffer("q_bias_pos", q_bias)  # (1, N, H, rank)
        self.register_buffer("k_bias_pos", k_bias)
        self.register_buffer("bias_rel_error", rel)

    def forward(self, x, mask=None):
        b_, n, c = x.shape
        qkv = self.qkv(x).view(b_, n, 3, self.heads, c // self.heads)
        q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
        scale = torch.clamp(self.logit_scale, max=4.6052).exp().view(1, 1, self.heads, 1)
        q = (torch.nn.functional.normalize(q, dim=-1) * scale).to(self.dtype)
        k = torch.nn.functional.normalize(k, dim=-1).to(self.dtype)
        if mask is not None:
            nw = mask.shape[0]
            mask = mask.to(self.dtype)[None, :, None].expand(b_ // nw, nw, 1, n, n).reshape(b_, 1, n, n)
        o = flash_bias_func(q, k, v.to(self.dtype), self.q_bias_pos, self.k_bias_pos, mask, False, 1.0)
        return self.proj(o.reshape(b_, n, c).to(x.dtype))
