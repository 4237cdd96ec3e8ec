"""``flash_bias_func``: the reference's operator on MI355X.

Mirrors ``FlashBiasFunc`` of the reference (flash_bias/flash_bias_triton.py:1345-1405): same
name, same positional arguments and defaults, same return values, backed by the HIP kernels
of ``libflashbias_hip.so`` through its C ABI.  PyTorch only provides device memory and the
stream.  Differences from the reference, all on purpose:

* gradients of factors that broadcast over batch or heads are summed over those
  dimensions (the reference indexes the un-expanded tensors with expanded strides in its
  backward, flash_bias_triton.py:1227-1231, :1364);
* ``lse`` is (B, H, Lq), not rounded up to a multiple of 128 (:1145-1146);
* ``softmax_scale`` of ``None`` or 0 gives ``1/sqrt(d)`` as in the reference (:1110).
"""
import math

import torch

from . import _lib


def _tensor(x):
    """(B, L, H, c) tensor -> FbTensor with (batch, head, seq) element strides."""
    return _lib.FbTensor(x.data_ptr(), x.stride(0), x.stride(2), x.stride(1))


def _dtype_code(dtype):
    if dtype == torch.float16:
        return _lib.FB_F16
    if dtype == torch.bfloat16:
        return _lib.FB_BF16
    if dtype == torch.float32:
        return _lib.FB_F32
    raise TypeError(f"unsupported dtype {dtype}")


def _last_dim_contiguous(x):
    return x if x.stride(-1) == 1 else x.contiguous()


# A vector mask on a problem of at least this many (batch, head, query, key) pairs is folded into
# the factors (below that the extra tensor operations cost more than the kernels gain: measured
# at B2 H4 d32 r8, 2.09 against 2.96 ms fwd+bwd at L=16384, 0.38 against 0.32 ms at L=4096).
_FOLD_MIN_PAIRS = 1 << 29


_MAX_RANK = 128  # FB_MAX_RANK of include/flashbias.h


def _fold_keeps_rank_in_range(rank):
    """One more factor column, padded to the next multiple of 8, must still be a rank the library
    takes (rank 128 stays with the kernels' own vector-mask path)."""
    return rank is None or -(-(rank + 1) // 8) * 8 <= _MAX_RANK


def _fold_vector_mask(q, q_bias, k_bias, mask):
    """An additive (B|1, H|1, 1, Lk) mask is itself a rank-1 bias, 1_i * mask_j: appended to the
    factors as one more column it rides through the kernels' rank steps (which pad the rank to
    a multiple of 16 anyway) instead of being loaded by every query tile.  Exact for a mask of
    the input dtype: the products 1 * mask_j are summed in fp32 like every other bias term, and
    -inf entries stay -inf.  Returns (q_bias', k_bias'); the gradients of the added columns
    are dropped by the caller."""
    batch, seqlen_q, nheads, _ = q.shape
    seqlen_k = mask.shape[-1]
    col = mask.permute(0, 3, 1, 2)  # (B|1, Lk, H|1, 1)
    if q_bias is None:
        return q.new_ones((1, seqlen_q, 1, 1)), col
    kb, hb = max(k_bias.shape[0], col.shape[0]), max(k_bias.shape[2], col.shape[2])
    k_new = torch.cat([k_bias.expand(kb, seqlen_k, hb, -1), col.expand(kb, seqlen_k, hb, 1)], dim=-1)
    q_new = torch.cat([q_bias, q_bias.new_ones(q_bias.shape[:-1] + (1,))], dim=-1)
    return q_new, k_new


def _resize_rank(x, rank):
    """`x` (..., r) with its last dim zero-padded to `rank`: one launch of the library (fb_resize_rank, through the
    C++ extension's autograd function) for contiguous 16-bit GPU tensors, the tensor library's pad otherwise (a
    permuted view keeps its permuted layout there)."""
    ext = _extension()
    if ext is not None and x.is_cuda and x.is_contiguous() and x.element_size() == 2 and x.numel() > 0:
        return ext.resize_rank(x, rank)
    return torch.nn.functional.pad(x, (0, rank - x.shape[-1]))


def _prepare_factors(q, k, q_bias, k_bias, mask):
    """What the kernels get in place of (q_bias, k_bias, mask): a large vector mask folded into the
    factors, the rank zero-padded to a multiple of 8, the channel dimension contiguous.  Done once
    per forward; the backward reuses the result."""
    batch, seqlen_q, nheads, _ = q.shape
    seqlen_k = k.shape[1]
    if (mask is not None and mask.dim() == 4 and mask.shape[2] == 1 and mask.shape[3] == seqlen_k
            and mask.dtype == q.dtype and mask.is_cuda
            and batch * nheads * seqlen_q * seqlen_k >= _FOLD_MIN_PAIRS
            and _fold_keeps_rank_in_range(None if q_bias is None else q_bias.shape[-1])):
        q_bias, k_bias = _fold_vector_mask(q, q_bias, k_bias, mask)
        mask = None
    if q_bias is not None:
        assert k_bias is not None and q_bias.dtype == k_bias.dtype == q.dtype
        assert q_bias.is_cuda and k_bias.is_cuda
        rank = q_bias.shape[-1]
        assert k_bias.shape[-1] == rank
        if rank % 8:
            # zero columns change nothing in q_bias k_bias^T; a multiple of 8 makes the rows 16-byte
            # aligned, which selects the kernels with vector loads (ALiBi r=2, distance bias r=5).
            # Ranks below 8 are padded to 16, not 8: they are closed-form factors whose columns can be
            # large functions of position (ALiBi: m * i in the thousands, cancelling against m * j),
            # and a rank of 16 selects the kernels that keep the factors as they are and apply the
            # softmax scale to the fp32 accumulator.  The kernels that fold the scale into a 16-bit
            # operand (rank 8) carry every bias term with a relative error of 2^-17, which is 0.05 in
            # the logits at |term| = 7000.  A caller whose factors have small entries (a distance bias
            # over points in a unit box) opts in to rank 8 by padding them itself, once
            # (factors.pad_rank): the choice depends on nothing but the shapes it passes.
            target = 16 if rank < 8 else -(-rank // 8) * 8
            q_bias, k_bias = _resize_rank(q_bias, target), _resize_rank(k_bias, target)
        # (padding a permuted view keeps its permuted layout)
        q_bias, k_bias = _last_dim_contiguous(q_bias), _last_dim_contiguous(k_bias)
    if mask is not None:
        assert mask.dtype in (q.dtype, torch.float)
        assert mask.is_cuda
        assert mask.dim() == 4
        if mask.stride(-1) != 1:
            mask = mask.contiguous()
    return q_bias, k_bias, mask


def _prepare(q, k, v, factors, causal, softmax_scale):
    """Argument checks of _flash_attn_forward (flash_bias_triton.py:1100-1143) and the
    parameter block shared by forward and backward; `factors` = _prepare_factors(...).
    Returns (params, keepalive)."""
    q_bias, k_bias, mask = factors
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, _, _ = k.shape
    assert k.shape == (batch, seqlen_k, nheads, d)
    assert v.shape == (batch, seqlen_k, nheads, d)
    assert d <= 128, "FlashBias only supports head dimensions up to 128"
    assert q.dtype == k.dtype == v.dtype, "All tensors must have the same type"
    assert q.dtype in (torch.float16, torch.bfloat16), "Only support fp16 and bf16"
    assert q.is_cuda and k.is_cuda and v.is_cuda
    p = _lib.new_params()
    p.dtype = _dtype_code(q.dtype)
    p.B, p.H, p.Lq, p.Lk, p.d = batch, nheads, seqlen_q, seqlen_k, d
    p.causal = int(bool(causal))
    p.scale = softmax_scale or 1.0 / math.sqrt(d)
    p.q, p.k, p.v = _tensor(q), _tensor(k), _tensor(v)
    keep = []
    if q_bias is not None:
        rank = q_bias.shape[-1]
        # stride-0 broadcast over batch / heads (:1135-1136)
        qbe = q_bias.expand(batch, seqlen_q, nheads, rank)
        kbe = k_bias.expand(batch, seqlen_k, nheads, rank)
        p.r = rank
        p.q_bias, p.k_bias = _tensor(qbe), _tensor(kbe)
        keep += [qbe, kbe]
    if mask is not None:
        if mask.shape[2:] == (1, seqlen_k):
            p.mask_type = _lib.FB_MASK_VECTOR
        elif mask.shape[2:] == (seqlen_q, seqlen_k):
            p.mask_type = _lib.FB_MASK_MATRIX
        else:
            raise RuntimeError("Last 2 dimensions of mask must be (1, seqlen_k) or (seqlen_q, seqlen_k)")
        me = mask.expand(batch, nheads, seqlen_q, seqlen_k)
        p.mask = _lib.FbTensor(me.data_ptr(), me.stride(0), me.stride(1), me.stride(2))
        p.mask_dtype = _dtype_code(mask.dtype)
        keep.append(me)
    return p, keep


def _params(q, k, v, q_bias, k_bias, mask, causal, softmax_scale):
    """Parameter block for direct calls of the C ABI (tests, harness): (params, keepalive)."""
    factors = _prepare_factors(q, k, q_bias, k_bias, mask)
    p, keep = _prepare(q, k, v, factors, causal, softmax_scale)
    return p, keep + [t for t in factors if t is not None]


def _stream(device=None):
    """Raw handle of torch's current stream on `device` (default: the current device)."""
    index = torch.cuda.current_device() if device is None or device.index is None else device.index
    return torch._C._cuda_getCurrentRawStream(index)


def _launch(fn, p, device):
    """One C-ABI call on torch's current stream of `device`, with that device current."""
    if device.index is None or device.index == torch.cuda.current_device():
        _lib.check_status(fn(p, _stream(device)))
    else:
        with torch.cuda.device(device):
            _lib.check_status(fn(p, _stream(device)))


def _flash_bias_forward(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, factors=None):
    """(o, lse, softmax_scale), as _flash_attn_forward of the reference (flash_bias_triton.py:1100-1194)."""
    return _forward_with_block(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, factors)[:3]


def _forward_with_block(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, factors=None):
    """Returns (o, lse, softmax_scale, block): block = the parameter block of the call and the
    tensors its pointers refer to, which a backward over the same tensors may reuse."""
    lib = _lib.load()
    if factors is None:
        factors = _prepare_factors(q, k, q_bias, k_bias, mask)
    p, keep = _prepare(q, k, v, factors, causal, softmax_scale)
    o = torch.empty_like(q)
    lse = torch.empty((p.B, p.H, p.Lq), device=q.device, dtype=torch.float32)
    p.o, p.lse = _tensor(o), lse.data_ptr()
    _launch(lib.fb_fwd, p, q.device)
    return o, lse, p.scale, (p, keep)


def _flash_bias_backward(do, q, k, v, o, q_bias, k_bias, lse, mask, causal, softmax_scale, factors=None, block=None,
                         factor_grads=True):
    """factor_grads=False: neither factor asks for its gradient (constant factors: ALiBi slopes, tables loaded from
    a file, coordinates); the library is then given no dq_bias / dk_bias and its kernels skip them."""
    lib = _lib.load()
    do = _last_dim_contiguous(do)
    if block is not None and (block[0].q.ptr, block[0].k.ptr, block[0].v.ptr) == (q.data_ptr(), k.data_ptr(), v.data_ptr()):
        p, keep = block  # the forward's block: same tensors (the factors and the mask are kept alive by it)
    else:
        if factors is None:
            factors = _prepare_factors(q, k, q_bias, k_bias, mask)
        p, keep = _prepare(q, k, v, factors, causal, softmax_scale)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    p.o, p.lse, p.dout = _tensor(o), lse.data_ptr(), _tensor(do)
    p.dq, p.dk, p.dv = _tensor(dq), _tensor(dk), _tensor(dv)
    dqb_full = dkb_full = None
    p.dq_bias = p.dk_bias = _lib.FbTensor()  # (the block may be the forward's, or an earlier backward's)
    # factors shared by a large batch of short sequences: a workgroup walks `group` batch entries (it then loads the
    # factor operand it keeps once), sums their factor gradients itself, and the full-shape tensors shrink by that factor
    # (only for factors that are saved with a batch of one: a factor expanded over the batch by its caller also has
    # batch stride 0, but autograd wants its gradient in the expanded shape)
    shared = q_bias is not None and q_bias.shape[0] == 1 and k_bias.shape[0] == 1 and p.B > 1
    group = p.bias_grad_group = (lib.fb_suggest_bias_grad_group(p) if shared else 1) if p.r else 0
    if p.r and factor_grads and q_bias is not None:
        rows = -(-p.B // group)
        dqb_full = torch.empty((rows, p.Lq, p.H, p.r), device=q.device, dtype=q.dtype)
        dkb_full = torch.empty((rows, p.Lk, p.H, p.r), device=q.device, dtype=q.dtype)
        p.dq_bias, p.dk_bias = _tensor(dqb_full), _tensor(dkb_full)
    # scratch of the backward: -delta and lse * log2(e), sized by the library
    delta = torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=lse.device, dtype=torch.float32)
    p.delta = delta.data_ptr()
    _launch(lib.fb_bwd, p, q.device)
    del keep
    dq_bias = dk_bias = None
    if dqb_full is not None:
        dq_bias = _reduce_like(dqb_full, q_bias)
        dk_bias = _reduce_like(dkb_full, k_bias)
    return dq, dk, dv, dq_bias, dk_bias


def _reduce_like(full, ref):
    """The gradient of ``ref`` from the full (B, L, H, r') gradient the kernels wrote: summed over
    the dims in which ``ref`` was broadcast (in fp32; over the batch by the library's own
    streaming kernel, bit-reproducibly), without the zero columns the kernels may have run with."""
    rank = ref.shape[-1]
    over_batch = ref.shape[0] == 1 and full.shape[0] != 1
    over_heads = ref.shape[2] == 1 and full.shape[2] != 1
    n = full[0].numel()
    if over_batch and full.is_contiguous() and n % 8 == 0:
        out = torch.empty((1,) + full.shape[1:], device=full.device, dtype=torch.float32 if over_heads else full.dtype)
        batch = full.shape[0]

        def call(_, stream):
            return _lib.load().fb_sum_over_batch(full.data_ptr(), out.data_ptr(), _dtype_code(full.dtype),
                                                 _dtype_code(out.dtype), batch, n, n, stream)
        _launch(call, None, full.device)
        full, over_batch = out, False
    dims = [i for i, over in ((0, over_batch), (2, over_heads)) if over]
    if dims:
        full = full.sum(dim=dims, keepdim=True, dtype=torch.float32)
    full = full[..., :rank].to(ref.dtype)
    return full if full.is_contiguous() else full.contiguous()


class FlashBiasFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, q_bias=None, k_bias=None, mask=None, causal=False, softmax_scale=None):
        """
        q: (batch_size, seqlen_q, nheads, headdim)
        k, v: (batch_size, seqlen_k, nheads, headdim)
        q_bias: (batch_size | 1, seqlen_q, nheads | 1, rankdim)
        k_bias: (batch_size | 1, seqlen_k, nheads | 1, rankdim)
        mask: optional additive mask broadcastable to (batch, nheads, seqlen_q, seqlen_k) whose
            last two dims are (1, seqlen_k) or (seqlen_q, seqlen_k); receives no gradient
        softmax_scale: multiplies q k^T only; defaults to 1 / sqrt(headdim)
        """
        if q_bias is not None:
            q, k, v, q_bias, k_bias = [_last_dim_contiguous(x) for x in (q, k, v, q_bias, k_bias)]
        else:
            q, k, v = [_last_dim_contiguous(x) for x in (q, k, v)]
        # (what the kernels consume in place of q_bias, k_bias, mask: kept for the backward)
        ctx.kernel_factors = _prepare_factors(q, k, q_bias, k_bias, mask)
        o, lse, ctx.softmax_scale, ctx.block = _forward_with_block(q, k, v, q_bias, k_bias, mask, causal,
                                                                   softmax_scale, ctx.kernel_factors)
        ctx.save_for_backward(q, k, v, o, q_bias, k_bias, lse, mask)
        ctx.causal = causal
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, q_bias, k_bias, lse, mask = ctx.saved_tensors
        assert not ctx.needs_input_grad[5], "FlashBias does not support mask gradient yet"
        dq, dk, dv, dq_bias, dk_bias = _flash_bias_backward(
            do, q, k, v, o, q_bias, k_bias, lse, mask, ctx.causal, ctx.softmax_scale, ctx.kernel_factors, ctx.block,
            factor_grads=ctx.needs_input_grad[3] or ctx.needs_input_grad[4])
        return dq, dk, dv, dq_bias, dk_bias, None, None, None


_ext = False  # the C++ autograd function: False = not looked for yet, None = not built


def _extension():
    """flashbias_amd/_fb_torch.so (csrc/fb_torch.cpp): the autograd function of the operator in C++,
    over the same C ABI.  None when it has not been built; the Python FlashBiasFunc then serves."""
    global _ext
    if _ext is False:
        try:
            from . import _fb_torch
            lib = _lib.load()
            # (a module built against another version of the parameter block would fail every call with
            # FB_ERR_ABI: the Python function serves instead)
            import ctypes
            ok = getattr(_fb_torch, "abi", lambda: None)() == (lib.fb_version(), ctypes.sizeof(_lib.FbParams))
            _ext = _fb_torch if ok else None
        except ImportError:
            _ext = None
    return _ext


def flash_bias_func(q, k, v, q_bias=None, k_bias=None, mask=None, causal=False, softmax_scale=None):
    """``FlashBiasFunc.apply`` of the reference (flash_bias/flash_bias_triton.py:1405): same positional
    arguments and defaults.  Runs the autograd function in C++ when that extension is built (the
    same checks, allocations and launches without the interpreter: a forward + backward costs the
    host about half as much, which is what sequence lengths up to a few thousand are bound by),
    else the Python FlashBiasFunc above.  The rare preparations (a large vector mask folded into the
    factors, a rank padded to a multiple of 8) are ordinary differentiable tensor operations here,
    so their gradients come from autograd."""
    ext = _extension()
    if ext is None:
        return FlashBiasFunc.apply(q, k, v, q_bias, k_bias, mask, causal, softmax_scale)
    # the launcher's assertions (:1100-1143), as assertions
    assert q.dim() == 4 and k.dim() == 4 and k.shape[0] == q.shape[0] and k.shape[2:] == q.shape[2:] and v.shape == k.shape
    assert q.shape[-1] <= 128, "FlashBias only supports head dimensions up to 128"
    assert q.dtype == k.dtype == v.dtype, "All tensors must have the same type"
    assert q.dtype in (torch.float16, torch.bfloat16), "Only support fp16 and bf16"
    assert q.is_cuda and k.is_cuda and v.is_cuda
    if (q_bias is not None and q_bias.shape[-1] % 8) or (mask is not None and mask.dim() == 4 and mask.shape[2] == 1):
        if q_bias is not None:
            q, k, v, q_bias, k_bias = [_last_dim_contiguous(x) for x in (q, k, v, q_bias, k_bias)]
        q_bias, k_bias, mask = _prepare_factors(q, k, q_bias, k_bias, mask)
    return ext.flash_bias(q, k, v, q_bias, k_bias, mask, bool(causal), float(softmax_scale or 0.0))
