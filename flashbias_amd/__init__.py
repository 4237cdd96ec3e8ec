"""FlashBias attention for AMD Instinct MI355X (gfx950).

``flash_bias_func(q, k, v, q_bias, k_bias, mask, causal, softmax_scale)`` computes
``softmax(scale * q k^T + q_bias k_bias^T + mask) v`` with forward and backward HIP kernels;
it is a drop-in for the operator of the same name in the reference
(flash_bias/flash_bias_triton.py:1405).
"""
from .interface import FlashBiasFunc, flash_bias_func  # noqa: F401

__all__ = ["FlashBiasFunc", "flash_bias_func"]
