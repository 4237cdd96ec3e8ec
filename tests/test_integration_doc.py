"""The ctypes binding printed in the integration notes at the repository root is executed as printed: its parameter block must be the
one the library expects (size check of every entry point, FB_ERR_ABI otherwise) and its field
offsets those of flashbias_amd/_lib.py."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NOTES = "INTEGRATION.md"


def _documented_binding():
    text = open(os.path.join(ROOT, NOTES)).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    block = next(b for b in blocks if "class FbParams" in b)
    ns = {}
    cwd = os.getcwd()
    os.chdir(ROOT)  # (the snippet loads the library by its path from the repository root)
    try:
        exec(compile(block, NOTES, "exec"), ns)
    finally:
        os.chdir(cwd)
    return ns


def test_documented_parameter_block_is_accepted():
    from flashbias_amd import _lib
    ns = _documented_binding()
    lib, FbParams, FbTensor = ns["lib"], ns["FbParams"], ns["FbTensor"]
    assert ctypes.sizeof(FbParams) == ctypes.sizeof(_lib.FbParams)
    for name, _ in _lib.FbParams._fields_:
        assert getattr(FbParams, name).offset == getattr(_lib.FbParams, name).offset, name
    p = FbParams()
    p.size = ctypes.sizeof(FbParams)
    p.dtype, p.B, p.H, p.Lq, p.Lk, p.d, p.r, p.scale = 1, 2, 4, 128, 128, 32, 8, 0.25
    fake = 1 << 20  # fb_check reads no memory: any aligned non-null address will do
    dense = lambda c, L: FbTensor(fake, L * p.H * c, c, p.H * c)
    p.q, p.k, p.v, p.o, p.dout = (dense(32, 128) for _ in range(5))
    p.dq, p.dk, p.dv = (dense(32, 128) for _ in range(3))
    p.q_bias, p.k_bias, p.dq_bias, p.dk_bias = (dense(8, 128) for _ in range(4))
    p.lse = p.delta = fake
    lib.fb_check.argtypes = [ctypes.POINTER(FbParams), ctypes.c_int]
    for which in (0, 1):
        assert lib.fb_check(ctypes.byref(p), which) == 0, lib.fb_last_error()
    assert lib.fb_bwd_workspace_bytes(ctypes.byref(p)) == 24 * p.B * p.H * p.Lq
    p.size -= 8  # the block as it was documented before bias_grad_group existed
    assert lib.fb_check(ctypes.byref(p), 0) == -7


def test_every_export_is_listed_in_the_document():
    from flashbias_amd import _lib
    text = open(os.path.join(ROOT, NOTES)).read()
    for name in _lib.EXPORTS:
        assert name in text, name
