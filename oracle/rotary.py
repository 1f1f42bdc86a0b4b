"""Half-split rotary position embedding.  TEST ORACLE.

Follows ``llama/llama_mem.py:95-149``: ``inv_freq = base**(-2i/d)`` (``:98``),
tables ``cos/sin(t * inv_freq)`` duplicated over both halves (``:103-107``) and
cast to the model dtype (``:121-124``); application
``x*cos + rotate_half(x)*sin`` with ``rotate_half(x) = cat(-x2, x1)``
(``:127-149``).  In a bf16 model each of the three elementwise operations
rounds to bf16; the product of two bf16 numbers is exact in fp32, so doing the
arithmetic in fp32 and rounding after each operation reproduces that bit for
bit, which is what :func:`apply_rotary` does.

Pinned by ``tests/test_oracle_retrieval.py``: position 0 is the identity,
rotation preserves the norm of every (i, i+d/2) pair in fp64, relative-position
property <rot(q,m), rot(k,n)> depends on m-n only, and equality with torch's
own bf16 elementwise arithmetic.
"""
from __future__ import annotations

import torch


def rotary_tables(n_pos: int, dim: int, dtype=torch.float32, base: float = 10000.0):
    """(cos, sin), each (n_pos, dim), built in fp32 then cast to ``dtype``."""
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
    t = torch.arange(n_pos, dtype=torch.float32)
    ang = torch.outer(t, inv_freq)
    ang = torch.cat((ang, ang), dim=-1)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rotary(x, cos, sin, pos):
    """Rotate ``x (..., n, dim)`` at integer positions ``pos`` (broadcastable to
    ``x.shape[:-1]``), rounding to ``x.dtype`` after each elementwise op."""
    wide = torch.promote_types(x.dtype, torch.float32)
    c = cos[pos].to(wide)
    s = sin[pos].to(wide)
    xf = x.to(wide)
    a = (xf * c).to(x.dtype).to(wide)
    b = (rotate_half(xf) * s).to(x.dtype).to(wide)
    return (a + b).to(x.dtype)
