"""Rotary position embedding on the HIP kernel, with the reference's call surface.

``apply_rotary_pos_emb(q, k, cos, sin, position_ids)`` mirrors ``llama/llama_mem.py:134-149``:
``cos``/``sin`` are the ``(1, 1, n_pos, hd)`` (or ``(n_pos, hd)``) model-dtype tables of
``LlamaRotaryEmbedding`` (``:95-124``), ``position_ids`` is ``(bs, seq)`` or ``(1, seq)`` int64, ``q`` may
be ``None`` (``:143-144``).  One launch for q and k together (one per tensor when their shapes differ) replaces the reference's gather of the table rows,
two products, ``rotate_half``'s concatenation and the sum, and gives the same bits: every one of the
three elementwise operations rounds to the model dtype, as torch's 16-bit arithmetic does.
"""
from __future__ import annotations

import torch

from . import _lib
from .retrieval import _tables


def _rotate(x, cos, sin, position_ids, out=None):
    B, H, L, D = x.shape
    assert position_ids.dim() == 2 and position_ids.shape[1] == L and position_ids.shape[0] in (1, B)
    assert position_ids.dtype == torch.int64 and position_ids.device == x.device
    x = _lib.kernel_ready(x)
    position_ids = position_ids.contiguous()
    if out is None:
        out = torch.empty_like(x)
    with _lib.on_device(x.device):
        rc = _lib.lib().lmk_apply_rotary(_lib.tensor4(x), _lib.tensor4(out), cos.data_ptr(), sin.data_ptr(),
                                         cos.stride(0), cos.shape[0], position_ids.data_ptr(),
                                         L if position_ids.shape[0] == B and B > 1 else 0, B, H, L, D,
                                         _lib.DTYPE_CODES[x.dtype], _lib.current_stream(x.device))
    _lib.check(rc)
    return out


def _rotate_qk(q, k, cos, sin, position_ids):
    B, H, L, D = q.shape
    q, k = _lib.kernel_ready(q), _lib.kernel_ready(k)
    position_ids = position_ids.contiguous()
    q_embed, k_embed = torch.empty_like(q), torch.empty_like(k)
    with _lib.on_device(q.device):
        rc = _lib.lib().lmk_apply_rotary_qk(_lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(q_embed),
                                            _lib.tensor4(k_embed), cos.data_ptr(), sin.data_ptr(), cos.stride(0),
                                            cos.shape[0], position_ids.data_ptr(),
                                            L if position_ids.shape[0] == B and B > 1 else 0, B, H, L, D,
                                            _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
    _lib.check(rc)
    return q_embed, k_embed


def _transposed_sin(sin):
    """The sine table of the transposed rotation.  ``y = x*cos + rotate_half(x)*sin`` is linear in x, and its
    transpose is the same expression with ``sin`` replaced by ``-cat(sin[..., hd/2:], sin[..., :hd/2])``
    (for LLaMA's tables, whose halves are equal, simply ``-sin``: the rotation by the opposite angle).  The
    gradient therefore goes through the same kernel, with the same three roundings torch's autograd applies
    to the reference expression in a 16-bit model."""
    h = sin.shape[-1] // 2
    return (-torch.cat((sin[..., h:], sin[..., :h]), dim=-1)).contiguous()


class _Rotary(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cos, sin, position_ids):
        ctx.save_for_backward(cos, sin, position_ids)
        return _rotate(x, cos, sin, position_ids)

    @staticmethod
    def backward(ctx, dy):
        cos, sin, position_ids = ctx.saved_tensors
        return _rotate(dy, cos, _transposed_sin(sin), position_ids), None, None, None


class _RotaryQK(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, cos, sin, position_ids):
        ctx.save_for_backward(cos, sin, position_ids)
        return _rotate_qk(q, k, cos, sin, position_ids)

    @staticmethod
    def backward(ctx, dq, dk):
        cos, sin, position_ids = ctx.saved_tensors
        gq, gk = _rotate_qk(dq, dk, cos, _transposed_sin(sin), position_ids)
        return gq, gk, None, None, None


def apply_rotary_pos_emb(q, k, cos, sin, position_ids):
    """``(q_embed, k_embed)`` as ``llama_mem.py:134-149`` returns them; ``q_embed`` is ``None`` when
    ``q`` is.  q, k: ``(B, nh, L, hd)`` bf16/fp16 on the GPU with hd 64 or 128.  Differentiable in q and k,
    as the reference's expression is (the tables and positions get no gradient)."""
    assert k.is_cuda and k.dtype in _lib.DTYPE_CODES
    cos, sin = _tables(cos, sin, k.dtype)
    if q is None:
        return None, _Rotary.apply(k, cos, sin, position_ids)
    if q.shape != k.shape:                      # e.g. fewer key heads: one launch per tensor
        return _Rotary.apply(q, cos, sin, position_ids), _Rotary.apply(k, cos, sin, position_ids)
    B, H, L, D = q.shape
    assert q.dtype == k.dtype and q.device == k.device
    assert position_ids.dim() == 2 and position_ids.shape[1] == L and position_ids.shape[0] in (1, B)
    assert position_ids.dtype == torch.int64 and position_ids.device == q.device
    return _RotaryQK.apply(q, k, cos, sin, position_ids)
