"""``fused_landmark_attention`` with the reference's call surface
(``llama/ltriton/flash_landmark_attention.py:308-403``), backed by the HIP kernels.

Differences a caller can observe, all of them relaxations:
* ``is_mem=None`` is accepted and means "landmarks at fixed stride" (the reference's
  README promises this, its code dereferences ``is_mem.shape``, ``:393``);
* q/k/v views with arbitrary batch/head/row strides are read in place when their last
  dim is dense and 16-byte aligned (the reference always copies, ``:312-314``).
"""
from __future__ import annotations

import math

import torch

from . import _lib

SUPPORTED_BLOCKS = (32, 64, 128)
SUPPORTED_HEAD_DIMS = (64, 128)


def _launch_fwd(q, k, v, n_prefix, sm_scale, block):
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    o = torch.empty_like(q)        # keeps q's memory layout: a (B,L,H,D)-backed q gives an output whose
    #                                transpose(1, 2).reshape(B, L, H*D) for o_proj (llama_mem.py:484-486) is a view
    L = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
    M = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
    rc = _lib.lib().lmk_attn_fwd(_lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o),
                                 L.data_ptr(), M.data_ptr(), B, H, Lq, Lk, D, float(sm_scale), int(block),
                                 int(n_prefix), _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
    _lib.check(rc)
    return o, L, M


def _launch_bwd(q, k, v, o, do, L, M, n_prefix, sm_scale, block):
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    lib = _lib.lib()
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)     # each in its input's layout
    nbytes = lib.lmk_attn_bwd_workspace_bytes(B, H, Lq, Lk, int(block))
    ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
    rc = lib.lmk_attn_bwd(_lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o), _lib.tensor4(do),
                          L.data_ptr(), M.data_ptr(), _lib.tensor4(dq), _lib.tensor4(dk), _lib.tensor4(dv),
                          ws.data_ptr(), nbytes, B, H, Lq, Lk, D, float(sm_scale), int(block), int(n_prefix),
                          _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
    _lib.check(rc)
    return dq, dk, dv


class FusedLandmarkAttention(torch.autograd.Function):
    """Same ``forward(ctx, q, k, v, n_prefix_q, sm_scale, block_size)`` /
    ``backward(ctx, do) -> (dq, dk, dv, None, None, None)`` contract as the reference
    (``flash_landmark_attention.py:308-389``)."""

    @staticmethod
    def forward(ctx, q, k, v, n_prefix_q, sm_scale, block_size):
        batch, nheads, seqlen_q, d = q.shape
        seqlen_k = k.shape[2]
        assert k.shape == (batch, nheads, seqlen_k, d)
        assert v.shape == (batch, nheads, seqlen_k, d)
        assert d <= 128, "FlashAttention only support head dimensions up to 128"
        assert q.dtype == k.dtype == v.dtype, "All tensors must have the same type"
        assert q.is_cuda and k.is_cuda and v.is_cuda
        assert q.dtype in _lib.DTYPE_CODES, "HIP kernels are built for bf16 and fp16"
        assert d in SUPPORTED_HEAD_DIMS, f"HIP kernels are built for head dims {SUPPORTED_HEAD_DIMS}"
        assert block_size in SUPPORTED_BLOCKS, f"HIP kernels are built for block sizes {SUPPORTED_BLOCKS}"
        q, k, v = _lib.kernel_ready(q), _lib.kernel_ready(k), _lib.kernel_ready(v)
        with _lib.on_device(q.device):
            o, L, m = _launch_fwd(q, k, v, n_prefix_q, sm_scale, block_size)
        ctx.save_for_backward(q, k, v, o, L, m)
        ctx.sm_scale = sm_scale
        ctx.N_PREFIX_Q = n_prefix_q
        ctx.BLOCK = block_size
        return o

    @staticmethod
    def backward(ctx, do):
        BLOCK = ctx.BLOCK
        q, k, v, o, l, m = ctx.saved_tensors
        assert q.shape[2] % BLOCK == 0, "Backward supported only for full blocks"
        assert k.shape[2] % BLOCK == 0, "Backward supported only for full blocks"
        do = _lib.kernel_ready(do)
        with _lib.on_device(q.device):
            dq, dk, dv = _launch_bwd(q, k, v, o, do, l, m, ctx.N_PREFIX_Q, ctx.sm_scale, BLOCK)
        return dq, dk, dv, None, None, None


# Masks that have already passed the check of ``flash_landmark_attention.py:393-394``, keyed by what
# identifies a tensor's content without reading it: storage address, in-place version counter, layout.
# A layer stack hands the same mask to every layer and every step, so the device->host sync of the
# comparison is paid once per mask instead of once per call.
_VALIDATED_MASKS: dict = {}
_VALIDATED_MASKS_MAX = 64


def _check_is_mem(is_mem, block_size):
    key = (is_mem.device, is_mem.data_ptr(), is_mem._version, tuple(is_mem.shape), tuple(is_mem.stride()),
           is_mem.dtype, int(block_size))
    if key in _VALIDATED_MASKS:
        return
    expected_is_mem = torch.arange(0, is_mem.shape[-1], device=is_mem.device) % block_size == (block_size - 1)
    assert (is_mem == expected_is_mem).all()
    if len(_VALIDATED_MASKS) >= _VALIDATED_MASKS_MAX:
        _VALIDATED_MASKS.clear()
    # the entry keeps the tensor alive, so its address cannot be handed to another mask meanwhile
    _VALIDATED_MASKS[key] = is_mem


def fused_landmark_attention(q, k, v, is_mem, sm_scale=None, block_size=64):
    """Landmark grouped-softmax causal attention, landmarks at every ``block_size``-th key.

    q: (B, H, Lq, D); k, v: (B, H, Lk, D) with ``Lk - Lq`` a whole number of blocks of
    history.  ``is_mem`` (bool, last dim Lk) must mark exactly the positions
    ``j % block_size == block_size - 1`` (checked as in the reference, ``:393-394``; the check
    costs one device->host sync, paid once per distinct mask tensor state, not per call); pass
    ``None`` to skip the check.
    """
    if is_mem is not None:
        _check_is_mem(is_mem, block_size)

    n_history_kv = k.shape[-2] - q.shape[-2]
    assert n_history_kv % block_size == 0
    n_history_blocks = n_history_kv // block_size

    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.size(-1))

    return FusedLandmarkAttention.apply(q, k, v, n_history_blocks, sm_scale, block_size)
