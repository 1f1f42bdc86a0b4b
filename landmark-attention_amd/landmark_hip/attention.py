"""``fused_landmark_attention`` with the reference's call surface
(``llama/ltriton/flash_landmark_attention.py:308-403``), backed by the HIP kernels.

Block sizes other than 32, 64 and 128 (the training models use ``mem_freq + 1 = 51``) run on the
64- or 128-slot kernels, which read and write the tensors as they are: a block's normal tokens occupy its
first slots, its landmark the last one, and the kernels translate slots to token rows as they load and store
and mask the slots in between (``lmk_attn_fwd_blocks`` / ``lmk_attn_bwd_blocks``).  Nothing is repacked or
copied.  Blocks wider than 128 tokens are rejected.

Head dims 16 and 32 are zero-padded to 64 by ``fused_landmark_attention``.

Differences a caller can observe, all of them relaxations:
* ``is_mem=None`` is accepted and means "landmarks at fixed stride" (the reference's
  README promises this, its code dereferences ``is_mem.shape``, ``:393``);
* q/k/v views with arbitrary batch/head/row strides are read in place when their last
  dim is dense and 16-byte aligned (the reference always copies, ``:312-314``).
"""
from __future__ import annotations

import math
import os

import torch

from . import _lib

SUPPORTED_BLOCKS = (32, 64, 128)      # block sizes the kernels run without repacking
MAX_BLOCK = 128
SUPPORTED_HEAD_DIMS = (64, 128)
# Two backward paths exist for block 32.  With a workspace of lmk_attn_bwd_handover_workspace_bytes() the dQ kernel
# leaves dS behind for the dK/dV kernel (2 bytes per visible (query, key) pair), which then forms neither dP nor dS
# again.  That can only pay while the tiles stay in the GPU's 256 MB last-level cache between the two kernels (it
# loses once they have to travel through HBM: 7 % slower at B2 H32 L2048, 307 MB), so workspaces above this many
# bytes are not allocated and the recomputing kernels run in 4 * (2 + 3 * Lk / block) bytes per query row ...
HANDOVER_MAX_BYTES = int(os.environ.get("LMK_BWD_HANDOVER_MAX_MB", "160")) << 20
# ... and only for sequences from this many keys on: below, the recomputing pair is as fast or faster (B4 H32 L512:
# 112 against 114 us for forward + backward; B2 H32 L1024: 159 against 160) in a fraction of the workspace, while a
# few long heads gain 3-4 % (B1 H16 L2048: 188 against 193 us, B1 H8 L4096: 330 against 345).
HANDOVER_MIN_KEYS = int(os.environ.get("LMK_BWD_HANDOVER_MIN_KEYS", "2048"))
PADDED_HEAD_DIMS = (16, 32)          # accepted by fused_landmark_attention, zero-padded to 64


def storage_block(block_size: int) -> int:
    """Slots per block the kernels work on for blocks of ``block_size`` tokens."""
    if block_size in SUPPORTED_BLOCKS:
        return block_size
    if not 2 <= block_size <= MAX_BLOCK:
        raise ValueError(f"block_size {block_size} is outside what the HIP kernels cover (2..{MAX_BLOCK})")
    return 64 if block_size <= 64 else 128


def _repack(x, block_size, block, unpad=False, rows=None):
    """Pad (or, with ``unpad``, strip) the blocks of a (B, H, L, D) tensor; ``rows`` = real rows."""
    B, H, _, D = x.shape
    lib = _lib.lib()
    rows = x.shape[2] if rows is None else rows
    out_rows = rows if unpad else lib.lmk_padded_rows(rows, int(block_size), int(block))
    out = torch.empty((B, H, out_rows, D), device=x.device, dtype=x.dtype)
    fn = lib.lmk_unpad_blocks if unpad else lib.lmk_pad_blocks
    _lib.check(fn(_lib.tensor4(x), _lib.tensor4(out), B, H, rows, D, int(block_size), int(block),
                  _lib.current_stream(x.device)))
    return out


def _launch_fwd_blocks(q, k, v, n_prefix, sm_scale, block_tokens):
    """Forward for any block size 2..128 on the tensors as they are; L, M are indexed by token rows."""
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    o = torch.empty_like(q)
    L = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
    M = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
    rc = _lib.lib().lmk_attn_fwd_blocks(_lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o),
                                        L.data_ptr(), M.data_ptr(), B, H, Lq, Lk, D, float(sm_scale), int(block_tokens),
                                        int(n_prefix), _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
    _lib.check(rc)
    return o, L, M


def _launch_bwd_blocks(q, k, v, o, do, L, M, n_prefix, sm_scale, block_tokens):
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    lib = _lib.lib()
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    nbytes = lib.lmk_attn_bwd_blocks_workspace_bytes(B, H, Lq, Lk, int(block_tokens))
    ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
    rc = lib.lmk_attn_bwd_blocks(_lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o), _lib.tensor4(do),
                                 L.data_ptr(), M.data_ptr(), _lib.tensor4(dq), _lib.tensor4(dk), _lib.tensor4(dv),
                                 ws.data_ptr(), nbytes, B, H, Lq, Lk, D, float(sm_scale), int(block_tokens),
                                 int(n_prefix), _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
    _lib.check(rc)
    return dq, dk, dv


def _launch_fwd(q, k, v, n_prefix, sm_scale, block, block_real=None):
    block_real = block if block_real is None else block_real
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    o = torch.empty_like(q)        # keeps q's memory layout: a (B,L,H,D)-backed q gives an output whose
    #                                transpose(1, 2).reshape(B, L, H*D) for o_proj (llama_mem.py:484-486) is a view
    L = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
    M = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
    rc = _lib.lib().lmk_attn_fwd_padded(_lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o),
                                        L.data_ptr(), M.data_ptr(), B, H, Lq, Lk, D, float(sm_scale), int(block),
                                        int(block_real), int(n_prefix), _lib.DTYPE_CODES[q.dtype],
                                        _lib.current_stream(q.device))
    _lib.check(rc)
    return o, L, M


def _launch_bwd(q, k, v, o, do, L, M, n_prefix, sm_scale, block, block_real=None):
    block_real = block if block_real is None else block_real
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    lib = _lib.lib()
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)     # each in its input's layout
    nbytes = lib.lmk_attn_bwd_workspace_bytes(B, H, Lq, Lk, int(block))
    if block_real == block:
        ho = lib.lmk_attn_bwd_handover_workspace_bytes(B, H, Lq, Lk, int(block))
        if 0 < ho <= HANDOVER_MAX_BYTES and Lk >= HANDOVER_MIN_KEYS:
            nbytes = ho          # the library picks the hand-over kernels from the size it is handed
    ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
    rc = lib.lmk_attn_bwd_padded(_lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o),
                                 _lib.tensor4(do), L.data_ptr(), M.data_ptr(), _lib.tensor4(dq), _lib.tensor4(dk),
                                 _lib.tensor4(dv), ws.data_ptr(), nbytes, B, H, Lq, Lk, D, float(sm_scale),
                                 int(block), int(block_real), int(n_prefix), _lib.DTYPE_CODES[q.dtype],
                                 _lib.current_stream(q.device))
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
        block = storage_block(block_size)
        q, k, v = _lib.kernel_ready(q), _lib.kernel_ready(k), _lib.kernel_ready(v)
        ctx.sm_scale = sm_scale
        ctx.N_PREFIX_Q = n_prefix_q
        ctx.BLOCK = block_size
        ctx.real_rows = (seqlen_q, seqlen_k)
        with _lib.on_device(q.device):
            if block == block_size:
                o, L, m = _launch_fwd(q, k, v, n_prefix_q, sm_scale, block_size)
            else:
                o, L, m = _launch_fwd_blocks(q, k, v, n_prefix_q, sm_scale, block_size)
            ctx.save_for_backward(q, k, v, o, L, m)
            return o

    @staticmethod
    def backward(ctx, do):
        BLOCK = ctx.BLOCK
        q, k, v, o, l, m = ctx.saved_tensors
        rows_q, rows_k = ctx.real_rows
        assert rows_q % BLOCK == 0, "Backward supported only for full blocks"
        assert rows_k % BLOCK == 0, "Backward supported only for full blocks"
        block = storage_block(BLOCK)
        do = _lib.kernel_ready(do)
        with _lib.on_device(q.device):
            if block == BLOCK:
                dq, dk, dv = _launch_bwd(q, k, v, o, do, l, m, ctx.N_PREFIX_Q, ctx.sm_scale, BLOCK)
            else:
                dq, dk, dv = _launch_bwd_blocks(q, k, v, o, do, l, m, ctx.N_PREFIX_Q, ctx.sm_scale, BLOCK)
        return dq, dk, dv, None, None, None


class FusedLandmarkAttentionGroupScale(torch.autograd.Function):
    """``FusedLandmarkAttention`` with group dropout (``lm_benchmark/models/landmark.py:110-113``): ``group_scale``
    (B, H, Lk / block_size, Lq) fp32 multiplies what earlier block b contributes to query row i -- 0 for a dropped
    block, 1 / (1 - p) for a kept one -- while the softmax over the landmarks is left as it is.  The draw is the
    caller's (e.g. ``torch.nn.functional.dropout(torch.ones(...), p)``), so results are reproducible from the mask."""

    @staticmethod
    def forward(ctx, q, k, v, group_scale, n_prefix_q, sm_scale, block_size):
        B, H, Lq, D = q.shape
        Lk = k.shape[2]
        assert k.shape == v.shape == (B, H, Lk, D) and q.dtype == k.dtype == v.dtype and q.dtype in _lib.DTYPE_CODES
        assert q.is_cuda and D in SUPPORTED_HEAD_DIMS and 2 <= block_size <= MAX_BLOCK
        assert group_scale.shape == (B, H, Lk // block_size, Lq) and group_scale.dtype == torch.float32
        assert group_scale.device == q.device
        q, k, v = _lib.kernel_ready(q), _lib.kernel_ready(k), _lib.kernel_ready(v)
        group_scale = group_scale.contiguous()
        o = torch.empty_like(q)
        L = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
        M = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
        with _lib.on_device(q.device):
            rc = _lib.lib().lmk_attn_fwd_group_scale(
                _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o), L.data_ptr(), M.data_ptr(),
                group_scale.data_ptr(), B, H, Lq, Lk, D, float(sm_scale), int(block_size), int(n_prefix_q),
                _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
        _lib.check(rc)
        ctx.save_for_backward(q, k, v, o, L, M, group_scale)
        ctx.args = (n_prefix_q, sm_scale, block_size)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, L, M, group_scale = ctx.saved_tensors
        n_prefix_q, sm_scale, block_size = ctx.args
        B, H, Lq, D = q.shape
        Lk = k.shape[2]
        assert Lq % block_size == 0 and Lk % block_size == 0, "Backward supported only for full blocks"
        do = _lib.kernel_ready(do)
        lib = _lib.lib()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        nbytes = lib.lmk_attn_bwd_group_scale_workspace_bytes(B, H, Lq, Lk, int(block_size))
        ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
        with _lib.on_device(q.device):
            rc = lib.lmk_attn_bwd_group_scale(
                _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o), _lib.tensor4(do), L.data_ptr(),
                M.data_ptr(), group_scale.data_ptr(), _lib.tensor4(dq), _lib.tensor4(dk), _lib.tensor4(dv), ws.data_ptr(),
                nbytes, B, H, Lq, Lk, D, float(sm_scale), int(block_size), int(n_prefix_q), _lib.DTYPE_CODES[q.dtype],
                _lib.current_stream(q.device))
        _lib.check(rc)
        return dq, dk, dv, None, None, None, None


class LandmarkSegments:
    """Blocks of unequal length cut out by a mask with landmarks at irregular positions: ``seg[b]`` is the first
    token of block b, every block ends in its landmark except -- ``last_is_partial`` -- the tokens behind the last
    landmark.  Held on the host (checked by every call of the library) and on the device (read by the kernels)."""

    def __init__(self, is_mem_row, device):
        import ctypes
        marks = [bool(x) for x in is_mem_row]
        ends = [j + 1 for j, m in enumerate(marks) if m]
        self.last_is_partial = not marks or not marks[-1]
        seg = [0] + ends + ([len(marks)] if self.last_is_partial else [])
        self.n_blocks = len(seg) - 1
        lengths = [b - a for a, b in zip(seg[:-1], seg[1:])]
        n_full = self.n_blocks - int(self.last_is_partial)
        # the tokens behind the last landmark count one more: their block must leave its last slot, the landmark's, free
        widths = lengths[:n_full] + ([lengths[-1] + 1] if self.last_is_partial else [])
        assert self.n_blocks > 0 and max(widths) <= MAX_BLOCK, \
            f"a block of more than {MAX_BLOCK} tokens between two landmarks is outside what the HIP kernels cover"
        assert all(n >= 2 for n in lengths[:n_full]), "two landmarks in a row (a block without a normal token) are not covered"
        self.max_len = max(max(widths), 2)
        self.seg = seg
        self.seg_host = (ctypes.c_int32 * len(seg))(*seg)
        self.seg_dev = torch.tensor(seg, dtype=torch.int32, device=device)

    def history_blocks(self, n_history_tokens: int) -> int:
        assert n_history_tokens in self.seg[:-1], "the keys in front of the first query must be whole blocks"
        return self.seg.index(n_history_tokens)


class FusedLandmarkAttentionSegments(torch.autograd.Function):
    """``FusedLandmarkAttention`` for landmarks at irregular positions (blocks of unequal length, each at most 128
    tokens): the grouped softmax of the reference's high-level path (``llama/llama_mem.py:222-243``) on the fused
    kernels.  The reference's own fused path rejects such masks (``flash_landmark_attention.py:393-394``)."""

    @staticmethod
    def forward(ctx, q, k, v, segments, sm_scale):
        B, H, Lq, D = q.shape
        Lk = k.shape[2]
        assert k.shape == v.shape == (B, H, Lk, D) and q.dtype == k.dtype == v.dtype and q.dtype in _lib.DTYPE_CODES
        assert q.is_cuda and D in SUPPORTED_HEAD_DIMS and segments.seg[-1] == Lk
        n_prefix = segments.history_blocks(Lk - Lq)
        q, k, v = _lib.kernel_ready(q), _lib.kernel_ready(k), _lib.kernel_ready(v)
        o = torch.empty_like(q)
        L = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
        M = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
        with _lib.on_device(q.device):
            rc = _lib.lib().lmk_attn_fwd_segments(
                _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o), L.data_ptr(), M.data_ptr(),
                segments.seg_host, segments.seg_dev.data_ptr(), segments.n_blocks, segments.max_len,
                int(segments.last_is_partial), B, H, Lq, Lk, D, float(sm_scale), n_prefix, _lib.DTYPE_CODES[q.dtype],
                _lib.current_stream(q.device))
        _lib.check(rc)
        ctx.save_for_backward(q, k, v, o, L, M)
        ctx.args = (segments, n_prefix, sm_scale)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, L, M = ctx.saved_tensors
        segments, n_prefix, sm_scale = ctx.args
        assert not segments.last_is_partial, "Backward supported only for full blocks"
        B, H, Lq, D = q.shape
        Lk = k.shape[2]
        do = _lib.kernel_ready(do)
        lib = _lib.lib()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        nbytes = lib.lmk_attn_bwd_segments_workspace_bytes(B, H, segments.n_blocks, n_prefix, segments.max_len)
        ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
        with _lib.on_device(q.device):
            rc = lib.lmk_attn_bwd_segments(
                _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o), _lib.tensor4(do), L.data_ptr(),
                M.data_ptr(), _lib.tensor4(dq), _lib.tensor4(dk), _lib.tensor4(dv), ws.data_ptr(), nbytes,
                segments.seg_host, segments.seg_dev.data_ptr(), segments.n_blocks, segments.max_len, B, H, Lq, Lk, D,
                float(sm_scale), n_prefix, _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
        _lib.check(rc)
        return dq, dk, dv, None, None


# Masks that have already passed the check of ``flash_landmark_attention.py:393-394``, keyed by what
# identifies a tensor's content without reading it: storage address, in-place version counter, layout.
# (A write through ``.data`` or a custom kernel bypasses the counter; such a mask has to be a new tensor.)
# A layer stack hands the same mask to every layer and every step, so the device->host sync of the
# comparison is paid once per mask instead of once per call.
_VALIDATED_MASKS: dict = {}
_VALIDATED_MASKS_MAX = 64


def _check_is_mem(is_mem, block_size, offset=0, irregular_ok=False):
    """None when ``is_mem`` marks exactly the last token of every block of ``block_size`` (the check of
    ``flash_landmark_attention.py:393-394``); otherwise an AssertionError -- or, with ``irregular_ok``, the
    ``LandmarkSegments`` of the mask.  offset: tokens of the first block that lie in front of the mask (a stream
    cut between two landmarks)."""
    # tensors created under torch.inference_mode() track no version counter (reading it raises): they are checked
    # on every call rather than cached
    cacheable = not is_mem.is_inference()
    if cacheable:
        key = (is_mem.device, is_mem.data_ptr(), is_mem._version, tuple(is_mem.shape), tuple(is_mem.stride()),
               is_mem.dtype, int(block_size), int(offset))
        if key in _VALIDATED_MASKS:
            found = _VALIDATED_MASKS[key][1]
            assert found is None or irregular_ok, _IRREGULAR_MESSAGE.format(block_size)
            return found
    expected_is_mem = (torch.arange(0, is_mem.shape[-1], device=is_mem.device) + offset) % block_size == (block_size - 1)
    found = None
    if not bool((is_mem == expected_is_mem).all()):
        assert irregular_ok, _IRREGULAR_MESSAGE.format(block_size)
        rows = is_mem.reshape(-1, is_mem.shape[-1])
        assert bool((rows == rows[:1]).all()), "landmarks at irregular positions must be the same for every sequence of the batch"
        found = LandmarkSegments(rows[0].tolist(), is_mem.device)
    if cacheable:
        if len(_VALIDATED_MASKS) >= _VALIDATED_MASKS_MAX:
            _VALIDATED_MASKS.clear()
        # the entry keeps the tensor alive, so its address cannot be handed to another mask meanwhile
        _VALIDATED_MASKS[key] = (is_mem, found)
    return found


_IRREGULAR_MESSAGE = ("is_mem must mark exactly the last token of every block of {}: landmarks at irregular positions "
                      "are covered by fused_landmark_attention only (head dims 64 and 128, no group dropout)")


def fused_landmark_attention(q, k, v, is_mem, sm_scale=None, block_size=64, group_scale=None):
    """Landmark grouped-softmax causal attention, landmarks at every ``block_size``-th key.

    q: (B, H, Lq, D); k, v: (B, H, Lk, D) with ``Lk - Lq`` a whole number of blocks of
    history.  ``is_mem`` (bool, last dim Lk) marks the positions ``j % block_size == block_size - 1``
    (checked as in the reference, ``:393-394``; the check costs one device->host sync, paid once per
    distinct mask tensor state, not per call); pass ``None`` to skip the check.  A mask with landmarks
    at other positions -- which the reference's fused path rejects and only its high-level path takes --
    runs on the same kernels with blocks of unequal length (``FusedLandmarkAttentionSegments``: every
    block at most 128 tokens and at least one normal token, the same mask for every sequence of the
    batch, the keys in front of the first query whole blocks).  ``group_scale`` (not in the reference's signature): the group-dropout factors of
    ``FusedLandmarkAttentionGroupScale``, (B, H, Lk / block_size, Lq) fp32, for head dims 64 and 128.
    """
    if is_mem is not None:
        segments = _check_is_mem(is_mem, block_size, irregular_ok=group_scale is None)
        if segments is not None:
            # not in the reference's fused path (its check rejects the mask): blocks of unequal length, what its
            # high-level path computes for such a mask; block_size plays no part
            if sm_scale is None:
                sm_scale = 1.0 / math.sqrt(q.size(-1))
            return FusedLandmarkAttentionSegments.apply(q, k, v, segments, sm_scale)

    n_history_kv = k.shape[-2] - q.shape[-2]
    assert n_history_kv % block_size == 0
    n_history_blocks = n_history_kv // block_size

    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.size(-1))

    if group_scale is not None:
        return FusedLandmarkAttentionGroupScale.apply(q, k, v, group_scale, n_history_blocks, sm_scale, block_size)

    d = q.size(-1)
    if d in PADDED_HEAD_DIMS:
        # head dims 16 and 32 (flash_landmark_attention.py:321) run on the 64-wide kernels: zero columns add
        # nothing to a score and give zero output columns, which are dropped again; autograd differentiates
        # through the padding and the slice
        pad = (0, 64 - d)
        q, k, v = (torch.nn.functional.pad(t, pad) for t in (q, k, v))
        return FusedLandmarkAttention.apply(q, k, v, n_history_blocks, sm_scale, block_size)[..., :d]
    return FusedLandmarkAttention.apply(q, k, v, n_history_blocks, sm_scale, block_size)


def fused_landmark_attention_rotary_q(q, k, v, cos, sin, position_ids, is_mem=None, sm_scale=None, block_size=64):
    """Forward only (no autograd): ``fused_landmark_attention(rot(q), k, v, ...)`` with the rotary embedding of
    ``q`` (``apply_rotary_pos_emb``, ``llama/llama_mem.py:298``) applied inside the kernel as it loads the
    queries -- same bits as rotating first, one pass over ``q`` less.  ``k`` must already be rotated.

    q: (B, H, Lq, D) without rotary; cos, sin: (n_pos, D) or (1, 1, n_pos, D) model-dtype tables;
    position_ids: int64 (B, Lq) or (1, Lq), the positions of the query rows.  Native block sizes only."""
    from .retrieval import _tables
    assert not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)), \
        "forward only: rotate q with apply_rotary_pos_emb and call fused_landmark_attention to differentiate"
    if is_mem is not None:
        _check_is_mem(is_mem, block_size)
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    assert k.shape == v.shape == (B, H, Lk, D) and q.dtype == k.dtype == v.dtype and q.dtype in _lib.DTYPE_CODES
    assert q.is_cuda and D in SUPPORTED_HEAD_DIMS and block_size in SUPPORTED_BLOCKS
    assert (Lk - Lq) % block_size == 0
    assert position_ids.dim() == 2 and position_ids.shape[1] == Lq and position_ids.shape[0] in (1, B)
    assert position_ids.dtype == torch.int64 and position_ids.device == q.device
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    cos, sin = _tables(cos, sin, q.dtype)
    q, k, v = _lib.kernel_ready(q), _lib.kernel_ready(k), _lib.kernel_ready(v)
    position_ids = position_ids.contiguous()
    o = torch.empty_like(q)
    L = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
    M = torch.empty((B * H, Lq), device=q.device, dtype=torch.float32)
    with _lib.on_device(q.device):
        rc = _lib.lib().lmk_attn_fwd_rotary_q(
            _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o), L.data_ptr(), M.data_ptr(),
            cos.data_ptr(), sin.data_ptr(), cos.stride(0), cos.shape[0], position_ids.data_ptr(),
            Lq if position_ids.shape[0] == B and B > 1 else 0, B, H, Lq, Lk, D, float(sm_scale), int(block_size),
            (Lk - Lq) // block_size, _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
    _lib.check(rc)
    return o
