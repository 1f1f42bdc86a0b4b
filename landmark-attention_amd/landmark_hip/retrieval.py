"""Mem-cache retrieval at inference: landmark scoring, top-k block selection and
attention over the gathered blocks, on the HIP kernels.

Mirrors ``LlamaAttention.forward`` (``llama/llama_mem.py:318-430`` retrieval, ``:447-477``
attend): the per-head, per-token selection (``aggregate is None``) and the selection shared by
all queries of a head (``aggregate == "max_over_tokens"``, ``:373-377``), with the reference's own
conventions: ``past_key_value = (K_without_rotary, V)`` each ``(B, nh, S, hd)`` (``:424-430``),
``block = mem_freq + 1`` with the landmark as the last token of a block, queries and local
keys already rotated (``:298``), ``cos/sin`` the model-dtype tables of
``LlamaRotaryEmbedding`` (``:121-124``).  The cache may end in an incomplete block (the state
between two landmarks while decoding): retrieval then covers the complete blocks and the tail
joins the local window (``:321-342``).
"""
from __future__ import annotations

import math

import torch

from . import _lib
from .attention import _launch_fwd


def _tables(cos, sin, dtype):
    cos = cos.reshape(-1, cos.shape[-1])
    sin = sin.reshape(-1, sin.shape[-1])
    assert cos.dtype == sin.dtype == dtype, "rotary tables must be in the model dtype (llama_mem.py:121-124)"
    assert cos.shape == sin.shape
    if cos.stride(1) != 1 or cos.stride(0) % 8 or cos.data_ptr() % 16:
        cos = cos.contiguous()
    if sin.stride(1) != 1 or sin.stride(0) != cos.stride(0) or sin.data_ptr() % 16:
        sin = sin.contiguous()
        cos = cos.contiguous()
    return cos, sin


def retrieve_topk(q, k_cache, cos, sin, block: int, top_k: int, aggregate=None, return_block_probs=False,
                  workspace=None, reuse_landmark_keys=False):
    """Indices ``(B, nh, T, k)`` int64, ascending, of the ``k = min(top_k, S // block)`` cached
    blocks whose landmark keys score highest against each query (``llama_mem.py:344-384``).

    Equivalent to ``(q @ rot(landmark_keys)^T / sqrt(hd)).topk(k).indices.sort()`` with the
    product accumulated sequentially in fp32 and ties broken towards the lower index.

    ``aggregate="max_over_tokens"`` (``:373-377``): one set per head, ``(B, nh, 1, k)`` -- the
    scores go through an fp32 softmax over the blocks, are rounded to the model dtype and reduced
    with a maximum over the queries before the top-k; ``return_block_probs`` also returns that
    per-head vector ``(B, nh, 1, S // block)`` (``mem_attn_weights`` after ``:377``).

    ``workspace``: a uint8 device tensor to use instead of a fresh allocation (at least
    ``lmk_retrieve_workspace_bytes`` long).  ``reuse_landmark_keys``: the workspace still holds the
    rotated landmark keys of the previous call and neither the complete cached blocks nor their
    number have changed -- the case of every decode step between two landmarks -- so they are not
    rotated again (per-token selection only)."""
    if aggregate not in (None, "max_over_tokens"):
        raise NotImplementedError(aggregate)                            # llama_mem.py:381-382
    assert aggregate or not return_block_probs, "the per-head vector exists only with aggregate='max_over_tokens'"
    B, H, T, D = q.shape
    S = k_cache.shape[2]
    assert k_cache.shape == (B, H, S, D) and q.dtype == k_cache.dtype and q.is_cuda and k_cache.is_cuda
    q, k_cache = _lib.kernel_ready(q), _lib.kernel_ready(k_cache)
    cos, sin = _tables(cos, sin, q.dtype)
    lib = _lib.lib()
    k = min(top_k, S // block)                      # complete blocks only (llama_mem.py:321-324,358-359)
    idx = torch.empty((B, H, 1 if aggregate else T, k), device=q.device, dtype=torch.int64)
    nbytes = lib.lmk_retrieve_workspace_bytes(B, H, T, S, D, int(block))
    probs = None
    assert not (reuse_landmark_keys and (aggregate or workspace is None))
    with _lib.on_device(q.device):
        if workspace is None:
            ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
        else:
            ws = workspace
            assert ws.dtype == torch.uint8 and ws.is_contiguous() and ws.numel() >= nbytes and ws.device == q.device
        tail = (ws.data_ptr(), nbytes, B, H, T, S, D, int(block), int(top_k), _lib.DTYPE_CODES[q.dtype],
                _lib.current_stream(q.device))
        head = (_lib.tensor4(q), _lib.tensor4(k_cache), cos.data_ptr(), sin.data_ptr(), cos.stride(0), cos.shape[0],
                idx.data_ptr())
        if aggregate:
            if return_block_probs:
                probs = torch.empty((B, H, 1, S // block), device=q.device, dtype=q.dtype)
            rc = lib.lmk_retrieve_topk_shared(*head, probs.data_ptr() if return_block_probs else None, *tail)
        elif reuse_landmark_keys:
            rc = lib.lmk_retrieve_topk_reuse(*head, *tail)
        else:
            rc = lib.lmk_retrieve_topk(*head, *tail)
    _lib.check(rc)
    return (idx, probs) if return_block_probs else idx


def retrieve_topk_from_landmarks(q, landmark_keys, cos, sin, block: int, top_k: int, workspace=None):
    """The ``max_over_tokens`` selection when the cached blocks are not on the GPU (``offload_cache_to_cpu``,
    ``llama_mem.py:326-328,344-356``): ``landmark_keys (B, nh, n_blocks, hd)`` is ``past_key_value[2]`` of that
    branch, the un-rotated landmark key of every complete block.  Returns ``(B, nh, 1, k)`` int64, as
    ``retrieve_topk(..., aggregate="max_over_tokens")`` does for the same blocks."""
    B, H, T, D = q.shape
    n = landmark_keys.shape[2]
    assert landmark_keys.shape == (B, H, n, D) and q.dtype == landmark_keys.dtype and q.is_cuda and landmark_keys.is_cuda
    q, landmark_keys = _lib.kernel_ready(q), _lib.kernel_ready(landmark_keys)
    cos, sin = _tables(cos, sin, q.dtype)
    lib = _lib.lib()
    idx = torch.empty((B, H, 1, min(top_k, n)), device=q.device, dtype=torch.int64)
    nbytes = lib.lmk_retrieve_workspace_bytes(B, H, T, n * int(block), D, int(block))
    with _lib.on_device(q.device):
        ws = workspace if workspace is not None and workspace.numel() >= nbytes else \
            torch.empty(nbytes, device=q.device, dtype=torch.uint8)
        rc = lib.lmk_retrieve_topk_shared_landmarks(
            _lib.tensor4(q), _lib.tensor4(landmark_keys), cos.data_ptr(), sin.data_ptr(), cos.stride(0), cos.shape[0],
            idx.data_ptr(), None, ws.data_ptr(), nbytes, B, H, T, n, D, int(block), int(top_k),
            _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
    _lib.check(rc)
    return idx


def gather_attend(q, k_cache, v_cache, idx, k_loc, v_loc, cos, sin, block: int, top_k: int, sm_scale=None):
    """Attention output ``(B, nh, T, hd)`` over the blocks ``idx`` selects plus the local window
    (``llama_mem.py:386-412,447-477``).  The local window -- the new chunk, behind the tail of
    an incomplete cached block if there is one (``:329-342``) -- is attended with the fused
    forward kernel; the gather kernel reads the selected blocks in place and merges both parts."""
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
    q, k_cache, v_cache, k_loc, v_loc = (_lib.kernel_ready(t) for t in (q, k_cache, v_cache, k_loc, v_loc))
    cos, sin = _tables(cos, sin, q.dtype)
    return _attend(q, k_cache, v_cache, idx, k_loc, v_loc, cos, sin, block, top_k, sm_scale)


def _attend(q, k_cache, v_cache, idx, k_loc, v_loc, cos, sin, block, top_k, sm_scale):
    """Local window, fused forward on it and gather + attend through the one-call entry point (inputs
    already in kernel layout): one trip through the binding instead of three, one scratch allocation
    instead of six -- a decode step spends more time on the host than on the GPU."""
    B, H, T, D = q.shape
    S = k_cache.shape[2]
    assert idx.dtype == torch.int64 and idx.is_contiguous() and idx.shape[:3] == (B, H, T)
    assert S % block == 0 or T + S % block <= block, "new chunk and cached tail must fit one block (llama_mem.py:330)"
    lib = _lib.lib()
    nbytes = lib.lmk_attend_workspace_bytes(B, H, T, S, D, int(block))
    with _lib.on_device(q.device):
        ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
        out = torch.empty_like(q)
        _lib.check(lib.lmk_attend(
            _lib.tensor4(q), _lib.tensor4(k_cache), _lib.tensor4(v_cache), idx.data_ptr(), _lib.tensor4(k_loc),
            _lib.tensor4(v_loc), cos.data_ptr(), sin.data_ptr(), cos.stride(0), cos.shape[0], _lib.tensor4(out),
            ws.data_ptr(), nbytes, B, H, T, S, D, float(sm_scale), int(block), int(top_k),
            _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device)))
    return out


def attend_shared(q, k_cache, v_cache, idx, k_loc, v_loc, cos, sin, block: int, top_k: int, sm_scale=None):
    """Attention output ``(B, nh, T, hd)`` when all queries of a head share the blocks
    ``idx (B, nh, 1, k)`` (``llama_mem.py:400-406``): the selected blocks, rotated at their slot
    positions, and the local window form one key/value sequence, and the fused forward kernel
    runs on it with the selected blocks as history (``:441-446``)."""
    B, H, T, D = q.shape
    S = k_cache.shape[2]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    q, k_cache, v_cache, k_loc, v_loc = (_lib.kernel_ready(t) for t in (q, k_cache, v_cache, k_loc, v_loc))
    cos, sin = _tables(cos, sin, q.dtype)
    inc = S % block
    k = min(top_k, S // block)
    assert idx.shape == (B, H, 1, k) and idx.dtype == torch.int64 and idx.is_contiguous()
    assert inc == 0 or T + inc <= block, "new chunk and cached tail must fit one block (llama_mem.py:330)"
    with _lib.on_device(q.device):
        k_win, v_win = (torch.empty((B, H, k * block + inc + T, D), device=q.device, dtype=q.dtype) for _ in range(2))
        q_win = torch.empty((B, H, inc + T, D), device=q.device, dtype=q.dtype) if inc else None
        _lib.check(_lib.lib().lmk_gather_window(
            _lib.tensor4(q), _lib.tensor4(k_cache), _lib.tensor4(v_cache), idx.data_ptr(), _lib.tensor4(k_loc),
            _lib.tensor4(v_loc), cos.data_ptr(), sin.data_ptr(), cos.stride(0), cos.shape[0],
            _lib.tensor4(q_win) if inc else None, _lib.tensor4(k_win), _lib.tensor4(v_win), B, H, T, S, D, int(block),
            int(top_k), _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device)))
        o, _, _ = _launch_fwd(q_win if inc else q, k_win, v_win, k, sm_scale, block)
    return o[:, :, inc:] if inc else o


def retrieve_and_attend(q, past_key_value, k_loc, v_loc, cos, sin, block: int, top_k: int, sm_scale=None,
                        aggregate=None, workspace=None, reuse_landmark_keys=False):
    """One inference step of the mem-cache path: returns ``(out, idx)``.

    ``past_key_value = (K_without_rotary, V)``; ``k_loc`` rotated, ``v_loc``: the new chunk.
    ``aggregate`` as in ``llama_mem.py:369-382``: ``None`` selects per (head, query),
    ``"max_over_tokens"`` once per head.  The caller appends the un-rotated new keys and values to
    the cache afterwards (``:424-430``)."""
    k_cache, v_cache = past_key_value[0], past_key_value[1]
    if aggregate:
        idx = retrieve_topk(q, k_cache, cos, sin, block, top_k, aggregate)
        return attend_shared(q, k_cache, v_cache, idx, k_loc, v_loc, cos, sin, block, top_k, sm_scale), idx
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
    q, k_cache, v_cache, k_loc, v_loc = (_lib.kernel_ready(t) for t in (q, k_cache, v_cache, k_loc, v_loc))
    cos, sin = _tables(cos, sin, q.dtype)
    # Selection and attend step through the one-call entry point.  (Running the local-window attention on a
    # second stream beside the selection was tried: the fork and join cost more than the 20 us it hides.)
    B, H, T, D = q.shape
    S = k_cache.shape[2]
    assert k_cache.shape == (B, H, S, D) and q.dtype == k_cache.dtype and q.is_cuda and k_cache.is_cuda
    assert S % block == 0 or T + S % block <= block, "new chunk and cached tail must fit one block (llama_mem.py:330)"
    assert not (reuse_landmark_keys and workspace is None)
    lib = _lib.lib()
    rbytes = lib.lmk_retrieve_workspace_bytes(B, H, T, S, D, int(block))
    abytes = lib.lmk_attend_workspace_bytes(B, H, T, S, D, int(block))
    with _lib.on_device(q.device):
        if workspace is None:
            workspace = torch.empty(rbytes, device=q.device, dtype=torch.uint8)
        else:
            assert (workspace.dtype == torch.uint8 and workspace.is_contiguous() and workspace.numel() >= rbytes
                    and workspace.device == q.device)
        idx = torch.empty((B, H, T, min(top_k, S // block)), device=q.device, dtype=torch.int64)
        aws = torch.empty(abytes, device=q.device, dtype=torch.uint8)
        out = torch.empty_like(q)
        _lib.check(lib.lmk_retrieve_and_attend(
            _lib.tensor4(q), _lib.tensor4(k_cache), _lib.tensor4(v_cache), _lib.tensor4(k_loc), _lib.tensor4(v_loc),
            cos.data_ptr(), sin.data_ptr(), cos.stride(0), cos.shape[0], idx.data_ptr(), _lib.tensor4(out),
            workspace.data_ptr(), rbytes, int(bool(reuse_landmark_keys)), aws.data_ptr(), abytes, B, H, T, S, D,
            float(sm_scale), int(block), int(top_k), _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device)))
    return out, idx
