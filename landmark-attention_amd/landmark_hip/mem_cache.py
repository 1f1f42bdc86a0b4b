"""Ring cache of landmark blocks with block selection on the GPU.

Host-side mirror of ``MemLMCacheStorage`` (``lm_benchmark/models/caches/mem_cache.py:21-158``): the same
buffers (``cache_mem_k/v`` of shape (B, mem_cache_size, block, nh, hs), the tokens behind the last complete
block in ``last_incomplete_*``), the same counters (``cache_iter`` = next slot to write = oldest block once
the ring is full, ``cache_size``, ``last_incomplete_len``) and the same ``store_in_cache`` behaviour,
including the newest-blocks-win truncation of a chunk larger than the ring.  The selection half of
``retrieve_for_query`` (``:50-85``) runs in the HIP library: landmark keys are read from the ring in
place, rotated at the positions of ``:56-58``, scored, soft-maxed, reduced by ``cache_selection_method``
and the ``cache_topk`` best slots come back ordered by age, as the reference's order-restoring sort
leaves them.  ``attend`` is the rest of ``retrieve_for_query`` (``:86-109``) together with the attention the
layer computes over its result (``lm_benchmark/models/landmark.py:192-240``): the picked blocks are read in
place from the ring, rotated at ``k_indices``, and merged with the chunk's own attention through the grouped
softmax.  Buffers are kept in the 16-bit model dtype (the reference's are fp32 holding 16-bit values
under autocast).
"""
from __future__ import annotations

import torch

from . import _lib
from .retrieval import _tables

SELECTION_METHODS = {"per_token_and_head": 0, "max_over_heads": 1, "max_over_tokens": 2}


class MemLMCacheStorage:
    def __init__(self, batch_size: int, mem_cache_size: int, mem_cache_freq: int, n_head: int, head_dim: int,
                 dtype=torch.bfloat16, device="cuda", cache_topk: int = 1,
                 cache_selection_method: str = "per_token_and_head"):
        if cache_selection_method not in SELECTION_METHODS:
            raise NotImplementedError(cache_selection_method)                        # mem_cache.py:69-70
        block = mem_cache_freq + 1
        self.cache_topk, self.cache_selection_method = cache_topk, cache_selection_method
        self.cache_mem_k = torch.empty((batch_size, mem_cache_size, block, n_head, head_dim), dtype=dtype, device=device)
        self.cache_mem_v = torch.empty_like(self.cache_mem_k)
        self.last_incomplete_k = torch.empty((batch_size, n_head, block, head_dim), dtype=dtype, device=device)
        self.last_incomplete_v = torch.empty_like(self.last_incomplete_k)
        self.last_incomplete_ismem = torch.empty((batch_size, block), dtype=torch.bool, device=device)
        self._ws = None
        self.clear_state()

    def clear_state(self) -> None:
        self.last_incomplete_len = 0
        self.cache_iter = 0
        self.cache_size = 0

    # ------------------------------------------------------------------ geometry
    @property
    def block(self) -> int:
        return self.cache_mem_k.shape[2]

    @property
    def filled(self) -> int:
        """Slots that hold a block (``cache_size`` also counts blocks that were dropped, ``:143,158``)."""
        return min(self.cache_size, self.cache_mem_k.shape[1])

    @property
    def oldest_slot(self) -> int:
        n = self.filled
        return self.cache_iter % n if n else 0

    # --------------------------------------------------------------------- store
    def store_in_cache(self, keys, values_dict) -> None:
        """``store_in_cache`` (``:111-158``): keys (B, nh, T, hs) without positions, ``values_dict`` with
        ``'v'`` (B, nh, T, hs) and ``'is_mem'`` (B, T)."""
        B = keys.shape[0]
        n0, bs, cap = self.last_incomplete_len, self.block, self.cache_mem_k.shape[1]
        k = torch.cat((self.last_incomplete_k[:B, :, :n0], keys.to(self.cache_mem_k.dtype)), dim=2)
        v = torch.cat((self.last_incomplete_v[:B, :, :n0], values_dict["v"].to(self.cache_mem_v.dtype)), dim=2)
        is_mem = torch.cat((self.last_incomplete_ismem[:B, :n0], values_dict["is_mem"]), dim=1)
        _, nh, total, hs = k.shape
        rest = total % bs
        full = total - rest
        self.last_incomplete_k[:B, :, :rest] = k[:, :, full:]
        self.last_incomplete_v[:B, :, :rest] = v[:, :, full:]
        self.last_incomplete_ismem[:B, :rest] = is_mem[:, full:]
        self.last_incomplete_len = rest
        n_new = full // bs
        marks = is_mem[:, :full].view(B, n_new, bs)
        expected = torch.zeros(bs, dtype=torch.bool, device=marks.device)
        expected[-1] = True
        assert bool((marks == expected).all()), "every block must end in its landmark and hold no other"
        kept = min(n_new, cap)
        dropped = n_new - kept
        # (B, nh, rows, hs) -> (B, blocks, bs, nh, hs), newest `kept` blocks only
        kb = k[:, :, dropped * bs:full].transpose(1, 2).reshape(B, kept, bs, nh, hs)
        vb = v[:, :, dropped * bs:full].transpose(1, 2).reshape(B, kept, bs, nh, hs)
        start = (self.cache_iter + dropped) % cap
        first = min(kept, cap - start)                         # blocks that fit before the end of the ring
        self.cache_mem_k[:B, start:start + first] = kb[:, :first]
        self.cache_mem_v[:B, start:start + first] = vb[:, :first]
        self.cache_mem_k[:B, :kept - first] = kb[:, first:]
        self.cache_mem_v[:B, :kept - first] = vb[:, first:]
        self.cache_iter = (start + kept) % cap if start + kept >= cap else start + kept
        self.cache_size += n_new

    # ----------------------------------------------------------------- selection
    def select_blocks(self, q, cos, sin):
        """Slots of the ``cache_topk`` blocks each query retrieves, oldest first (``:50-85``).

        q: (B, nh, T, hs) rotated queries; cos, sin: (n_pos, hs) half-split tables in q's dtype.
        Returns int64 (B, nh, T, k) for ``per_token_and_head``, (B, T, k) for ``max_over_heads`` (one
        selection for all heads), (B, nh, k) for ``max_over_tokens`` (one for all queries)."""
        n = self.filled
        if n == 0 or self.cache_topk == 0:
            raise ValueError("nothing to select from: the cache holds no block or cache_topk is 0")   # :47-48 returns early
        B, nh, T, hs = q.shape
        assert q.dtype == self.cache_mem_k.dtype and q.is_cuda
        lib = _lib.lib()
        q = _lib.kernel_ready(q)
        cos, sin = _tables(cos, sin, q.dtype)
        kring = self.cache_mem_k[:B, :n].flatten(1, 2).transpose(1, 2)        # (B, nh, n*block, hs) view, no copy
        method = SELECTION_METHODS[self.cache_selection_method]
        shape = {0: (B, nh, T), 1: (B, T), 2: (B, nh)}[method] + (self.cache_topk,)
        idx = torch.empty(shape, dtype=torch.int64, device=q.device)
        nbytes = lib.lmk_retrieve_workspace_bytes(B, nh, T, n * self.block, hs, self.block)
        if self._ws is None or self._ws.numel() < nbytes or self._ws.device != q.device:
            self._ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        with _lib.on_device(q.device):
            rc = lib.lmk_ring_retrieve_topk(_lib.tensor4(q), _lib.tensor4(kring), cos.data_ptr(), sin.data_ptr(),
                                            cos.stride(0), cos.shape[0], idx.data_ptr(), self._ws.data_ptr(), nbytes, B,
                                            nh, T, n, hs, self.block, self.cache_topk, self.oldest_slot, method,
                                            _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
        _lib.check(rc)
        return idx

    def key_positions(self, idx):
        """``k_indices`` of ``:95-97`` for slots ``idx (..., k)``: positions at which the gathered keys are
        rotated, (..., k * block)."""
        n, k, bs = self.filled, self.cache_topk, self.block
        age = (idx - self.oldest_slot) % n
        newest = age >= n - k
        base = torch.arange(k * bs, device=idx.device).view(k, bs)
        return (newest.to(torch.int64) * bs).unsqueeze(-1).add(base).flatten(-2)

    # ------------------------------------------------------------ gather + attend
    def attend(self, q, k, v, is_mem, cos, sin, start_index: int, sm_scale=None):
        """Attention of a chunk over the cache and itself: ``retrieve_for_query`` (``mem_cache.py:41-109``)
        followed by what ``CausalSelfAttention.forward`` does between ``adapt_keys`` and ``c_proj``
        (``lm_benchmark/models/landmark.py:192-240``), without materialising the gathered blocks, the
        (T, prefix + T) score matrix or its masks.

        q, k: (B, nh, T, hs) rotated at positions ``start_index ..`` (``adapt_queries`` / ``adapt_keys``);
        v: (B, nh, T, hs); is_mem: (B, T) bool, which must continue the stream's pattern (a landmark closes every
        block of ``mem_cache_freq + 1`` tokens, counted from the first token behind the last complete block);
        cos, sin: (n_pos, hs) half-split tables in q's dtype, ``n_pos >= start_index + T``.
        Returns ``(y (B, nh, T, hs), slots)``: y is ``att @ v + att_prefix @ cache_v`` (``:235-240``), slots the
        picked blocks in the shape of ``select_blocks`` (None while the cache holds no block or ``cache_topk`` is 0,
        ``:48-49``).  Call ``store_in_cache`` afterwards, as the layer does (``:246-248``)."""
        from .attention import _check_is_mem, _launch_fwd_blocks
        import math
        B, nh, T, hs = q.shape
        block, tail = self.block, self.last_incomplete_len
        assert q.dtype == self.cache_mem_k.dtype and q.is_cuda and k.shape == v.shape == q.shape
        # is_mem must continue the stream (a landmark closes every block); the check costs a device->host sync, paid
        # once per mask tensor state and tail length, not per call
        _check_is_mem(is_mem, block, offset=tail)
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(hs)
        cos, sin = _tables(cos, sin, q.dtype)
        if tail:
            # the tokens behind the last complete block open the chunk's first block (:43-46): their keys rotated at
            # start_index - tail .., zero rows standing in for their queries -- one launch writes the three windows
            assert start_index >= tail
            q, k, v = (_lib.kernel_ready(t) for t in (q, k, v))
            q_win, k_win, v_win = (torch.empty((B, nh, tail + T, hs), dtype=q.dtype, device=q.device) for _ in range(3))
            with _lib.on_device(q.device):
                rc = _lib.lib().lmk_ring_local_window(
                    _lib.tensor4(q), _lib.tensor4(self.last_incomplete_k[:B]), _lib.tensor4(self.last_incomplete_v[:B]),
                    _lib.tensor4(k), _lib.tensor4(v), cos.data_ptr(), sin.data_ptr(), cos.stride(0), cos.shape[0],
                    _lib.tensor4(q_win), _lib.tensor4(k_win), _lib.tensor4(v_win), B, nh, T, tail,
                    int(start_index - tail), hs, _lib.DTYPE_CODES[q.dtype], _lib.current_stream(q.device))
            _lib.check(rc)
        else:
            q_win, k_win, v_win = (_lib.kernel_ready(t) for t in (q, k, v))
        W = tail + T
        with _lib.on_device(q.device):
            # blocks of any size up to 128 tokens, read as they are (the benchmark's 51 run in 64 slots)
            o_win, L, M = _launch_fwd_blocks(q_win, k_win, v_win, 0, sm_scale, block)
            o_loc, L_loc, M_loc, stat_stride = o_win[:, :, tail:], L[:, tail:], M[:, tail:], W
            n = self.filled
            if n == 0 or self.cache_topk == 0:
                return o_loc, None
            slots = self.select_blocks(q, cos, sin)
            q = _lib.kernel_ready(q)
            out = torch.empty_like(q)
            kring = self.cache_mem_k[:B, :n].flatten(1, 2).transpose(1, 2)    # (B, nh, n*block, hs) views, no copy
            vring = self.cache_mem_v[:B, :n].flatten(1, 2).transpose(1, 2)
            rc = _lib.lib().lmk_ring_gather_attend(
                _lib.tensor4(q), _lib.tensor4(kring), _lib.tensor4(vring), slots.data_ptr(), cos.data_ptr(),
                sin.data_ptr(), cos.stride(0), cos.shape[0], _lib.tensor4(o_loc), L_loc.data_ptr(), M_loc.data_ptr(),
                stat_stride, _lib.tensor4(out), B, nh, T, n, hs, float(sm_scale), block, self.cache_topk,
                self.oldest_slot, SELECTION_METHODS[self.cache_selection_method], _lib.DTYPE_CODES[q.dtype],
                _lib.current_stream(q.device))
        _lib.check(rc)
        return out, slots
