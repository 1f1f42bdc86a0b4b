"""Growing KV cache for the mem-cache inference path.

The reference keeps ``past_key_value = (K_without_rotary, V)`` and appends every new chunk with
``torch.cat`` (``llama/llama_mem.py:424-430``), which copies the whole cache once per layer and
step.  ``LandmarkKVCache`` holds the same two tensors in buffers with spare room along the
sequence axis, so an append writes only the new rows; ``past_key_value`` hands out
``(B, nh, S, hd)`` views of the filled part, which the retrieval kernels read in place through
their strides.  Blocks stay contiguous per (batch, head): block ``m`` of a head is the
``block * hd`` elements at row ``m * block``, the landmark key its last row.
"""
from __future__ import annotations

import torch

from . import _lib
from .retrieval import attend_shared, retrieve_and_attend, retrieve_topk_from_landmarks


class LandmarkKVCache:
    """``(K_without_rotary, V)`` of one attention layer with amortised O(new rows) appends."""

    def __init__(self, batch: int, heads: int, head_dim: int, dtype, device, capacity: int = 4096):
        self._k = torch.empty((batch, heads, capacity, head_dim), dtype=dtype, device=device)
        self._v = torch.empty_like(self._k)
        self.length = 0
        self._ws = None                     # retrieval workspace, kept between steps
        self._ws_key = None                 # what the rotated landmark keys in it were made for

    @property
    def capacity(self) -> int:
        return self._k.shape[2]

    @property
    def past_key_value(self):
        """The reference's cache tuple (``llama_mem.py:430``): views, no copy."""
        return self._k[:, :, : self.length], self._v[:, :, : self.length]

    def _reserve(self, rows: int) -> None:
        if rows <= self.capacity:
            return
        cap = max(rows, 2 * self.capacity)
        for name in ("_k", "_v"):
            old = getattr(self, name)
            new = torch.empty(old.shape[:2] + (cap, old.shape[3]), dtype=old.dtype, device=old.device)
            new[:, :, : self.length] = old[:, :, : self.length]
            setattr(self, name, new)

    def append(self, key_states_before_pos, value_states) -> None:
        """``torch.cat([past, new], dim=2)`` of ``llama_mem.py:424-425`` without re-copying ``past``."""
        t = key_states_before_pos.shape[2]
        assert key_states_before_pos.shape == value_states.shape == self._k.shape[:2] + (t, self._k.shape[3])
        self._reserve(self.length + t)
        self._k[:, :, self.length : self.length + t] = key_states_before_pos
        self._v[:, :, self.length : self.length + t] = value_states
        self.length += t

    def step(self, query_states, key_states, key_states_before_pos, value_states, cos, sin, block: int, top_k: int,
             sm_scale=None, aggregate=None):
        """Attention of a new chunk against the cache, then the append (``llama_mem.py:318-430,447-477``):
        ``query_states`` and ``key_states`` rotated at the chunk's positions, ``key_states_before_pos`` the
        same keys without rotary.  Needs at least one complete cached block; returns ``(out, idx)``.

        The landmark keys are rotated at positions that move only when a cached block completes
        (``:359-365``), and appends never touch complete blocks, so between two landmarks the rotated keys of
        the previous step are reused (per-token selection; same tables, block and top_k)."""
        B, H, T, D = query_states.shape
        nbytes = _lib.lib().lmk_retrieve_workspace_bytes(B, H, T, self.length, D, int(block))
        if self._ws is None or self._ws.numel() < nbytes or self._ws.device != query_states.device:
            self._ws = torch.empty(max(nbytes, 2 * (self._ws.numel() if self._ws is not None else 0)),
                                   device=query_states.device, dtype=torch.uint8)
            self._ws_key = None
        key = (self.length // block, int(block), int(top_k), cos.data_ptr(), sin.data_ptr(), self._k.data_ptr())
        reuse = aggregate is None and key == self._ws_key
        out, idx = retrieve_and_attend(query_states, self.past_key_value, key_states, value_states, cos, sin,
                                       block, top_k, sm_scale, aggregate, workspace=self._ws,
                                       reuse_landmark_keys=reuse)
        self._ws_key = key if aggregate is None else None
        self.append(key_states_before_pos, value_states)
        return out, idx


class OffloadedLandmarkCache:
    """The cache of the reference's ``offload_cache_to_cpu`` branch (``llama/llama_mem.py:326-328,344-356,
    427-428``): keys (without rotary) and values live in pinned host memory, only the landmark key of every
    complete block stays on the GPU (``past_key_value[2]``), and every head retrieves one set of blocks per
    step (``aggregate = "max_over_tokens"``, ``:369-372``).

    The reference gathers the selected blocks on the CPU and copies them over (``:393-398``).  Here the
    host buffers are mapped into the GPU's address space (pinned allocations are), so the kernel that builds
    the key/value window reads the ``k`` selected blocks of each head -- and the few tokens of an incomplete
    last block -- straight out of host memory: no index round trip to the host, no staging copy, and only
    ``k * block`` rows per head cross the bus.  Appends are device-to-host copies of the new rows on the
    caller's stream."""

    def __init__(self, batch: int, heads: int, head_dim: int, block: int, dtype, device, capacity: int = 4096):
        self.block = int(block)
        self._k = torch.empty((batch, heads, capacity, head_dim), dtype=dtype, pin_memory=True)
        self._v = torch.empty((batch, heads, capacity, head_dim), dtype=dtype, pin_memory=True)
        self._lm = torch.empty((batch, heads, max(1, capacity // self.block), head_dim), dtype=dtype, device=device)
        self.length = 0
        self._ws = None

    @property
    def n_blocks(self) -> int:
        return self.length // self.block

    @property
    def landmark_keys(self):
        """``past_key_value[2]`` (``:344-347``): the un-rotated landmark keys of the complete blocks, on the GPU."""
        return self._lm[:, :, : self.n_blocks]

    @property
    def host_key_value(self):
        """Views of the filled part of the pinned host buffers, (B, nh, S, hd) each.  ``append`` fills them with
        asynchronous device->host copies on the caller's stream: synchronise that stream before reading the views
        on the host (kernels on the same stream see the rows in order)."""
        return self._k[:, :, : self.length], self._v[:, :, : self.length]

    def _reserve(self, rows: int) -> None:
        if rows <= self._k.shape[2]:
            return
        cap = max(rows, 2 * self._k.shape[2])
        torch.cuda.current_stream(self._lm.device).synchronize()     # copies into the old buffers have landed
        for name in ("_k", "_v"):
            old = getattr(self, name)
            new = torch.empty(old.shape[:2] + (cap, old.shape[3]), dtype=old.dtype, pin_memory=True)
            new[:, :, : self.length] = old[:, :, : self.length]
            setattr(self, name, new)
        lm = torch.empty(self._lm.shape[:2] + (cap // self.block, self._lm.shape[3]), dtype=self._lm.dtype,
                         device=self._lm.device)
        lm[:, :, : self.n_blocks] = self._lm[:, :, : self.n_blocks]
        self._lm = lm

    def append(self, key_states_before_pos, value_states) -> None:
        """``:424-428``: the new rows go to the host buffers, landmark keys of blocks they complete to the GPU array."""
        t = key_states_before_pos.shape[2]
        self._reserve(self.length + t)
        self._k[:, :, self.length: self.length + t].copy_(key_states_before_pos, non_blocking=True)
        self._v[:, :, self.length: self.length + t].copy_(value_states, non_blocking=True)
        first = (-(self.length + 1)) % self.block                    # offset of the first new landmark token, if any
        if first < t:
            n_new = (t - first + self.block - 1) // self.block
            self._lm[:, :, self.n_blocks: self.n_blocks + n_new] = key_states_before_pos[:, :, first::self.block]
        self.length += t

    def step(self, query_states, key_states, key_states_before_pos, value_states, cos, sin, top_k: int, sm_scale=None):
        """Attention of a new chunk against the offloaded cache, then the append; returns ``(out, idx)`` with
        ``idx (B, nh, 1, k)``.  Needs at least one complete cached block."""
        assert self.n_blocks >= 1, "no complete cached block yet"
        B, nh, T, hd = query_states.shape
        nbytes = _lib.lib().lmk_retrieve_workspace_bytes(B, nh, T, self.n_blocks * self.block, hd, self.block)
        if self._ws is None or self._ws.numel() < nbytes or self._ws.device != query_states.device:
            self._ws = torch.empty(max(nbytes, 2 * (self._ws.numel() if self._ws is not None else 0)),
                                   device=query_states.device, dtype=torch.uint8)     # grown on demand, kept between steps
        idx = retrieve_topk_from_landmarks(query_states, self.landmark_keys, cos, sin, self.block, top_k, self._ws)
        k_host, v_host = self.host_key_value
        out = attend_shared(query_states, k_host, v_host, idx, key_states, value_states, cos, sin, self.block, top_k,
                            sm_scale)
        self.append(key_states_before_pos, value_states)
        return out, idx
