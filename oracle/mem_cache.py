"""Ring cache of landmark blocks: storage bookkeeping and block selection.  TEST ORACLE.

Restates ``MemLMCacheStorage`` of ``lm_benchmark/models/caches/mem_cache.py``: the ring-buffer
bookkeeping of ``store_in_cache`` (``:111-158``), the selection half of ``retrieve_for_query``
(``:50-85``) -- landmark positions, scores, softmax, the three selection methods, top-k and the
order-restoring sort -- the gather half (``:86-109``: picked blocks' keys rotated at ``k_indices``, their
scores, values and ``is_mem`` prefix, the tokens behind the last complete block appended) and the attention
``CausalSelfAttention.forward`` computes over that prefix and the current chunk
(``lm_benchmark/models/landmark.py:181-236``).  Nothing here is used by the library; the tests compare the
HIP selection with it index for index and the HIP attention with it to 2e-2.

What the reference leaves to the libraries is fixed the same way as for the llama-flavour cache
(``oracle/retrieval.py``): scores under the sequential-accumulation score contract, the softmax by
``softmax_contract`` in fp32 (under the benchmark's autocast the score product is a 16-bit matmul and
``softmax`` returns fp32, ``optim/base.py:49-50``), ties at the k-th place by (probability descending,
slot ascending).  Positions use the kernels' half-split tables; the benchmark's interleaved pairs
(``models/positional_encoders/rotary_utils.py:17-31``) are the same rotation with the even head dims
moved in front of the odd ones, which leaves every q.k unchanged (checked in
``tests/test_oracle_mem_cache.py`` against a restatement of the interleaved form).

Pinned in ``tests/test_oracle_mem_cache.py``: the ring against a plain Python list of blocks that is
appended to and truncated (contents, age order, slot of the oldest block, for chunks that wrap, fill
exactly, and exceed the capacity); slot ages and landmark positions on hand-worked cases; the
where/sort/where sequence against a brute-force sort by age; the selection of a ring against the
already pinned flat-cache selection (``oracle/retrieval.py``) applied to the same blocks laid out oldest
first; ``max_over_heads`` / ``max_over_tokens`` against literal loops; ``torch.topk`` on rows without a
boundary tie; ``retrieve_for_query`` / ``attention_with_cache`` in float64 against the closed form
(``oracle/s1.py``) on [picked blocks rotated at their positions ; tail ; chunk] and against the flat-cache
step of ``oracle/retrieval.py`` on the same blocks laid out oldest first (rotary is relative, so the two
position conventions agree when ``start_index`` is what ``MemLMCache.forward`` hands out, ``mem_cache.py:188``).
"""
from __future__ import annotations

import math

import torch

from .retrieval import sequential_dot_fp32, softmax_contract
from .rotary import apply_rotary

METHODS = ("per_token_and_head", "max_over_heads", "max_over_tokens")


class RingStore:
    """Buffers and counters of ``MemLMCacheStorage`` (``mem_cache.py:23-39``), CPU tensors.

    ``cache_k/v``: (B, capacity, block, nh, hs); ``pending_*``: the tokens behind the last complete
    block (``last_incomplete_*``).  ``cache_size`` keeps the reference's quirk of counting blocks that
    were dropped or overwritten, so the number of filled slots is ``min(cache_size, capacity)``."""

    def __init__(self, batch: int, capacity: int, block: int, heads: int, head_dim: int, dtype=torch.float32):
        self.capacity, self.block = capacity, block
        self.cache_k = torch.zeros(batch, capacity, block, heads, head_dim, dtype=dtype)
        self.cache_v = torch.zeros_like(self.cache_k)
        self.pending_k = torch.zeros(batch, heads, 0, head_dim, dtype=dtype)
        self.pending_v = torch.zeros_like(self.pending_k)
        self.pending_is_mem = torch.zeros(batch, 0, dtype=torch.bool)
        self.cache_iter = 0
        self.cache_size = 0

    @property
    def filled(self) -> int:
        return min(self.cache_size, self.capacity)          # what ``[:, :self.cache_size]`` keeps (``:51``)

    @property
    def last_incomplete_len(self) -> int:
        return self.pending_k.shape[2]

    def store(self, keys, values, is_mem) -> None:
        """``store_in_cache`` (``:111-158``): keys, values (B, nh, T, hs), is_mem (B, T)."""
        k = torch.cat((self.pending_k, keys), dim=2)                                  # :114-116
        v = torch.cat((self.pending_v, values), dim=2)
        im = torch.cat((self.pending_is_mem, is_mem), dim=1)
        B, nh, T, hs = k.shape
        bs, cap = self.block, self.capacity
        rest = T % bs                                                                 # :119-128
        full = T - rest
        self.pending_k, self.pending_v, self.pending_is_mem = k[:, :, full:], v[:, :, full:], im[:, full:]
        blocks_mem = im[:, :full].reshape(B, -1, bs)                                  # :131-134
        assert blocks_mem[..., -1].all() and not blocks_mem[..., :-1].any()
        n_new = full // bs
        kb = k[:, :, :full].transpose(1, 2).reshape(B, n_new, bs, nh, hs)             # :136-137
        vb = v[:, :, :full].transpose(1, 2).reshape(B, n_new, bs, nh, hs)
        kept = min(n_new, cap)                                                        # :138-143: only the newest fit
        dropped = n_new - kept
        kb, vb = kb[:, dropped:], vb[:, dropped:]
        self.cache_iter = (self.cache_iter + dropped) % cap
        self.cache_size += dropped
        if self.cache_iter + kept >= cap:                                             # :146-152: the write wraps
            head = cap - self.cache_iter
            nxt = self.cache_iter + kept - cap
            self.cache_k[:, self.cache_iter:] = kb[:, :head]
            self.cache_v[:, self.cache_iter:] = vb[:, :head]
            self.cache_k[:, :nxt] = kb[:, head:]
            self.cache_v[:, :nxt] = vb[:, head:]
        else:                                                                         # :153-156
            nxt = self.cache_iter + kept
            self.cache_k[:, self.cache_iter:nxt] = kb
            self.cache_v[:, self.cache_iter:nxt] = vb
        self.cache_iter = nxt                                                         # :158-159
        self.cache_size += kept


def slot_ages(n: int, cache_iter: int):
    """Age rank of every filled slot, 0 = oldest (``mem_indices`` of ``mem_cache.py:52-55``)."""
    return torch.cat((torch.arange(n - cache_iter, n), torch.arange(0, n - cache_iter)))


def landmark_slots(n: int, cache_iter: int, top_k: int):
    """Position slot of every filled block (``:57``): the ``top_k`` newest get 1..top_k, the rest 0."""
    age = slot_ages(n, cache_iter)
    return torch.where(age >= n - top_k, age - (n - top_k) + 1, 0)


def landmark_token_positions(n: int, cache_iter: int, top_k: int, block: int):
    """``mem_token_indices`` (``:58``)."""
    return landmark_slots(n, cache_iter, top_k) * block + block - 1


def ring_scores(q, cache_k, n: int, cache_iter: int, top_k: int, cos, sin):
    """(B, nh, T, n) scores in q.dtype (``:51,59-60``) under the score contract.
    q: (B, nh, T, hs) rotated; cache_k: (B, capacity, block, nh, hs)."""
    block, hs = cache_k.shape[2], cache_k.shape[-1]
    lk = cache_k[:, :n, -1].transpose(1, 2).to(q.dtype)                               # (B, nh, n, hs)
    lk = apply_rotary(lk, cos, sin, landmark_token_positions(n, cache_iter, top_k, block))
    dot = sequential_dot_fp32(q, lk)
    return (dot.to(q.dtype).float() / torch.tensor(math.sqrt(hs), dtype=torch.float32)).to(q.dtype)


def block_probabilities(scores, method: str):
    """fp32 (B, nh, T, n): softmax over the blocks, reduced as ``cache_selection_method`` says (``:61-70``)."""
    B, nh, T, n = scores.shape
    prob = softmax_contract(scores, torch.float32)
    if method == "max_over_heads":
        return prob.amax(dim=1, keepdim=True).expand(B, nh, T, n)
    if method == "max_over_tokens":
        return prob.amax(dim=2, keepdim=True).expand(B, nh, T, n)
    if method == "per_token_and_head":
        return prob
    raise NotImplementedError(method)


def restore_order(picked, n: int, cache_iter: int):
    """The order-restoring sort of ``:73-84`` applied to slot numbers (…, top_k): to age, sort, back to slots."""
    if picked.shape[-1] == 1:
        return picked
    age = torch.where(picked < cache_iter, (n - cache_iter) + picked, picked - cache_iter)
    age = age.sort(dim=-1).values
    return torch.where(age >= n - cache_iter, age - (n - cache_iter), age + cache_iter)


def select_blocks(scores, cache_iter: int, top_k: int, method: str):
    """Slots (B, nh, T, top_k) int64, oldest block first; ties by (probability descending, slot ascending)."""
    n = scores.shape[-1]
    # per_token_and_head ranks by the score itself: softmax is monotone, so this is the probability order wherever
    # two probabilities differ, and it also orders scores whose exponentials collapse to one fp32 value (underflow),
    # where torch.topk on the probabilities (``:72``) leaves the choice open
    prob = scores.float() if method == "per_token_and_head" else block_probabilities(scores, method)
    order = torch.sort(prob, dim=-1, descending=True, stable=True).indices[..., :top_k]
    return restore_order(order, n, cache_iter)


def boundary_tie_rows(scores, top_k: int, method: str):
    """Bool (B, nh, T): rows whose k-th and (k+1)-th best probabilities are equal."""
    prob = torch.sort(block_probabilities(scores, method), dim=-1, descending=True).values
    if prob.shape[-1] <= top_k:
        return torch.zeros(prob.shape[:-1], dtype=torch.bool)
    return prob[..., top_k - 1] == prob[..., top_k]


def gathered_key_positions(slots, n: int, cache_iter: int, top_k: int, block: int):
    """``k_indices`` (``:95-97``): positions at which the gathered keys are rotated, (…, top_k * block).
    The j-th picked block sits at tokens j*block .., one block further when it is one of the newest."""
    chosen = landmark_slots(n, cache_iter, top_k)[slots]                               # position slot of each pick
    base = torch.arange(top_k * block).view(top_k, block)
    return (((chosen > 0) * block).unsqueeze(-1) + base).flatten(-2)


# ------------------------------------------------------------ gather + attend
def gather_ring_blocks(cache, slots):
    """``take_along_dim`` of ``mem_cache.py:87-92``: cache (B, n, block, nh, hs), slots (B, nh, T, k) ->
    (B, nh, T, k * block, hs), the picked blocks of every (head, query) in the order of ``slots``."""
    B, n, block, nh, hs = cache.shape
    per_head = cache.permute(0, 3, 1, 2, 4)                                           # (B, nh, n, block, hs)
    T, k = slots.shape[2], slots.shape[3]
    wide = per_head[:, :, None].expand(B, nh, T, n, block, hs)
    sel = slots[..., None, None].expand(B, nh, T, k, block, hs)
    return torch.take_along_dim(wide, sel, dim=3).flatten(3, 4)


def expand_slots(slots, method: str, B: int, nh: int, T: int):
    """Slots in the shape a selection method returns them -> (B, nh, T, k)."""
    k = slots.shape[-1]
    if method == "max_over_heads":
        return slots.reshape(B, 1, T, k).expand(B, nh, T, k)
    if method == "max_over_tokens":
        return slots.reshape(B, nh, 1, k).expand(B, nh, T, k)
    return slots.reshape(B, nh, T, k)


def retrieve_for_query(store: RingStore, q, cos, sin, top_k: int, method: str, start_index: int, slots=None):
    """``MemLMCacheStorage.retrieve_for_query`` (``mem_cache.py:41-109``).

    q: (B, nh, T, hs) already rotated at ``start_index ..``.  Returns ``(att_prefix (B, nh, T, P), v_prefix
    (B, nh, T, P, hs), is_mem_prefix (B, P), slots)`` with ``P = top_k * block + last_incomplete_len``; without a
    filled slot or with ``top_k == 0`` only the tokens behind the last complete block remain (``:48-49``).
    Products run in the dtype of ``q`` (fp32 / fp64 for the closed-form comparisons, 16-bit for the kernels')."""
    B, nh, T, hs = q.shape
    block, tail = store.block, store.last_incomplete_len
    inv = 1.0 / math.sqrt(hs)
    tail_k = apply_rotary(store.pending_k.to(q.dtype), cos, sin, torch.arange(start_index - tail, start_index))   # :43
    att_tail = (q @ tail_k.transpose(-2, -1)) * inv                                   # :44
    v_tail = store.pending_v.to(q.dtype)[:, :, None].expand(B, nh, T, tail, hs)       # :45
    mem_tail = store.pending_is_mem                                                   # :46
    n = store.filled
    if n == 0 or top_k == 0:
        return att_tail, v_tail, mem_tail, None
    if slots is None:
        scores = ring_scores(q, store.cache_k, n, store.cache_iter, top_k, cos, sin)
        slots = select_blocks(scores, store.cache_iter, top_k, method)
    slots = expand_slots(slots, "per_token_and_head", B, nh, T)
    mem_k = gather_ring_blocks(store.cache_k[:, :n].to(q.dtype), slots)               # :87-90
    mem_v = gather_ring_blocks(store.cache_v[:, :n].to(q.dtype), slots)               # :91-92
    k_indices = gathered_key_positions(slots, n, store.cache_iter, top_k, block)      # :94-96
    mem_k = apply_rotary(mem_k, cos, sin, k_indices)                                  # :100
    att_k = (q.unsqueeze(3) @ mem_k.transpose(-2, -1)).squeeze(3) * inv               # :101
    is_mem = torch.zeros(top_k, block, dtype=torch.bool)
    is_mem[:, -1] = True                                                              # :98
    is_mem = is_mem.flatten().expand(B, top_k * block)
    return (torch.cat((att_k, att_tail), dim=-1), torch.cat((mem_v, v_tail), dim=-2),
            torch.cat((is_mem, mem_tail), dim=-1), slots)


def attention_with_cache(store: RingStore, q, k, v, is_mem, cos, sin, top_k: int, method: str, start_index: int,
                         n_buckets: int, slots=None):
    """``CausalSelfAttention.forward`` between the projections and ``c_proj`` with a cache
    (``lm_benchmark/models/landmark.py:181-236``).  q, k: (B, nh, T, hs) rotated at ``start_index ..``; v: (B, nh, T,
    hs); is_mem: (B, T).  Returns ``(y (B, nh, T, hs), slots)``."""
    from .highlevel import grouped_softmax, masks_from_is_mem
    B, nh, T, hs = q.shape
    att_prefix, v_prefix, mem_prefix, slots = retrieve_for_query(store, q, cos, sin, top_k, method, start_index, slots)
    att = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(hs))                           # :195
    causal_masked = ~torch.tril(torch.ones(T, T, dtype=torch.bool))[None, None].expand(B, nh, T, T)
    att = att.masked_fill(causal_masked, float("-inf"))                               # :197
    P = att_prefix.shape[-1]
    att = torch.cat((att_prefix, att), dim=-1)                                        # :202
    mem_all = torch.cat((mem_prefix, is_mem), dim=-1)                                 # :204
    attn_mask = torch.cat((torch.zeros(B, nh, T, P, dtype=torch.bool), causal_masked), dim=-1)   # :207
    masked, im, ls = masks_from_is_mem(mem_all[:, None, None, :], attn_mask)          # :214-222
    att = att.masked_fill(masked, float("-inf"))                                      # :223
    w = grouped_softmax(att, im, ls, n_buckets, attn_mask=masked, guard_empty=True)   # :226-231
    w_prefix, w_loc = w[..., :P], w[..., P:]                                          # :234
    y = w_loc.to(v.dtype) @ v + (w_prefix.to(v.dtype).unsqueeze(3) @ v_prefix).squeeze(3)   # :235-240
    return y, slots
