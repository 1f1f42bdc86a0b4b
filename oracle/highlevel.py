"""Restatement of the reference's high-level (mask + bucketed softmax) path.  TEST ORACLE.

The reference evaluates landmark attention without a fused kernel by assigning
every key of a score row to a bucket and running one softmax per bucket with
scatter/gather primitives, then multiplying the within-block probabilities by
the probability of the block's landmark:

* llama flavour         ``llama/llama_mem.py:168-243``  (fixed 64 buckets, ``finfo.min``
                        masking, no guards for empty buckets)
* lm_benchmark flavour  ``lm_benchmark/models/landmark.py:37-119`` (``-inf`` masking with
                        guards ``:48,54``; bucket count is a parameter)
* mask construction     ``lm_benchmark/models/landmark.py:216-224`` (from ``is_mem`` and the
                        causal mask), ``llama/llama_mem.py:807-815`` (same, additive mask),
                        ``llama/ltriton/test_flash_landmark_attention.py:107-123`` (closed form
                        for the fixed-stride case)

Bucket rule (``llama_mem.py:229-233``): keys of the row's own block ("last
section") and every visible landmark share the final bucket ``n_buckets - 1``;
a non-landmark key of an earlier block goes to bucket ``#landmarks before it``.
After the per-bucket softmax, an earlier normal key is scaled by the
probability of the landmark that closes its block (``:238-240``).

This file follows that algorithm with its own code; it exists so that the
closed form in ``oracle/s1.py`` can be checked against an independently written
statement of the same mathematics (``tests/test_oracle_highlevel.py``).
"""
from __future__ import annotations

import math

import torch


def _bucketed_softmax(x, bucket, n_buckets: int, guard_empty: bool):
    """Softmax of ``x`` along the last dim, separately inside every bucket.

    Mirrors ``LandmarkGroupedSoftmaxFunction.forward`` (``llama_mem.py:172-196``;
    ``landmark.py:41-63``): per-bucket amax by scatter-reduce, exp of the shifted
    scores, per-bucket sums by scatter-add, divide.  Differentiable by autograd
    (the reference's hand-written backward ``llama_mem.py:198-220`` is the
    derivative of exactly this expression with the max treated as a constant).
    """
    shape = x.shape[:-1] + (n_buckets,)
    top = torch.zeros(shape, dtype=x.dtype, device=x.device)
    top = top.scatter_reduce(-1, bucket, x.detach(), reduce="amax", include_self=False)
    shift = top.gather(-1, bucket)
    if guard_empty:                                     # landmark.py:48
        shift = torch.where(torch.isinf(shift), torch.zeros_like(shift), shift)
    # llama_mem.py:180 upcasts the shifted scores to fp32 (fp64 inputs stay fp64 here)
    e = torch.exp((x - shift).to(torch.promote_types(x.dtype, torch.float32)))
    tot = torch.zeros(shape, dtype=e.dtype, device=x.device).scatter_add(-1, bucket, e)
    z = tot.gather(-1, bucket)
    if guard_empty:                                     # landmark.py:54
        return torch.where(z < 0.5, torch.zeros_like(e), e / z)
    return e / z


def grouped_softmax(x, is_mem, last_section, n_buckets: int = 64, attn_mask=None, guard_empty: bool = False,
                    group_keep=None):
    """Landmark grouped softmax over the last dim of ``x``.

    ``group_keep`` (broadcastable to ``x.shape[:-1] + (n_buckets,)``), optional: the outcome of the group dropout
    of ``landmark.py:110-113`` written as a factor per bucket -- ``dropout(group_prob, p)`` multiplies each
    landmark probability by 0 or 1 / (1 - p) before it scales its block; the last bucket is overwritten
    afterwards (``:112``), so its entry is not used.

    ``is_mem``        bool, True at visible landmark keys
    ``last_section``  bool, True at visible keys of the query's own block
    ``attn_mask``     bool, True at masked keys (lm_benchmark flavour only; it
                      joins the final bucket, ``landmark.py:93``)
    ``n_buckets``     64 in the llama flavour (``llama_mem.py:228``)
    """
    final = last_section if attn_mask is None else (last_section | attn_mask)
    seen = torch.cumsum(is_mem.to(torch.int64), dim=-1)          # landmarks up to and including j
    last = n_buckets - 1
    bucket = torch.where(final | is_mem, torch.full_like(seen, last), seen)
    bucket = bucket.expand(x.shape)
    probs = _bucketed_softmax(x, bucket, n_buckets, guard_empty)

    # probability of each landmark, filed under the index of the block it closes
    slot = torch.where(is_mem, seen - 1, torch.full_like(seen, last)).expand(x.shape)
    by_block = torch.zeros(x.shape[:-1] + (n_buckets,), dtype=probs.dtype, device=x.device)
    by_block = by_block.scatter(-1, slot, probs)
    if group_keep is not None:                                   # landmark.py:110-111
        by_block = by_block * group_keep
    if attn_mask is not None:                                    # landmark.py:115
        by_block = by_block.clone()
        by_block[..., last] = (probs * last_section).sum(-1)
    outer = torch.where(final | is_mem, last_section.to(probs.dtype).expand(x.shape), by_block.gather(-1, bucket))
    return probs * outer


def masks_from_is_mem(is_mem_row, causal_masked):
    """Masks of the lm_benchmark path (``landmark.py:216-224``).

    is_mem_row: (..., 1 or T, Lk) bool landmarks; causal_masked: (..., T, Lk)
    bool, True where the causal mask hides the key.  Returns
    ``(masked, is_mem_visible, last_section)``.
    """
    im = is_mem_row.expand(causal_masked.shape)
    before = torch.cumsum(im.to(torch.int64), -1) - im.to(torch.int64)   # landmarks strictly before j
    ids = torch.where(causal_masked, torch.zeros_like(before), before)
    last_section = ids == ids.amax(-1, keepdim=True)
    masked = causal_masked | (im & last_section)         # own block's landmark is hidden
    return masked, im & ~masked, last_section & ~masked


def attention_lm_benchmark(q, k, v, is_mem, n_buckets: int):
    """Forward of ``CausalSelfAttention`` without cache/positional terms
    (``lm_benchmark/models/landmark.py:196-236``).  q, k, v: (B, H, T, D),
    is_mem: (B, T) bool."""
    T, d = q.shape[-2], q.shape[-1]
    att = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(d))
    causal_masked = ~torch.tril(torch.ones(T, T, dtype=torch.bool, device=q.device))[None, None]
    att = att.masked_fill(causal_masked, float("-inf"))
    masked, im, ls = masks_from_is_mem(is_mem[:, None, None, :], causal_masked.expand(att.shape))
    att = att.masked_fill(masked, float("-inf"))
    w = grouped_softmax(att, im, ls, n_buckets, attn_mask=masked, guard_empty=True)
    return w @ v


def attention_fixed_stride(q, k, v, block: int, n_buckets: int | None = None, scale: float | None = None):
    """The comparison the reference's kernel test makes
    (``llama/ltriton/test_flash_landmark_attention.py:105-125``): landmarks at
    fixed stride, history allowed (``Lk >= Lq``), ``-inf`` masking, llama-flavour
    softmax, masked weights zeroed afterwards (``:123``)."""
    lq, d = q.shape[-2], q.shape[-1]
    lk = k.shape[-2]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    nb = -(-lk // block)
    if n_buckets is None:
        n_buckets = max(nb + 1, 2)
    att = (q @ k.transpose(-1, -2)) * scale
    j = torch.arange(lk, device=q.device)
    i = torch.arange(lk - lq, lk, device=q.device)
    causal = j[None, :] <= i[:, None]
    same = (j // block)[None, :] == (i // block)[:, None]
    is_mem = (j % block == block - 1)[None, :]
    visible = causal & ~(same & is_mem)
    ls = (same & visible)[None, None]
    im = (is_mem & visible)[None, None]
    att = att.masked_fill(~visible[None, None], float("-inf"))
    w = grouped_softmax(att, im.expand(att.shape), ls.expand(att.shape), n_buckets)
    w = w.masked_fill(~visible[None, None], 0.0)         # removes the NaNs of empty buckets
    return w.to(v.dtype) @ v
