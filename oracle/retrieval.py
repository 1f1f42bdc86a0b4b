"""Mem-cache retrieval: landmark scoring, top-k block selection, gather, attend.  TEST ORACLE.

Restates the per-head, per-token branch (``aggregate is None``) of
``LlamaAttention.forward`` in ``llama/llama_mem.py:318-430`` and the attend step
``:447-477`` with the mask preparation of ``LlamaModel.forward`` ``:807-815``.

Symbols: ``bs = mem_freq + 1`` (block), ``S`` cached tokens, ``T`` new tokens,
``num_mems = S // bs`` complete cached blocks, ``k = min(cache_top_k, num_mems)``.
When the cache ends in an incomplete block (``S % bs`` tokens, ``:321-324``) those tokens
are not retrieved from: they are rotated at their own positions and put in front of the
new chunk (``:329-342``), visible to every query, in no landmark group.
The cache holds keys WITHOUT rotary (``:424-425``); queries and local keys come
in already rotated (``:298``).

Score contract (``:367``).  The reference computes ``matmul(q, mem_key^T) /
sqrt(hd)`` in the model dtype: an fp32-accumulated product rounded to the model
dtype, then a division rounded again.  The reference leaves the accumulation
order of that product to the BLAS library, so it has to be fixed for indices to
be reproducible bit for bit.  This build fixes it to the plain sequential order:
``acc = fma(q[d], k[d], acc)`` in fp32 for ``d = 0 .. hd-1`` (a product of two
16-bit floats is exact in fp32, so every step is one correctly rounded fp32
addition, which numpy reproduces exactly), then ``acc -> model dtype``, then fp32
division by ``float32(sqrt(hd))`` ``-> model dtype``.  Selection contract
(``:384``): the ``k`` best under the total order (score descending, block index
ascending), returned in ascending index order.  ``torch.topk`` breaks ties in an implementation-defined
way; on rows without a tie at the k-th place both agree, which
``tests/test_oracle_retrieval.py`` checks, together with a brute-force loop,
the integer position formulas on hand-worked cases, and agreement of the
bf16-faithful attend with the fp32 closed form of ``oracle/s1.py``.

One selection per head (``aggregate == "max_over_tokens"``, ``:373-377``, the branch the
reference takes when the cache is offloaded to the CPU): the scores of every query go
through an fp32 softmax over the cached blocks, are rounded to the model dtype and reduced
with ``amax`` over the queries; the top-k of that per-head vector is shared by all queries,
the selected blocks become ordinary history blocks in front of the local window
(``:400-406``) and the attention is the fused forward's (``:441-446``).  ``torch.softmax``
leaves the exponential's last bit and the order of the sum to the library, so both are fixed
here (``exp2_contract``, ``softmax_contract``) with operations numpy and the GPU round
identically: no fused multiply-add, a polynomial evaluated by Horner's rule with separate
products and sums, a per-lane sequential sum followed by a halving tree.  Pinned in
``tests/test_oracle_retrieval.py`` against ``numpy.exp2`` / ``torch.softmax`` (to a few ulp),
against a literal Python loop, and against ``torch.topk`` on heads without a boundary tie.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from .highlevel import grouped_softmax
from .rotary import apply_rotary
from .s1 import s1_attention


# ------------------------------------------------------------------ positions
def retrieval_geometry(S: int, block: int, top_k: int):
    """Integer bookkeeping of ``llama_mem.py:321-324,358-365``.

    Returns dict with ``full_len, incomplete_len, num_mems, k, prefix_len`` and
    ``mem_pos`` (num_mems,) — the position at which each cached landmark key is
    rotated for SCORING: every block but the newest ``k`` sits in slot 0, the
    newest ``k`` in slots 1..k.
    """
    incomplete_len = S % block
    full_len = S - incomplete_len
    num_mems = full_len // block
    k = min(top_k, num_mems)
    prefix_len = full_len - (k + 1) * block
    slot = torch.cat((torch.zeros(max(0, num_mems - k), dtype=torch.long), torch.arange(1, k + 1, dtype=torch.long)))
    mem_pos = slot * block + (block - 1) + prefix_len
    return dict(full_len=full_len, incomplete_len=incomplete_len, num_mems=num_mems, k=k,
                prefix_len=prefix_len, mem_pos=mem_pos)


def gather_positions(idx, num_mems: int, k: int, block: int, prefix_len: int):
    """Positions at which the gathered keys are rotated (``llama_mem.py:386-388``).

    idx: (..., k) ascending block indices.  Slot ``j`` (rank in the ascending
    list) token ``t``: ``j*bs + t + (bs if idx[j] >= num_mems-k else 0) + prefix_len``.
    Returns (..., k, bs) int64.
    """
    j = torch.arange(k, dtype=torch.long, device=idx.device)
    t = torch.arange(block, dtype=torch.long, device=idx.device)
    bump = torch.where(idx >= num_mems - k, block, 0)
    return (j * block + bump)[..., None] + t + prefix_len


# -------------------------------------------------------------------- scoring
def sequential_dot_fp32(q, keys):
    """(…, T, M) fp32: ``sum_d q[t,d]*keys[m,d]`` accumulated in fp32 in the order
    d = 0, 1, … with one rounding per step (the score contract above).  q: (…, T, hd),
    keys: (…, M, hd), both holding 16-bit float values."""
    qf = q.float().numpy()
    kf = keys.float().numpy()
    acc = np.zeros(qf.shape[:-1] + (kf.shape[-2],), dtype=np.float32)
    for d in range(qf.shape[-1]):
        prod = qf[..., :, None, d] * kf[..., None, :, d]          # exact in fp32
        acc = (acc + prod).astype(np.float32)
    return torch.from_numpy(acc)


def landmark_scores(q, k_cache, cos, sin, block: int, top_k: int):
    """Scores (B, nh, T, num_mems) in q.dtype under the score contract."""
    S, hd = k_cache.shape[-2], k_cache.shape[-1]
    g = retrieval_geometry(S, block, top_k)
    lk = k_cache[..., : g["full_len"], :].unflatten(-2, (g["num_mems"], block))[..., block - 1, :]
    lk = apply_rotary(lk, cos, sin, g["mem_pos"])                     # :366
    dot = sequential_dot_fp32(q, lk)
    sc = dot.to(q.dtype).float() / torch.tensor(math.sqrt(hd), dtype=torch.float32)
    return sc.to(q.dtype)


def select_topk(scores, k: int):
    """Ascending indices (…, k) int64 of the k best under (score desc, index asc)."""
    order = torch.sort(scores.float(), dim=-1, descending=True, stable=True).indices
    return order[..., :k].sort(dim=-1).values


def boundary_tie_rows(scores, k: int):
    """Bool (…): rows whose k-th and (k+1)-th best scores are equal."""
    top = torch.sort(scores.float(), dim=-1, descending=True).values
    if top.shape[-1] <= k:
        return torch.zeros(top.shape[:-1], dtype=torch.bool)
    return top[..., k - 1] == top[..., k]


# --------------------------------------------------- one selection per head
_LOG2E = np.float32(1.4426950408889634)
# Taylor coefficients of 2**f = exp(f ln 2) up to degree 6 (|f| <= 1/2: truncation < 1.3e-7)
_EXP2_COEF = [np.float32(c) for c in (1.0, 0.6931471805599453, 0.2402265069591007, 0.05550410866482158,
                                      0.009618129107628477, 0.0013333558146428443, 0.00015403530393381608)]


def exp2_contract(t):
    """``2**t`` for fp32 ``t <= 0`` with every rounding fixed: ``n = rint(t)`` (ties to even),
    ``f = t - n`` (exact), degree-6 Horner polynomial in ``f`` with one fp32 rounding after each
    product and each sum, scaled by ``2**n`` (exact).  ``t < -126`` gives 0, so no fp32
    subnormal is ever produced here."""
    t = np.asarray(t, dtype=np.float32)
    n = np.rint(t)
    f = (t - n).astype(np.float32)
    p = np.full_like(f, _EXP2_COEF[6])
    for c in _EXP2_COEF[5::-1]:
        p = (p * f).astype(np.float32)
        p = (p + c).astype(np.float32)
    out = np.ldexp(p, np.maximum(n, -126).astype(np.int32)).astype(np.float32)
    return np.where(t < np.float32(-126.0), np.float32(0.0), out)


def softmax_contract(scores, dtype):
    """Softmax over the last dim of fp32 ``scores`` (…, M), rounded to ``dtype`` (``:376``).

    ``e_m = exp2_contract((x_m - max) * log2(e))``; the sum runs the way one 64-lane wave adds
    it: lane ``l`` adds ``e_l, e_{l+64}, …`` in that order, then the 64 partial sums are folded
    by halves (32, 16, … 1); ``p_m = e_m / sum`` is one correctly rounded fp32 division."""
    x = scores.float().numpy()
    mx = x.max(axis=-1, keepdims=True)
    e = exp2_contract(((x - mx).astype(np.float32) * _LOG2E).astype(np.float32))
    M = e.shape[-1]
    pad = (-M) % 64
    ep = np.concatenate((e, np.zeros(e.shape[:-1] + (pad,), np.float32)), axis=-1)
    ep = ep.reshape(e.shape[:-1] + (-1, 64))
    part = np.zeros(e.shape[:-1] + (64,), np.float32)
    for r in range(ep.shape[-2]):
        part = (part + ep[..., r, :]).astype(np.float32)
    w = 32
    while w >= 1:
        part = (part[..., :w] + part[..., w:2 * w]).astype(np.float32)
        w //= 2
    prob = (e / part).astype(np.float32)
    return torch.from_numpy(prob).to(dtype)


def aggregate_max_over_tokens(scores):
    """(B, nh, 1, M) in the scores' dtype: softmax over blocks per query, then the largest
    probability any query gives a block (``llama_mem.py:376-377``)."""
    return softmax_contract(scores, scores.dtype).amax(dim=2, keepdim=True)


def shared_window(k_cache, v_cache, k_loc, v_loc, idx, cos, sin, block: int, top_k: int):
    """Keys and values every query of a head attends to in the ``max_over_tokens`` branch
    (``llama_mem.py:400-406``): the ``k`` selected blocks, keys rotated at their slot positions
    (``:386-388,403``), then the local window (tail of an incomplete cached block, new chunk).
    idx: (B, nh, 1, k).  Returns (B, nh, k*bs + inc + T, hd) each."""
    S = k_cache.shape[2]
    g = retrieval_geometry(S, block, top_k)
    k = g["k"]
    if g["incomplete_len"]:
        k_loc, v_loc = local_window(k_cache, v_cache, k_loc, v_loc, cos, sin, block)
    pos = gather_positions(idx, g["num_mems"], k, block, g["prefix_len"])           # (B,nh,1,k,bs)
    ksel = apply_rotary(gather_blocks(k_cache, idx, block), cos, sin, pos)[:, :, 0].flatten(2, 3)
    vsel = gather_blocks(v_cache, idx, block)[:, :, 0].flatten(2, 3)
    return torch.cat((ksel, k_loc), dim=2), torch.cat((vsel, v_loc), dim=2)


def retrieve_and_attend_shared(q, k_cache, v_cache, k_loc, v_loc, is_mem_loc, cos, sin, block: int, top_k: int,
                               idx=None, n_buckets: int = 64):
    """The ``max_over_tokens`` step in the model dtype through the reference's high-level attend
    (``llama_mem.py:447-477``).  Returns ``(out (B,nh,T,hd), idx (B,nh,1,k) int64)``."""
    B, nh, T, hd = q.shape
    S = k_cache.shape[2]
    g = retrieval_geometry(S, block, top_k)
    inc, k = g["incomplete_len"], g["k"]
    if inc:
        assert T + inc <= block                                                     # :330
    if idx is None:
        idx = select_topk(aggregate_max_over_tokens(landmark_scores(q, k_cache, cos, sin, block, top_k)), k)
    keys, values = shared_window(k_cache, v_cache, k_loc, v_loc, idx, cos, sin, block, top_k)
    add, im_loc, ls_loc = local_masks(is_mem_loc, T, q.dtype)
    n_front = k * block + inc
    add = torch.cat((torch.zeros(add.shape[0], 1, T, n_front, dtype=add.dtype), add), dim=-1)
    im_front = torch.zeros(n_front, dtype=torch.bool)
    im_front[block - 1 : k * block : block] = True                                   # :415
    ls_front = torch.zeros(n_front, dtype=torch.bool)
    ls_front[k * block :] = True                                                     # :335 (tail), :420 (selected)
    im = torch.cat((im_front.expand(im_loc.shape[0], 1, T, -1), im_loc), dim=-1).expand(B, nh, T, -1)
    ls = torch.cat((ls_front.expand(ls_loc.shape[0], 1, T, -1), ls_loc), dim=-1).expand(B, nh, T, -1)
    x = (q @ keys.transpose(2, 3)) / math.sqrt(hd) + add                            # :448,460
    x = torch.max(x, torch.tensor(torch.finfo(q.dtype).min, dtype=q.dtype))         # :461
    w = grouped_softmax(x, im, ls, n_buckets).to(q.dtype)                           # :469
    return w @ values, idx                                                          # :477


def retrieve_and_attend_shared_s1(q, k_cache, v_cache, k_loc, v_loc, cos, sin, block: int, top_k: int, idx):
    """Same step as the fp32 closed form: the selected blocks are history blocks of the fused
    forward (``fused_landmark_attention`` with ``n_history_blocks = k``, ``llama_mem.py:441-446``).
    Returns (B, nh, T, hd) fp32."""
    B, nh, T, hd = q.shape
    inc = k_cache.shape[2] % block
    keys, values = shared_window(k_cache, v_cache, k_loc, v_loc, idx, cos, sin, block, top_k)
    if inc:                       # the tail opens the current block; zero rows stand in for its queries
        q = torch.cat((torch.zeros(B, nh, inc, hd, dtype=q.dtype), q), dim=2)
    out = torch.empty(B, nh, T, hd)
    for b in range(B):
        for h in range(nh):
            out[b, h] = s1_attention(q[b, h].float(), keys[b, h].float(), values[b, h].float(), block)[inc:]
    return out


# --------------------------------------------------------------------- gather
def gather_blocks(cache, idx, block: int):
    """``take_along_dim`` of ``llama_mem.py:393-398``: (B, nh, T, k, bs, hd)."""
    B, nh, S, hd = cache.shape
    num_mems = S // block
    blocks = cache[:, :, : num_mems * block].unflatten(2, (num_mems, block))       # (B,nh,M,bs,hd)
    T, k = idx.shape[2], idx.shape[3]
    flat = blocks[:, :, None].expand(B, nh, T, num_mems, block, hd)
    sel = idx[..., None, None].expand(B, nh, T, k, block, hd)
    return torch.take_along_dim(flat, sel, dim=3)


def local_window(k_cache, v_cache, k_loc, v_loc, cos, sin, block: int):
    """Keys and values of the local window when the cache ends in an incomplete block
    (``llama_mem.py:337-340``): the tail's keys rotated at positions ``full_len ..`` in front of
    the new chunk's, the tail's values in front of the new chunk's."""
    S = k_cache.shape[2]
    inc = S % block
    full_len = S - inc
    pos = torch.arange(full_len, S, dtype=torch.long)
    k_tail = apply_rotary(k_cache[:, :, full_len:], cos, sin, pos)
    return torch.cat((k_tail, k_loc), dim=2), torch.cat((v_cache[:, :, full_len:], v_loc), dim=2)


# ---------------------------------------------------------------- local masks
def local_masks(is_mem_loc, T: int, dtype):
    """Mask preparation of ``LlamaModel.forward`` (``llama_mem.py:807-815``) for a
    chunk of ``T`` new tokens (only the last ``T`` mask columns matter on this path).

    Returns additive mask (B,1,T,T) in ``dtype`` (0 / finfo.min), visible
    landmark mask and last-section mask, both (B,1,T,T) bool.
    """
    low = torch.finfo(dtype).min
    i = torch.arange(T)
    add = torch.where(i[None, :] <= i[:, None], torch.zeros((), dtype=dtype), torch.full((), low, dtype=dtype))[None, None]
    add = add.expand(is_mem_loc.shape[0], 1, T, T).clone()
    im = is_mem_loc[:, None, None, :]
    ids = torch.where(add < -1, 0, torch.cumsum(im, -1) - im.int())
    last_section = ids.amax(-1, keepdim=True) == ids
    add = add.masked_fill(last_section & im, low)
    vis = add > -1
    return add, im & vis, last_section & vis


# --------------------------------------------------------------------- attend
def retrieve_and_attend(q, k_cache, v_cache, k_loc, v_loc, is_mem_loc, cos, sin, block: int, top_k: int,
                        idx=None, n_buckets: int = 64):
    """Whole step in the model dtype with the reference's rounding points.

    q, k_loc: (B,nh,T,hd) rotated; k_cache (un-rotated), v_cache: (B,nh,S,hd);
    cos/sin: (n_pos, hd) tables in the model dtype.
    Returns ``(out (B,nh,T,hd), idx (B,nh,T,k) int64)``.
    """
    B, nh, T, hd = q.shape
    S = k_cache.shape[2]
    g = retrieval_geometry(S, block, top_k)
    inc = g["incomplete_len"]
    k = g["k"]
    if inc:
        assert T + inc <= block                                                     # :330
        k_loc, v_loc = local_window(k_cache, v_cache, k_loc, v_loc, cos, sin, block)
    if idx is None:
        idx = select_topk(landmark_scores(q, k_cache, cos, sin, block, top_k), k)
    pos = gather_positions(idx, g["num_mems"], k, block, g["prefix_len"])           # (B,nh,T,k,bs)
    ksel = apply_rotary(gather_blocks(k_cache, idx, block), cos, sin, pos)          # :408-410
    vsel = gather_blocks(v_cache, idx, block)
    ksel = ksel.flatten(3, 4)                                                       # (B,nh,T,k*bs,hd)
    vsel = vsel.flatten(3, 4)
    div = math.sqrt(hd)
    prefix = (q.unsqueeze(3) @ ksel.transpose(3, 4)).squeeze(3) / div               # :412
    add, im_loc, ls_loc = local_masks(is_mem_loc, T, q.dtype)
    if inc:                                                                         # :331-335 and the mask slice of :460
        add = torch.cat((torch.zeros(B, 1, T, inc, dtype=add.dtype), add), dim=-1)
        im_loc = torch.cat((torch.zeros(B, 1, T, inc, dtype=torch.bool).expand(im_loc.shape[0], 1, T, inc), im_loc), dim=-1)
        ls_loc = torch.cat((torch.ones(B, 1, T, inc, dtype=torch.bool).expand(ls_loc.shape[0], 1, T, inc), ls_loc), dim=-1)
    local = (q @ k_loc.transpose(2, 3)) / div + add                                 # :448,460
    local = torch.max(local, torch.tensor(torch.finfo(q.dtype).min, dtype=q.dtype)) # :461
    x = torch.cat((prefix, local), dim=-1)
    im_prefix = torch.zeros(k * block, dtype=torch.bool)
    im_prefix[block - 1 :: block] = True                                            # :415
    im = torch.cat((im_prefix.expand(B, 1, T, -1), im_loc), dim=-1).expand(B, nh, T, -1)
    ls = torch.cat((torch.zeros(B, 1, T, k * block, dtype=torch.bool), ls_loc), dim=-1).expand(B, nh, T, -1)
    w = grouped_softmax(x, im, ls, n_buckets).to(q.dtype)                           # :469
    w_prefix, w_loc = w[..., : k * block], w[..., k * block :]
    out = w_loc @ v_loc + (w_prefix.unsqueeze(3) @ vsel).squeeze(3)                 # :472-474
    return out, idx


def retrieve_and_attend_s1(q, k_cache, v_cache, k_loc, v_loc, cos, sin, block: int, top_k: int, idx,
                           heads=None, tokens=None):
    """Same step as fp32 closed form: the ``k`` retrieved blocks (rotated at their
    slot positions) act as history blocks in front of the local chunk, whose
    landmarks sit at fixed stride.  Evaluated for selected heads / tokens of
    batch 0..B-1; returns dict {(b, h, t): out (hd,) fp32}."""
    B, nh, T, hd = q.shape
    S = k_cache.shape[2]
    g = retrieval_geometry(S, block, top_k)
    k = g["k"]
    inc = g["incomplete_len"]
    if inc:                       # the tail opens the current block; zero rows stand in for its queries
        k_loc, v_loc = local_window(k_cache, v_cache, k_loc, v_loc, cos, sin, block)
        q = torch.cat((torch.zeros(B, nh, inc, hd, dtype=q.dtype), q), dim=2)
    heads = range(nh) if heads is None else heads
    tokens = range(T) if tokens is None else tokens
    res = {}
    for b in range(B):
        for h in heads:
            blocks_k = k_cache[b, h, : g["full_len"]].unflatten(0, (g["num_mems"], block))
            blocks_v = v_cache[b, h, : g["full_len"]].unflatten(0, (g["num_mems"], block))
            for t in tokens:
                sel = idx[b, h, t]
                pos = gather_positions(sel, g["num_mems"], k, block, g["prefix_len"])
                ks = apply_rotary(blocks_k[sel], cos, sin, pos).flatten(0, 1)
                vs = blocks_v[sel].flatten(0, 1)
                kk = torch.cat((ks, k_loc[b, h]), 0).float()
                vv = torch.cat((vs, v_loc[b, h]), 0).float()
                res[(b, h, t)] = s1_attention(q[b, h].float(), kk, vv, block, rows=[inc + t])[0]
    return res
