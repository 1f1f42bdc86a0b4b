"""Closed form ("S1") of landmark grouped-softmax causal attention.  TEST ORACLE.

What the reference's fused kernel computes
(``llama/ltriton/flash_landmark_attention.py:6-122`` forward, ``:152-305``
backward) and what its high-level path computes through masks and a grouped
softmax (``llama/llama_mem.py:222-243``; ``lm_benchmark/models/landmark.py:88-119``),
written as one formula per query row.

Notation.  ``block`` keys form a landmark block; the last key of every block is
the landmark.  ``P = (Lk - Lq) // block`` blocks of history precede the queries
(``flash_landmark_attention.py:396-398``).  Query row ``i`` sits at absolute
position ``p = i + P*block`` in block ``c = p // block``; a landmark query looks
one position to the left (``flash_landmark_attention.py:29-30``), so its limit
is ``lim = p - 1`` and otherwise ``lim = p``.

    s_j  = scale * <q_i, k_j>
    G_i  = {landmark keys of blocks b < c}  U  {j : c*block <= j <= lim}
    g    = softmax of s over G_i        (M_i = max, L_i = sum exp(s - M_i))
    out_i = sum_{j in block c, j <= lim} g_j v_j
          + sum_{b < c} g_{lm(b)} * sum_{j in block b, j != lm(b)} softmax_b(s)_j v_j

``softmax_b`` runs over the ``block - 1`` non-landmark keys of block ``b``.
Landmark *value* rows never enter the output.

Pinned by ``tests/test_oracle_s1.py``: the vectorised form against the literal
per-row loop, against textbook causal softmax attention where S1 reduces to it,
rows of weights summing to one, invariances, a hand-derived two-block case,
finite differences (gradients) and the explicit backward formulas against
autograd.
"""
from __future__ import annotations

import math

import torch


def default_scale(d: int) -> float:
    # flash_landmark_attention.py:400-401
    return 1.0 / math.sqrt(d)


# --------------------------------------------------------------------------
# literal per-row evaluation, Python floats.  Tiny shapes only.
# --------------------------------------------------------------------------
def s1_rows_python(q, k, v, block: int, scale: float | None = None):
    """Evaluate S1 row by row with Python ``float`` arithmetic (float64).

    q: (Lq, D), k, v: (Lk, D) nested lists / tensors.  Returns (out, L, M) as
    lists.  Written to share no code with :func:`s1_attention`.
    """
    q = [[float(x) for x in row] for row in q]
    k = [[float(x) for x in row] for row in k]
    v = [[float(x) for x in row] for row in v]
    lq, lk, d = len(q), len(k), len(q[0])
    if scale is None:
        scale = default_scale(d)
    assert (lk - lq) % block == 0
    hist = lk - lq
    outs, ls, ms = [], [], []
    for i in range(lq):
        p = i + hist
        c = p // block
        lim = p - 1 if p % block == block - 1 else p
        s = [scale * sum(a * b for a, b in zip(q[i], k[j])) for j in range(lk)]
        bucket = [b * block + block - 1 for b in range(c)]
        bucket += [j for j in range(c * block, lim + 1)]
        m = max(s[j] for j in bucket)
        e = {j: math.exp(s[j] - m) for j in bucket}
        ell = sum(e.values())
        o = [0.0] * d
        for j in range(c * block, lim + 1):
            w = e[j] / ell
            for t in range(d):
                o[t] += w * v[j][t]
        for b in range(c):
            members = list(range(b * block, b * block + block - 1))
            mb = max(s[j] for j in members)
            eb = [math.exp(s[j] - mb) for j in members]
            zb = sum(eb)
            gate = e[b * block + block - 1] / ell
            for j, ej in zip(members, eb):
                w = gate * ej / zb
                for t in range(d):
                    o[t] += w * v[j][t]
        outs.append(o)
        ls.append(ell)
        ms.append(m)
    return outs, ls, ms


def s1_rows_python_irregular(q, k, v, is_mem, scale: float | None = None):
    """S1 for landmarks at arbitrary positions, row by row in Python floats: what the reference's high-level
    path computes for any ``is_mem`` (``llama/llama_mem.py:222-243,807-815``;
    ``lm_benchmark/models/landmark.py:88-119,216-224``).

    q: (Lq, D), k, v: (Lk, D); is_mem: Lk booleans.  A block is a run of tokens that ends in a landmark; the
    tokens behind the last landmark form a last block without one.  Query row i sits at key position
    ``p = i + Lk - Lq``; it sees the keys of its own block up to ``p`` (a landmark query: up to ``p - 1``) and
    every earlier block through that block's landmark.  Returns ``out`` as lists.  Shares no code with
    :mod:`oracle.highlevel`.
    """
    q = [[float(x) for x in row] for row in q]
    k = [[float(x) for x in row] for row in k]
    v = [[float(x) for x in row] for row in v]
    is_mem = [bool(x) for x in is_mem]
    lq, lk, d = len(q), len(k), len(q[0])
    assert len(is_mem) == lk
    if scale is None:
        scale = default_scale(d)
    block_of, b = [], 0
    for j in range(lk):
        block_of.append(b)
        if is_mem[j]:
            b += 1
    members = {}
    for j in range(lk):
        members.setdefault(block_of[j], []).append(j)
    outs = []
    for i in range(lq):
        p = i + lk - lq
        c = block_of[p]
        lim = p - 1 if is_mem[p] else p
        s = [scale * sum(x * y for x, y in zip(q[i], k[j])) for j in range(lk)]
        own = [j for j in members[c] if j <= lim]
        landmarks = [members[bb][-1] for bb in range(c)]            # every earlier block ends in its landmark
        bucket = landmarks + own
        o = [0.0] * d
        if bucket:
            m = max(s[j] for j in bucket)
            e = {j: math.exp(s[j] - m) for j in bucket}
            ell = sum(e.values())
            for j in own:
                for t in range(d):
                    o[t] += e[j] / ell * v[j][t]
            for bb in range(c):
                normal = members[bb][:-1]
                if not normal:
                    continue                                         # a block of a landmark alone carries nothing
                mb = max(s[j] for j in normal)
                eb = [math.exp(s[j] - mb) for j in normal]
                zb = sum(eb)
                gate = e[members[bb][-1]] / ell
                for j, ej in zip(normal, eb):
                    for t in range(d):
                        o[t] += gate * ej / zb * v[j][t]
        outs.append(o)
    return outs


# --------------------------------------------------------------------------
# vectorised, differentiable form
# --------------------------------------------------------------------------
def _geometry(lq: int, lk: int, block: int, rows, device):
    assert (lk - lq) % block == 0, "history must be whole blocks (flash_landmark_attention.py:397)"
    hist = lk - lq
    if rows is None:
        rows = torch.arange(lq, device=device)
    else:
        rows = torch.as_tensor(rows, device=device, dtype=torch.long)
    pos = rows + hist                                   # absolute position of each query
    cur = pos // block                                  # its block
    lim = torch.where(pos % block == block - 1, pos - 1, pos)
    return rows, cur, lim


def s1_weights(q, k, block: int, scale: float | None = None, rows=None, group_scale=None):
    """Attention weights (…, R, Lk) of S1 plus the global-bucket statistics.

    ``group_scale`` (…, n_blocks, R), optional: factor of earlier block b's contribution to row i (group dropout,
    ``lm_benchmark/models/landmark.py:110-113``: the landmark probabilities that scale the earlier blocks are
    dropped or scaled by 1 / (1 - p), the softmax over the landmarks itself is not renormalised).

    q: (..., Lq, D), k: (..., Lk, D) in any float dtype; the arithmetic runs in
    that dtype.  ``rows`` optionally restricts the evaluation to some query rows
    (for long sequences).  Returns ``(w, L, M)``.
    """
    lq, d = q.shape[-2], q.shape[-1]
    lk = k.shape[-2]
    if scale is None:
        scale = default_scale(d)
    rows, cur, lim = _geometry(lq, lk, block, rows, q.device)
    qs = q.index_select(-2, rows)
    s = (qs @ k.transpose(-1, -2)) * scale              # (..., R, Lk)

    nb = -(-lk // block)
    pad = nb * block - lk
    if pad:
        s = torch.nn.functional.pad(s, (0, pad), value=0.0)
    j = torch.arange(nb * block, device=q.device)
    kb = j // block                                      # block of each key
    is_lm = (j % block) == block - 1
    in_range = j < lk

    earlier = kb[None, :] < cur[:, None]                 # (R, Lkp)
    same = (kb[None, :] == cur[:, None]) & (j[None, :] <= lim[:, None]) & in_range[None, :]
    bucket = (earlier & is_lm[None, :]) | same           # the global bucket G_i
    ninf = torch.finfo(s.dtype).min
    sg = torch.where(bucket, s, torch.full_like(s, ninf))
    M = sg.amax(-1, keepdim=True)
    eg = torch.where(bucket, torch.exp(sg - M), torch.zeros_like(s))
    L = eg.sum(-1, keepdim=True)
    g = eg / L                                           # softmax over the bucket

    # per-block softmax over the non-landmark keys of earlier blocks
    local = earlier & ~is_lm[None, :]
    sl = torch.where(local, s, torch.full_like(s, ninf)).unflatten(-1, (nb, block))
    ml = sl.amax(-1, keepdim=True)
    el = torch.where(local.unflatten(-1, (nb, block)), torch.exp(sl - ml), torch.zeros_like(sl))
    zl = el.sum(-1, keepdim=True)
    pl = el / torch.where(zl > 0, zl, torch.ones_like(zl))
    gate = g.unflatten(-1, (nb, block))[..., block - 1:block]      # g at each block's landmark
    if group_scale is not None:
        gate = gate * group_scale.transpose(-1, -2).unsqueeze(-1).to(gate.dtype)
    w = (pl * gate).flatten(-2) + torch.where(same, g, torch.zeros_like(g))
    if pad:
        w = w[..., :lk]
    return w, L.squeeze(-1), M.squeeze(-1)


def s1_attention(q, k, v, block: int, scale: float | None = None, rows=None, return_stats=False, group_scale=None):
    """out (…, R, D) of S1; differentiable through torch autograd."""
    w, L, M = s1_weights(q, k, block, scale, rows, group_scale)
    out = w @ v
    if return_stats:
        return out, L, M
    return out


# --------------------------------------------------------------------------
# explicit backward (the formulas a fused kernel evaluates)
# --------------------------------------------------------------------------
def s1_backward_formulas(q, k, v, do, block: int, scale: float | None = None):
    """dq, dk, dv from the tile formulas of ``flash_landmark_attention.py:152-305``.

    With ``do' = do / L`` and ``delta = rowsum(o * do')`` (``:125-149``):

      earlier block b:  P = local softmax, gt = exp(s_lm - M), dP = do' V^T,
                        nD = rowsum(P * dP) over the normal keys,
                        dS_normal = gt * P * (dP - nD),  dS_lm = gt * (nD - delta),
                        dV += (gt * P)^T do'
      current block:    p = exp(s - M) on visible keys, dS = p * (dP - delta), dV += p^T do'
      dK = scale * dS^T Q,  dQ = scale * dS K

    ``nD`` replaces the reference's extra ``P @ V`` product (``:274-276``):
    rowsum(do' * (P V)) == rowsum(P * (do' V^T)).
    Dense O(Lq*Lk) evaluation, all rows, for test sizes.
    """
    lq, d = q.shape[-2], q.shape[-1]
    lk = k.shape[-2]
    if scale is None:
        scale = default_scale(d)
    assert lk % block == 0 and lq % block == 0, "backward needs full blocks (flash_landmark_attention.py:359-360)"
    rows, cur, lim = _geometry(lq, lk, block, None, q.device)
    nb = lk // block
    j = torch.arange(lk, device=q.device)
    kb = j // block
    is_lm = (j % block) == block - 1
    earlier = kb[None, :] < cur[:, None]
    same = (kb[None, :] == cur[:, None]) & (j[None, :] <= lim[:, None])
    normal = earlier & ~is_lm[None, :]
    lm_e = earlier & is_lm[None, :]

    s = (q @ k.transpose(-1, -2)) * scale
    out, L, M = s1_attention(q, k, v, block, scale, return_stats=True)
    dos = do / L[..., None]
    delta = (out * dos).sum(-1, keepdim=True)                       # (…, Lq, 1)
    dP = dos @ v.transpose(-1, -2)                                  # (…, Lq, Lk)

    ninf = torch.finfo(s.dtype).min
    sl = torch.where(normal, s, torch.full_like(s, ninf)).unflatten(-1, (nb, block))
    el = torch.where(normal.unflatten(-1, (nb, block)), torch.exp(sl - sl.amax(-1, keepdim=True)), torch.zeros_like(sl))
    zl = el.sum(-1, keepdim=True)
    P = el / torch.where(zl > 0, zl, torch.ones_like(zl))           # (…, Lq, nb, block)
    gt = torch.exp(s - M[..., None])                                # exp(s - M) everywhere
    gt_lm = torch.where(lm_e, gt, torch.zeros_like(gt)).unflatten(-1, (nb, block))[..., block - 1:block]
    nD = (P * dP.unflatten(-1, (nb, block))).sum(-1, keepdim=True)  # (…, Lq, nb, 1)

    W_e = (gt_lm * P).flatten(-2)                                   # weights*L on earlier normal keys
    dS_e = (gt_lm * P * (dP.unflatten(-1, (nb, block)) - nD)).flatten(-2)
    dS_lm = (gt_lm * (nD - delta[..., None])).expand(*P.shape).flatten(-2)
    dS_lm = torch.where(lm_e, dS_lm, torch.zeros_like(dS_lm))
    p_cur = torch.where(same, gt, torch.zeros_like(gt))
    dS_cur = p_cur * (dP - delta)

    dS = dS_e + dS_lm + dS_cur
    W = W_e + p_cur
    dv = W.transpose(-1, -2) @ dos
    dk = scale * (dS.transpose(-1, -2) @ q)
    dq = scale * (dS @ k)
    return dq, dk, dv
