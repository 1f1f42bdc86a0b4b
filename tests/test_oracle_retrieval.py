"""Pins oracle/rotary.py and oracle/retrieval.py."""
import math

import pytest
import torch

from oracle import retrieval, rotary


def _rand(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * scale).to(dtype)


# ------------------------------------------------------------------ rotary
def test_rotary_identity_norm_and_relative_property():
    d = 16
    cos, sin = rotary.rotary_tables(64, d, torch.float64)
    x, y = _rand(5, d, seed=1, dtype=torch.float64), _rand(5, d, seed=2, dtype=torch.float64)
    assert torch.equal(rotary.apply_rotary(x, cos, sin, torch.zeros(5, dtype=torch.long)), x)
    pos = torch.tensor([6, 9, 17, 40, 63])
    xr = rotary.apply_rotary(x, cos, sin, pos)
    pair = lambda t: t[..., : d // 2] ** 2 + t[..., d // 2 :] ** 2
    assert torch.allclose(pair(xr), pair(x), atol=1e-12)
    # <rot(x, m), rot(y, n)> depends only on m - n
    a = (rotary.apply_rotary(x, cos, sin, pos) * rotary.apply_rotary(y, cos, sin, pos - 3)).sum(-1)
    b = (rotary.apply_rotary(x, cos, sin, pos - 2) * rotary.apply_rotary(y, cos, sin, pos - 5)).sum(-1)
    assert torch.allclose(a, b, atol=1e-10)
    # first pair rotates by the full angle: (x0, x_{d/2}) at position 1 turns by 1 radian
    e = torch.zeros(1, d, dtype=torch.float64)
    e[0, 0] = 1.0
    r = rotary.apply_rotary(e, cos, sin, torch.tensor([1]))
    assert abs(r[0, 0] - math.cos(1.0)) < 1e-7 and abs(r[0, d // 2] - math.sin(1.0)) < 1e-7


def test_rotary_equals_torch_bf16_elementwise():
    d = 32
    cos, sin = rotary.rotary_tables(128, d, torch.bfloat16)
    x = _rand(2, 3, 7, d, seed=3, dtype=torch.bfloat16)
    pos = torch.tensor([0, 5, 31, 64, 99, 100, 127])
    ours = rotary.apply_rotary(x, cos, sin, pos)
    theirs = x * cos[pos] + rotary.rotate_half(x) * sin[pos]         # torch rounds after every op
    assert torch.equal(ours, theirs)


# ---------------------------------------------------------------- geometry
def test_geometry_hand_worked():
    # 10 cached blocks of 4, top-3: prefix_len = 40 - 16 = 24; older blocks all at slot 0.
    g = retrieval.retrieval_geometry(40, 4, 3)
    assert (g["num_mems"], g["k"], g["prefix_len"], g["incomplete_len"]) == (10, 3, 24, 0)
    assert g["mem_pos"].tolist() == [27] * 7 + [31, 35, 39]          # newest three keep their true positions
    # benchmark config 4 numbers
    g = retrieval.retrieval_geometry(32768, 32, 4)
    assert g["prefix_len"] == 32608
    assert g["mem_pos"][:1020].unique().tolist() == [32639]
    assert g["mem_pos"][1020:].tolist() == [32671, 32703, 32735, 32767]
    # fewer cached blocks than top_k
    g = retrieval.retrieval_geometry(8, 4, 5)
    assert (g["k"], g["prefix_len"]) == (2, -4) and g["mem_pos"].tolist() == [3, 7]
    # incomplete tail
    g = retrieval.retrieval_geometry(43, 4, 3)
    assert (g["full_len"], g["incomplete_len"], g["num_mems"]) == (40, 3, 10)


def test_gather_positions_hand_worked():
    idx = torch.tensor([1, 4, 8, 9])                                  # 10 blocks, k=4: blocks >= 6 are "new"
    pos = retrieval.gather_positions(idx, 10, 4, 4, 20)
    assert pos[:, 0].tolist() == [20, 24, 28 + 4, 32 + 4]
    assert pos[2].tolist() == [32, 33, 34, 35]


# --------------------------------------------------------------- selection
def test_select_topk_brute_force_and_torch_topk_on_untied_rows():
    g = torch.Generator().manual_seed(4)
    sc = torch.randn(64, 40, generator=g).to(torch.bfloat16)          # bf16 -> plenty of ties
    k = 4
    got = retrieval.select_topk(sc, k)
    for r in range(sc.shape[0]):
        row = sc[r].float().tolist()
        order = sorted(range(len(row)), key=lambda j: (-row[j], j))
        assert got[r].tolist() == sorted(order[:k])
    ties = retrieval.boundary_tie_rows(sc, k)
    assert ties.any() and not ties.all()
    tk = sc.float().topk(k, dim=-1).indices.sort(-1).values
    assert torch.equal(got[~ties], tk[~ties])


def test_score_contract_rounding_points():
    B, nh, T, hd, bs, nm = 1, 2, 5, 16, 4, 6
    q = _rand(B, nh, T, hd, seed=5, dtype=torch.bfloat16, scale=0.5)
    kc = _rand(B, nh, nm * bs, hd, seed=6, dtype=torch.bfloat16, scale=0.5)
    cos, sin = rotary.rotary_tables(64, hd, torch.bfloat16)
    sc = retrieval.landmark_scores(q, kc, cos, sin, bs, 2)
    g = retrieval.retrieval_geometry(nm * bs, bs, 2)
    # recompute one entry by hand with python floats
    b, h, t, m = 0, 1, 3, 4
    lk = kc[b, h, m * bs + bs - 1]
    lkr = rotary.apply_rotary(lk[None], cos, sin, g["mem_pos"][m : m + 1])[0]
    import numpy as np
    acc = np.float32(0.0)
    for a, c in zip(q[b, h, t].float().tolist(), lkr.float().tolist()):
        acc = np.float32(acc + np.float32(np.float32(a) * np.float32(c)))     # one fp32 rounding per step
    two = torch.tensor(float(acc)).bfloat16().float() / torch.tensor(math.sqrt(hd)).float()
    assert sc[b, h, t, m] == two.bfloat16()
    # and the sequential sum stays within fp32 accumulation error of the exact dot product
    exact = sum(float(a) * float(c) for a, c in zip(q[b, h, t], lkr))
    assert abs(float(acc) - exact) < 1e-5
    assert sc.dtype == torch.bfloat16 and sc.shape == (B, nh, T, nm)


# ------------------------------------------------------------------ attend
def test_gather_blocks_is_a_copy_of_the_selected_blocks():
    B, nh, T, hd, bs, nm = 1, 2, 3, 4, 4, 5
    cache = _rand(B, nh, nm * bs, hd, seed=7)
    idx = torch.tensor([[0, 3], [1, 4], [2, 3]])[None, None].expand(B, nh, T, 2)
    got = retrieval.gather_blocks(cache, idx, bs)
    for t in range(T):
        for j in range(2):
            blk = int(idx[0, 0, t, j])
            assert torch.equal(got[0, 1, t, j], cache[0, 1, blk * bs : (blk + 1) * bs])


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
def test_attend_in_model_dtype_equals_fp32_closed_form(dtype, tol):
    B, nh, T, hd, bs, nm, k = 1, 2, 16, 16, 8, 6, 3
    S = nm * bs
    q = _rand(B, nh, T, hd, seed=8, dtype=dtype, scale=0.5)
    kc = _rand(B, nh, S, hd, seed=9, dtype=dtype, scale=0.5)
    vc = _rand(B, nh, S, hd, seed=10, dtype=dtype, scale=0.5)
    kl = _rand(B, nh, T, hd, seed=11, dtype=dtype, scale=0.5)
    vl = _rand(B, nh, T, hd, seed=12, dtype=dtype, scale=0.5)
    is_mem = (torch.arange(T) % bs == bs - 1)[None]
    cos, sin = rotary.rotary_tables(S + T, hd, dtype)
    out, idx = retrieval.retrieve_and_attend(q, kc, vc, kl, vl, is_mem, cos, sin, bs, k)
    assert idx.shape == (B, nh, T, k) and (idx[..., 1:] > idx[..., :-1]).all()
    ref = retrieval.retrieve_and_attend_s1(q, kc, vc, kl, vl, cos, sin, bs, k, idx)
    for (b, h, t), o in ref.items():
        assert (out[b, h, t].float() - o).abs().max() < tol, (b, h, t)


# ------------------------------------------------- incomplete cached block (decode between landmarks)
def _tail_case(dtype, inc, T, bs=8, nm=5, k=2, hd=16, nh=2, seed=20):
    S = nm * bs + inc
    q = _rand(1, nh, T, hd, seed=seed, dtype=dtype, scale=0.5)
    kc = _rand(1, nh, S, hd, seed=seed + 1, dtype=dtype, scale=0.5)
    vc = _rand(1, nh, S, hd, seed=seed + 2, dtype=dtype, scale=0.5)
    kl = _rand(1, nh, T, hd, seed=seed + 3, dtype=dtype, scale=0.5)
    vl = _rand(1, nh, T, hd, seed=seed + 4, dtype=dtype, scale=0.5)
    is_mem = ((torch.arange(T) + inc) % bs == bs - 1)[None]          # the block's landmark, if the chunk reaches it
    cos, sin = rotary.rotary_tables(S + T, hd, dtype)
    return q, kc, vc, kl, vl, is_mem, cos, sin, bs, k


def test_geometry_ignores_the_tail():
    # 5 complete blocks of 8 and 3 tail tokens: positions as for S = 40 (llama_mem.py:321-324,358-365)
    a, b = retrieval.retrieval_geometry(43, 8, 2), retrieval.retrieval_geometry(40, 8, 2)
    assert (a["full_len"], a["incomplete_len"], a["num_mems"], a["prefix_len"]) == (40, 3, 5, 16)
    assert torch.equal(a["mem_pos"], b["mem_pos"])


@pytest.mark.parametrize("inc,T", [(3, 1), (1, 6), (5, 3), (7, 1)])     # (5,3) and (7,1) end on the landmark
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
def test_attend_with_incomplete_cached_block_equals_closed_form(dtype, tol, inc, T):
    q, kc, vc, kl, vl, is_mem, cos, sin, bs, k = _tail_case(dtype, inc, T)
    out, idx = retrieval.retrieve_and_attend(q, kc, vc, kl, vl, is_mem, cos, sin, bs, k)
    # selection sees the complete blocks only
    full = kc[:, :, : kc.shape[2] - inc]
    assert torch.equal(idx, retrieval.select_topk(retrieval.landmark_scores(q, full, cos, sin, bs, k), k))
    ref = retrieval.retrieve_and_attend_s1(q, kc, vc, kl, vl, cos, sin, bs, k, idx)
    for (b, h, t), o in ref.items():
        assert (out[b, h, t].float() - o).abs().max() < tol, (b, h, t)


def test_incomplete_cached_block_literal_row():
    """One query written out by hand in float64: global bucket = landmarks of the retrieved blocks,
    the tail, the new tokens up to the query (the landmark query not itself); every retrieved block
    contributes its own softmax over its non-landmark keys, weighted by its landmark's share."""
    inc, T = 5, 3
    q, kc, vc, kl, vl, is_mem, cos, sin, bs, k = _tail_case(torch.float32, inc, T)
    out, idx = retrieval.retrieve_and_attend(q, kc, vc, kl, vl, is_mem, cos, sin, bs, k)
    g = retrieval.retrieval_geometry(kc.shape[2], bs, k)
    hd = q.shape[-1]
    for h in range(q.shape[1]):
        for t in range(T):
            qq = q[0, h, t].double()
            sel = idx[0, h, t]
            pos = retrieval.gather_positions(sel, g["num_mems"], k, bs, g["prefix_len"])
            blocks = [(rotary.apply_rotary(kc[0, h, b * bs : (b + 1) * bs], cos, sin, pos[j]).double(),
                       vc[0, h, b * bs : (b + 1) * bs].double()) for j, b in enumerate(sel.tolist())]
            tail_pos = torch.arange(g["full_len"], g["full_len"] + inc)
            wk = torch.cat((rotary.apply_rotary(kc[0, h, g["full_len"] :], cos, sin, tail_pos), kl[0, h])).double()
            wv = torch.cat((vc[0, h, g["full_len"] :], vl[0, h])).double()
            last = inc + t - (1 if (inc + t) % bs == bs - 1 else 0)      # the landmark query does not see itself
            s_win = (wk[: last + 1] @ qq) / math.sqrt(hd)
            s_lm = torch.stack([(kb[bs - 1] @ qq) / math.sqrt(hd) for kb, _ in blocks])
            z = torch.cat((s_lm, s_win))
            w = torch.softmax(z, 0)
            o = w[k:] @ wv[: last + 1]
            for j, (kb, vb) in enumerate(blocks):
                loc = torch.softmax((kb[: bs - 1] @ qq) / math.sqrt(hd), 0)
                o = o + w[j] * (loc @ vb[: bs - 1])
            assert (out[0, h, t].double() - o).abs().max() < 2e-5, (h, t)


# ------------------------------------------------- one selection per head (max_over_tokens, llama_mem.py:373-377)
def test_exp2_contract_against_numpy_and_exact_at_integers():
    import numpy as np
    t = -np.abs(np.random.default_rng(0).normal(size=50000)).astype(np.float32) * np.float32(25.0)
    got = retrieval.exp2_contract(t)
    want = np.exp2(t.astype(np.float64))
    assert got.dtype == np.float32
    assert (np.abs(got - want) <= 5e-7 * want).all()
    n = -np.arange(0, 127, dtype=np.float32)
    assert np.array_equal(retrieval.exp2_contract(n), np.exp2(n))           # powers of two come out exactly
    assert retrieval.exp2_contract(np.float32(-126.5)) == 0 and retrieval.exp2_contract(np.float32(-1e30)) == 0
    # monotone over a fine grid (a flipped coefficient sign or a dropped term breaks this)
    grid = -np.linspace(0, 40, 200001).astype(np.float32)
    assert (np.diff(retrieval.exp2_contract(grid)) <= 0).all()


def test_softmax_contract_literal_loop_and_torch_softmax():
    import numpy as np
    x = _rand(2, 3, 4, 200, seed=30, dtype=torch.bfloat16, scale=3.0).float()
    got = retrieval.softmax_contract(x, torch.bfloat16)
    # literal wave order on one row: 64 lanes add their strided elements in turn, then fold by halves
    row = x[1, 2, 3].numpy()
    e = retrieval.exp2_contract(((row - row.max()).astype(np.float32) * np.float32(1.4426950408889634)).astype(np.float32))
    lanes = [np.float32(0.0)] * 64
    for m in range(len(e)):
        lanes[m % 64] = np.float32(lanes[m % 64] + e[m])
    w = 32
    while w:
        lanes = [np.float32(lanes[i] + lanes[i + w]) for i in range(w)]
        w //= 2
    want = torch.tensor([np.float32(v / lanes[0]) for v in e]).to(torch.bfloat16)
    assert torch.equal(got[1, 2, 3], want)
    # library softmax: same values up to the last bit of the 16-bit result, and on nearly every element
    lib = torch.softmax(x, dim=-1, dtype=torch.float32)
    assert (got.float() - lib).abs().max() <= lib.max() * 2 ** -8
    assert (got != lib.to(torch.bfloat16)).float().mean() < 1e-3
    assert (got.float().sum(-1) - 1).abs().max() < 2e-2


def test_shared_selection_equals_torch_expression_on_untied_heads():
    B, nh, T, hd, bs, nm, k = 2, 4, 12, 16, 8, 40, 3
    S = nm * bs
    q = _rand(B, nh, T, hd, seed=31, dtype=torch.bfloat16, scale=1.5)
    kc = _rand(B, nh, S, hd, seed=32, dtype=torch.bfloat16, scale=1.5)
    cos, sin = rotary.rotary_tables(S + T, hd, torch.bfloat16)
    sc = retrieval.landmark_scores(q, kc, cos, sin, bs, k)
    agg = retrieval.aggregate_max_over_tokens(sc)
    assert agg.shape == (B, nh, 1, nm) and agg.dtype == torch.bfloat16
    idx = retrieval.select_topk(agg, k)
    assert idx.shape == (B, nh, 1, k)
    lib = torch.softmax(sc, dim=-1, dtype=torch.float32).to(sc.dtype).amax(dim=2, keepdim=True)      # :376-377
    lib_idx = lib.topk(k, dim=-1).indices.sort(dim=-1).values                                         # :384
    ok = ~retrieval.boundary_tie_rows(lib, k) & (lib == agg).all(-1)
    assert ok.float().mean() > 0.7
    assert torch.equal(idx[ok], lib_idx[ok])


@pytest.mark.parametrize("inc,T", [(0, 16), (0, 5), (3, 4), (5, 3)])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
def test_shared_attend_equals_closed_form_with_history_blocks(dtype, tol, inc, T):
    B, nh, hd, bs, nm, k = 1, 2, 16, 8, 6, 3
    S = nm * bs + inc
    q = _rand(B, nh, T, hd, seed=40, dtype=dtype, scale=0.5)
    kc = _rand(B, nh, S, hd, seed=41, dtype=dtype, scale=0.5)
    vc = _rand(B, nh, S, hd, seed=42, dtype=dtype, scale=0.5)
    kl = _rand(B, nh, T, hd, seed=43, dtype=dtype, scale=0.5)
    vl = _rand(B, nh, T, hd, seed=44, dtype=dtype, scale=0.5)
    is_mem = ((torch.arange(T) + inc) % bs == bs - 1)[None]
    cos, sin = rotary.rotary_tables(S + T, hd, dtype)
    out, idx = retrieval.retrieve_and_attend_shared(q, kc, vc, kl, vl, is_mem, cos, sin, bs, k)
    assert idx.shape == (B, nh, 1, k) and (idx[..., 1:] > idx[..., :-1]).all()
    ref = retrieval.retrieve_and_attend_shared_s1(q, kc, vc, kl, vl, cos, sin, bs, k, idx)
    assert (out.float() - ref).abs().max() < tol
    # every query of a head uses the head's one set: the per-token step with that set forced gives the same
    per_tok, _ = retrieval.retrieve_and_attend(q, kc, vc, kl, vl, is_mem, cos, sin, bs, k, idx=idx.expand(B, nh, T, k))
    assert (out.float() - per_tok.float()).abs().max() < tol


def test_shared_window_rows_hand_worked():
    # 5 blocks of 4 + tail of 2, top-2, head picks blocks {1, 4}: block 4 is among the newest two -> bumped one block
    bs, nm, inc, T, hd = 4, 5, 2, 1, 8
    S = nm * bs + inc
    kc = _rand(1, 1, S, hd, seed=50)
    vc = _rand(1, 1, S, hd, seed=51)
    kl, vl = _rand(1, 1, T, hd, seed=52), _rand(1, 1, T, hd, seed=53)
    cos, sin = rotary.rotary_tables(S + T, hd)
    idx = torch.tensor([1, 4]).view(1, 1, 1, 2)
    keys, values = retrieval.shared_window(kc, vc, kl, vl, idx, cos, sin, bs, 2)
    assert keys.shape == (1, 1, 2 * bs + inc + T, hd)
    prefix_len = 20 - 3 * 4
    want_pos = [prefix_len + r for r in range(4)] + [prefix_len + 4 + 4 + r for r in range(4)] + [20, 21]
    src = list(range(4, 8)) + list(range(16, 20)) + [20, 21]
    want = rotary.apply_rotary(kc[0, 0, src], cos, sin, torch.tensor(want_pos))
    assert torch.equal(keys[0, 0, : 2 * bs + inc], want) and torch.equal(keys[0, 0, -1], kl[0, 0, 0])
    assert torch.equal(values[0, 0, : 2 * bs + inc], vc[0, 0, src]) and torch.equal(values[0, 0, -1], vl[0, 0, 0])


# ---------------------------------------- the score contract against the reference's literal expression
@pytest.mark.parametrize("seed", [0, 1])
def test_score_contract_against_the_literal_torch_expression(seed):
    """The reference scores with ``torch.matmul(q, mem_key.transpose(2, 3)) / math.sqrt(hd)`` in the model
    dtype and selects with ``topk(k).indices.sort()`` (``llama/llama_mem.py:367,384``).  torch's bf16 matmul
    accumulates in fp32 in an order of its own; the contract fixes the sequential order.  On inputs of
    benchmark config 4's shape and distribution (8 of its 32 heads) this evaluates the literal expression
    with torch on the CPU and bounds how far the two are apart:

    * the division step is identical, element for element, given the same product;
    * the products differ in fewer than 2 in 10^4 elements, and every difference is either one bf16 ulp
      (an fp32 sum that sat next to a rounding boundary) or belongs to a product so close to zero
      (|dot| < 2^-12) that fp32 accumulation error (< 2^-19 absolute) spans several of its tiny ulps;
    * under the same total order the two score sets select the same blocks in every row but those holding
      a differing score, and ``torch.topk`` itself disagrees with the contract only in rows with a tie at
      the k-th place or a differing score.
    The measured rates are printed (run with -s) and recorded in the design notes."""
    H, T, S, D, block, k = 8, 256, 32768, 128, 32, 4
    q = _rand(1, H, T, D, seed=100 + seed, dtype=torch.bfloat16, scale=0.5)
    kc = _rand(1, H, S, D, seed=200 + seed, dtype=torch.bfloat16, scale=0.5)
    cos, sin = rotary.rotary_tables(S + T, D, torch.bfloat16)
    geo = retrieval.retrieval_geometry(S, block, k)
    lk = kc[..., : geo["full_len"], :].unflatten(-2, (geo["num_mems"], block))[..., block - 1, :]
    mem_key = rotary.apply_rotary(lk, cos, sin, geo["mem_pos"])                  # llama_mem.py:366
    product = torch.matmul(q, mem_key.transpose(2, 3))                           # the literal expression, :367
    literal = product / math.sqrt(D)
    assert literal.dtype == torch.bfloat16
    contract = retrieval.landmark_scores(q, kc, cos, sin, block, k)
    dot = retrieval.sequential_dot_fp32(q, mem_key)

    # the division: fp32 quotient by float32(sqrt(hd)), rounded once
    assert torch.equal(literal, (product.float() / torch.tensor(math.sqrt(D), dtype=torch.float32)).bfloat16())

    def ordinal(x):                                                               # bf16 values on an integer line
        i = x.view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)

    first = dot.bfloat16()
    ulps = (ordinal(product) - ordinal(first)).abs()
    n_diff = int((ulps > 0).sum())
    assert n_diff <= 2e-4 * ulps.numel()
    several = ulps > 1
    assert (dot[several].abs() < 2.0 ** -12).all()
    assert ((product.float() - first.float())[several].abs() < 2.0 ** -19).all()

    score_diff_rows = (literal != contract).any(-1)
    want = retrieval.select_topk(contract, k)
    same_order = retrieval.select_topk(literal, k)
    rows_same_order = (want != same_order).any(-1)
    assert not (rows_same_order & ~score_diff_rows).any()
    torch_topk = literal.float().topk(k, dim=-1).indices.sort(-1).values          # :384
    rows_topk = (want != torch_topk).any(-1)
    ties = retrieval.boundary_tie_rows(contract, k) | retrieval.boundary_tie_rows(literal, k)
    assert not (rows_topk & ~ties & ~score_diff_rows).any()
    print(f"seed {seed}: products differing {n_diff} of {ulps.numel()} ({n_diff / ulps.numel():.1e}), "
          f"{int(several.sum())} of them near zero by more than one ulp; scores differing "
          f"{int((literal != contract).sum())}; rows selecting other blocks under the same order "
          f"{int(rows_same_order.sum())} of {rows_topk.numel()}; rows where torch.topk differs {int(rows_topk.sum())} "
          f"(tie rows: {int(ties.sum())})")
