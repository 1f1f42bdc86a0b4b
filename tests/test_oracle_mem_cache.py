"""Pins oracle/mem_cache.py (the restatement of lm_benchmark/models/caches/mem_cache.py:41-158) with
checks that do not retype its formulas: a ring against a plain list of blocks, hand-worked age and
position tables, the where/sort/where sequence against a brute-force sort by age, a ring selection
against the flat-cache selection of oracle/retrieval.py on the same blocks, literal loops for the
aggregations, torch.topk on rows without a boundary tie, and the interleaved rotary of the benchmark
against the half-split tables."""
import itertools

import pytest
import torch

from oracle import mem_cache, retrieval, rotary


def _chunk(B, nh, T, hs, block, phase, g):
    """T tokens whose landmark flags continue a stream that is `phase` tokens into a block."""
    k = torch.randn(B, nh, T, hs, generator=g)
    v = torch.randn(B, nh, T, hs, generator=g)
    is_mem = ((torch.arange(T) + phase) % block == block - 1)[None].expand(B, T)
    return k, v, is_mem


@pytest.mark.parametrize("capacity,block,chunks", [
    (4, 3, [3, 3, 6, 3, 9]),             # fills exactly, then wraps by one, then by three
    (4, 3, [5, 2, 8, 1, 1, 1, 13]),      # ragged chunks: blocks complete across calls
    (3, 4, [40]),                        # one chunk far larger than the ring: only the newest blocks stay
    (3, 4, [4, 20, 4]),                  # an overflowing chunk into a partly filled ring
    (5, 2, [2, 2, 2, 2, 2, 2, 2]),
])
def test_ring_store_against_a_list_of_blocks(capacity, block, chunks):
    B, nh, hs = 2, 3, 4
    g = torch.Generator().manual_seed(capacity * 100 + block)
    ring = mem_cache.RingStore(B, capacity, block, nh, hs)
    all_k, all_v = [], []                # the whole token stream
    seen = 0
    for T in chunks:
        k, v, im = _chunk(B, nh, T, hs, block, seen % block, g)
        ring.store(k, v, im)
        all_k.append(k), all_v.append(v)
        seen += T
        stream_k, stream_v = torch.cat(all_k, 2), torch.cat(all_v, 2)
        n_blocks = seen // block
        want = list(range(max(0, n_blocks - capacity), n_blocks))        # stream blocks still cached, oldest first
        assert ring.filled == len(want)
        assert ring.last_incomplete_len == seen % block
        assert torch.equal(ring.pending_k, stream_k[:, :, n_blocks * block:])
        ages = mem_cache.slot_ages(ring.filled, ring.cache_iter)
        assert sorted(ages.tolist()) == list(range(ring.filled))
        for slot in range(ring.filled):
            blk = want[ages[slot]]
            assert torch.equal(ring.cache_k[:, slot].permute(0, 2, 1, 3), stream_k[:, :, blk * block:(blk + 1) * block])
            assert torch.equal(ring.cache_v[:, slot].permute(0, 2, 1, 3), stream_v[:, :, blk * block:(blk + 1) * block])
        # the next block is written over the oldest one once the ring is full
        if ring.filled == capacity:
            assert ages[ring.cache_iter] == 0


def test_a_block_with_a_misplaced_landmark_is_refused():
    ring = mem_cache.RingStore(1, 4, 3, 1, 2)
    k = torch.zeros(1, 1, 3, 2)
    with pytest.raises(AssertionError):
        ring.store(k, k, torch.tensor([[False, True, False]]))
    with pytest.raises(AssertionError):
        ring.store(k, k, torch.tensor([[True, False, True]]))


def test_ages_and_landmark_positions_hand_worked():
    # five filled slots, next write at slot 2: slot 2 is the oldest block, slot 1 the newest
    assert mem_cache.slot_ages(5, 2).tolist() == [3, 4, 0, 1, 2]
    # top_k = 2: the two newest blocks (slots 0 and 1) sit at position slots 1 and 2, every other at 0
    assert mem_cache.landmark_slots(5, 2, 2).tolist() == [1, 2, 0, 0, 0]
    assert mem_cache.landmark_token_positions(5, 2, 2, 51).tolist() == [101, 152, 50, 50, 50]
    # a ring that has not wrapped: cache_iter == n, slots are in age order
    assert mem_cache.slot_ages(3, 3).tolist() == [0, 1, 2]
    assert mem_cache.landmark_slots(3, 3, 1).tolist() == [0, 0, 1]
    assert mem_cache.slot_ages(4, 0).tolist() == [0, 1, 2, 3]
    # picks [slot 1 (newest), slot 3 (age 1)] -> by age: slot 3 first; positions: old block at 0.., newest one block on
    slots = mem_cache.restore_order(torch.tensor([1, 3]), 5, 2)
    assert slots.tolist() == [3, 1]
    pos = mem_cache.gathered_key_positions(slots, 5, 2, 2, 3)
    assert pos.tolist() == [0, 1, 2, 6, 7, 8]
    pos = mem_cache.gathered_key_positions(torch.tensor([0, 1]), 5, 2, 2, 3)      # the two newest: both shifted
    assert pos.tolist() == [3, 4, 5, 6, 7, 8]


def test_restore_order_is_a_sort_by_age():
    for n, top_k in [(5, 2), (7, 3), (4, 4), (6, 1)]:
        for cache_iter in range(0, n + 1):
            if cache_iter == n and n > 0:
                ages = list(range(n))                    # not wrapped
            else:
                ages = mem_cache.slot_ages(n, cache_iter).tolist()
            for pick in itertools.permutations(range(n), top_k):
                got = mem_cache.restore_order(torch.tensor(pick), n, cache_iter).tolist()
                want = sorted(pick, key=lambda s: ages[s]) if top_k > 1 else list(pick)
                assert got == want, (n, cache_iter, pick)


def _ring_and_flat(n, cache_iter, block, B, nh, hs, seed, dtype=torch.bfloat16):
    """A filled ring (capacity n) and the same blocks laid out oldest first as a flat (B,nh,S,hs) cache."""
    g = torch.Generator().manual_seed(seed)
    cache_k = torch.randn(B, n, block, nh, hs, generator=g).to(dtype)
    ages = mem_cache.slot_ages(n, cache_iter)
    flat = torch.empty(B, nh, n * block, hs, dtype=dtype)
    for slot in range(n):
        a = int(ages[slot])
        flat[:, :, a * block:(a + 1) * block] = cache_k[:, slot].permute(0, 2, 1, 3)
    return cache_k, flat, ages


@pytest.mark.parametrize("n,cache_iter,top_k", [(6, 2, 2), (9, 0, 3), (5, 4, 1), (8, 5, 4), (3, 1, 3)])
def test_ring_selection_equals_flat_selection_in_age_order(n, cache_iter, top_k):
    B, nh, T, hs, block = 2, 3, 5, 64, 4
    cache_k, flat, ages = _ring_and_flat(n, cache_iter, block, B, nh, hs, seed=n * 10 + cache_iter)
    q = torch.randn(B, nh, T, hs, generator=torch.Generator().manual_seed(7)).bfloat16()
    cos, sin = rotary.rotary_tables(64, hs, torch.bfloat16)
    sc_ring = mem_cache.ring_scores(q, cache_k, n, cache_iter, top_k, cos, sin)
    # the flat-cache oracle rotates at slot*block + block-1 + prefix_len; the ring uses prefix_len = 0, so shift the
    # tables by the flat cache's prefix_len (which may be negative by one block when top_k == n)
    geo = retrieval.retrieval_geometry(n * block, block, top_k)
    pre = geo["prefix_len"]
    pos = torch.arange(64 + max(pre, 0)) - pre
    cos_s, sin_s = rotary.rotary_tables(64 + 2 * abs(pre) + block, hs, torch.bfloat16)
    sc_flat = retrieval.landmark_scores(q, flat, cos_s[pos.clamp(min=0)], sin_s[pos.clamp(min=0)], block, top_k)
    assert torch.equal(sc_ring[..., :], sc_flat[..., ages])                  # same numbers, slot order vs age order
    slots = mem_cache.select_blocks(sc_ring, cache_iter, top_k, "per_token_and_head")
    flat_idx = retrieval.select_topk(sc_flat, top_k)                          # ascending age
    ties = retrieval.boundary_tie_rows(sc_flat, top_k) | _any_tie_among_top(sc_flat, top_k)
    assert torch.equal(ages[slots][~ties], flat_idx[~ties])
    assert (~ties).any()


def _any_tie_among_top(scores, k):
    top = torch.sort(scores.float(), dim=-1, descending=True).values[..., :k + 1]
    return (top[..., 1:] == top[..., :-1]).any(-1)


@pytest.mark.parametrize("method", mem_cache.METHODS)
def test_aggregations_against_literal_loops_and_topk(method):
    B, nh, T, n, top_k, cache_iter = 2, 3, 4, 7, 3, 3
    g = torch.Generator().manual_seed(5)
    scores = (torch.randn(B, nh, T, n, generator=g) * 2).bfloat16()
    prob = retrieval.softmax_contract(scores, torch.float32)
    ref = torch.softmax(scores.float(), dim=-1)
    assert (prob - ref).abs().max() < 1e-6
    agg = mem_cache.block_probabilities(scores, method)
    for b, h, t, m in itertools.product(range(B), range(nh), range(T), range(n)):
        if method == "max_over_heads":
            want = max(prob[b, x, t, m] for x in range(nh))
        elif method == "max_over_tokens":
            want = max(prob[b, h, x, m] for x in range(T))
        else:
            want = prob[b, h, t, m]
        assert agg[b, h, t, m] == want
    slots = mem_cache.select_blocks(scores, cache_iter, top_k, method)
    ties = mem_cache.boundary_tie_rows(scores, top_k, method)
    lib = agg.topk(top_k, dim=-1).indices                                     # mem_cache.py:72
    ages = mem_cache.slot_ages(n, cache_iter)
    assert torch.equal(slots.sort(-1).values[~ties], lib.sort(-1).values[~ties])      # same set of blocks
    a = ages[slots]
    assert (a[..., 1:] > a[..., :-1]).all()                                   # oldest first
    if method == "max_over_heads":
        assert (slots == slots[:, :1]).all()
    if method == "max_over_tokens":
        assert (slots == slots[:, :, :1]).all()
    with pytest.raises(NotImplementedError):
        mem_cache.block_probabilities(scores, "mean")


def test_interleaved_rotary_is_the_half_split_one_on_permuted_head_dims():
    # the benchmark rotates pairs (2i, 2i+1) (rotary_utils.py:17-31, rotary.py:27-37); the kernels' tables
    # rotate pairs (i, i + hs/2).  Moving the even dims in front of the odd ones turns one into the other.
    hs, n_pos = 16, 40
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, hs, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 20, 39])
    freqs = 10.0 ** (-4 * torch.arange(0, hs, 2, dtype=torch.float64) / hs)          # rotary.py:49
    ang = (pos[:, None] * freqs[None]).repeat_interleave(2, dim=-1)                   # each angle for its pair
    pairs = x.view(5, hs // 2, 2)
    rot_half = torch.stack((-pairs[..., 1], pairs[..., 0]), dim=-1).view(5, hs)
    inter = x * ang.cos() + rot_half * ang.sin()
    perm = torch.cat((torch.arange(0, hs, 2), torch.arange(1, hs, 2)))
    ang_split = torch.cat((pos[:, None] * freqs[None],) * 2, dim=-1)
    split = x[:, perm] * ang_split.cos() + rotary.rotate_half(x[:, perm]) * ang_split.sin()
    assert torch.allclose(inter[:, perm], split, atol=1e-12)
    y = torch.randn(5, hs, generator=g, dtype=torch.float64)
    assert torch.allclose((inter * y).sum(-1), (split * y[:, perm]).sum(-1), atol=1e-12)


# ---------------------------------------------------------------- gather + attend (mem_cache.py:86-109)
def _filled_ring(B, nh, hs, block, capacity, n_tokens, g, dtype=torch.float64):
    ring = mem_cache.RingStore(B, capacity, block, nh, hs, dtype=dtype)
    k = torch.randn(B, nh, n_tokens, hs, generator=g, dtype=dtype) * 0.5
    v = torch.randn(B, nh, n_tokens, hs, generator=g, dtype=dtype) * 0.5
    im = (torch.arange(n_tokens) % block == block - 1)[None].expand(B, n_tokens)
    ring.store(k, v, im)
    return ring


def _tables64(n_pos, hs):
    inv = 1.0 / (10000.0 ** (torch.arange(0, hs, 2, dtype=torch.float64) / hs))
    ang = torch.outer(torch.arange(n_pos, dtype=torch.float64), inv)
    ang = torch.cat((ang, ang), -1)
    return ang.cos(), ang.sin()


@pytest.mark.parametrize("method", mem_cache.METHODS)
@pytest.mark.parametrize("capacity,block,n_tokens,top_k,T", [
    (6, 5, 5 * 4 + 2, 2, 9),       # not yet full, tail of 2, chunk over two landmarks
    (4, 5, 5 * 7 + 3, 3, 4),       # wrapped ring (oldest block at slot 3), chunk completes the tail's block exactly... minus one
    (4, 7, 7 * 9, 2, 15),          # no tail, chunk of two blocks and one token
    (5, 4, 4 * 6 + 1, 5, 6),       # top_k = filled slots
])
def test_attention_with_cache_is_the_closed_form_over_picked_blocks_tail_and_chunk(method, capacity, block, n_tokens, top_k, T):
    # the picked blocks, rotated at k_indices, are earlier landmark blocks in front of [tail ; chunk]; zero rows stand
    # in for the tail's queries.  float64, so only the mathematics is compared.
    from oracle import s1
    B, nh, hs = 2, 3, 8
    g = torch.Generator().manual_seed(capacity * 31 + block + top_k)
    ring = _filled_ring(B, nh, hs, block, capacity, n_tokens, g)
    tail, n = ring.last_incomplete_len, ring.filled
    start = (top_k + 1) * block + tail
    cos, sin = _tables64(start + T, hs)
    q0 = torch.randn(B, nh, T, hs, generator=g, dtype=torch.float64)
    k0 = torch.randn(B, nh, T, hs, generator=g, dtype=torch.float64)
    v = torch.randn(B, nh, T, hs, generator=g, dtype=torch.float64)
    pos = torch.arange(start, start + T)
    q, k = rotary.apply_rotary(q0, cos, sin, pos), rotary.apply_rotary(k0, cos, sin, pos)
    is_mem = ((torch.arange(T) + tail) % block == block - 1)[None].expand(B, T)
    y, slots = mem_cache.attention_with_cache(ring, q, k, v, is_mem, cos, sin, top_k, method, start, n_buckets=top_k + T // block + 3)
    assert slots.shape == (B, nh, T, top_k)
    tail_k = rotary.apply_rotary(ring.pending_k, cos, sin, torch.arange(start - tail, start))
    newest = mem_cache.slot_ages(n, ring.cache_iter) >= n - top_k
    for b, h, t in itertools.product(range(B), range(nh), range(T)):
        ks, vs = [], []
        for j, slot in enumerate(slots[b, h, t].tolist()):
            p0 = j * block + (block if newest[slot] else 0)
            ks.append(rotary.apply_rotary(ring.cache_k[b, slot, :, h], cos, sin, torch.arange(p0, p0 + block)))
            vs.append(ring.cache_v[b, slot, :, h])
        kk = torch.cat(ks + [tail_k[b, h], k[b, h]])
        vv = torch.cat(vs + [ring.pending_v[b, h], v[b, h]])
        qq = torch.cat((torch.zeros(tail, hs, dtype=torch.float64), q[b, h]))
        want = s1.s1_attention(qq, kk, vv, block, rows=[tail + t])[0]
        assert torch.allclose(y[b, h, t], want, atol=1e-12), (b, h, t)


def test_ring_attention_equals_the_flat_cache_step_on_the_same_blocks():
    # llama flavour (oracle/retrieval.py, llama_mem.py:386-477) on the ring's blocks laid out oldest first, with the
    # ring's picks translated to ages: positions differ by a constant (prefix_len), which rotary does not see
    B, nh, hs, block, capacity, top_k, T = 1, 2, 8, 6, 5, 2, 3
    g = torch.Generator().manual_seed(5)
    ring = _filled_ring(B, nh, hs, block, capacity, block * 8 + 2, g)          # wrapped, tail of 2; T + tail <= block
    tail, n = ring.last_incomplete_len, ring.filled
    ages = mem_cache.slot_ages(n, ring.cache_iter)
    order = torch.argsort(ages)                                                  # slots, oldest first
    flat_k = torch.cat([ring.cache_k[:, s].permute(0, 2, 1, 3) for s in order.tolist()] + [ring.pending_k], dim=2)
    flat_v = torch.cat([ring.cache_v[:, s].permute(0, 2, 1, 3) for s in order.tolist()] + [ring.pending_v], dim=2)
    S = flat_k.shape[2]
    cos, sin = _tables64(S + T, hs)
    q0 = torch.randn(B, nh, T, hs, generator=g, dtype=torch.float64)
    k0 = torch.randn(B, nh, T, hs, generator=g, dtype=torch.float64)
    v = torch.randn(B, nh, T, hs, generator=g, dtype=torch.float64)
    is_mem = ((torch.arange(T) + tail) % block == block - 1)[None].expand(B, T)
    start = (top_k + 1) * block + tail
    q_ring = rotary.apply_rotary(q0, cos, sin, torch.arange(start, start + T))
    k_ring = rotary.apply_rotary(k0, cos, sin, torch.arange(start, start + T))
    slots = torch.randint(0, n, (B, nh, T, 1), generator=g)
    slots = torch.cat((slots, (slots + 1 + torch.randint(0, n - 1, (B, nh, T, 1), generator=g)) % n), -1)   # two distinct slots
    slots = mem_cache.restore_order(slots, n, ring.cache_iter)
    y, _ = mem_cache.attention_with_cache(ring, q_ring, k_ring, v, is_mem, cos, sin, top_k, "per_token_and_head", start,
                                          n_buckets=top_k + 3, slots=slots)
    q_flat = rotary.apply_rotary(q0, cos, sin, torch.arange(S, S + T))
    k_flat = rotary.apply_rotary(k0, cos, sin, torch.arange(S, S + T))
    want, _ = retrieval.retrieve_and_attend(q_flat, flat_k, flat_v, k_flat, v, is_mem, cos, sin, block, top_k,
                                            idx=ages[slots], n_buckets=top_k + 3)
    assert torch.allclose(y, want, atol=1e-11)


def test_without_blocks_only_the_tail_joins_the_chunk():
    from oracle import s1
    B, nh, hs, block, T = 1, 2, 8, 5, 7
    g = torch.Generator().manual_seed(9)
    ring = _filled_ring(B, nh, hs, block, 4, 3, g)                               # three tokens, no complete block
    assert ring.filled == 0 and ring.last_incomplete_len == 3
    cos, sin = _tables64(64, hs)
    q, k, v = (torch.randn(B, nh, T, hs, generator=g, dtype=torch.float64) for _ in range(3))
    is_mem = ((torch.arange(T) + 3) % block == block - 1)[None]
    y, slots = mem_cache.attention_with_cache(ring, q, k, v, is_mem, cos, sin, 2, "per_token_and_head", 3, n_buckets=8)
    assert slots is None
    tail_k = rotary.apply_rotary(ring.pending_k, cos, sin, torch.arange(0, 3))
    for h in range(nh):
        qq = torch.cat((torch.zeros(3, hs, dtype=torch.float64), q[0, h]))
        want = s1.s1_attention(qq, torch.cat((tail_k[0, h], k[0, h])), torch.cat((ring.pending_v[0, h], v[0, h])), block)[3:]
        assert torch.allclose(y[0, h], want, atol=1e-12)


def test_per_token_and_head_orders_underflowed_probabilities_by_score():
    # scores so far below the row maximum that their fp32 probabilities are all 0: the pick follows the scores
    # (-150 before -200 before -300), not the slot numbers a tie on the probabilities would fall back to
    scores = torch.tensor([0.0, -200.0, -150.0, -300.0]).bfloat16().view(1, 1, 1, 4)
    prob = mem_cache.block_probabilities(scores, "per_token_and_head")
    assert prob[0, 0, 0, 1:].tolist() == [0.0, 0.0, 0.0]
    assert mem_cache.select_blocks(scores, 0, 2, "per_token_and_head").flatten().tolist() == [0, 2]
    assert mem_cache.select_blocks(scores, 0, 3, "per_token_and_head").flatten().tolist() == [0, 1, 2]
    # the aggregated methods do rank probabilities: equal ones fall back to the lower slot
    assert mem_cache.select_blocks(scores, 0, 2, "max_over_tokens").flatten().tolist() == [0, 1]
