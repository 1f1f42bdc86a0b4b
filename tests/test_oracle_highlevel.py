"""The scatter/gather restatement and the closed form are two independently
written statements of the same mathematics; they must agree."""
import math

import pytest
import torch

from oracle import highlevel, s1


def _rand(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


@pytest.mark.parametrize("lq,lk,block", [(24, 24, 8), (16, 32, 8), (32, 32, 4), (20, 20, 8)])
def test_fixed_stride_case_equals_closed_form(lq, lk, block):
    q, k, v = _rand(2, 2, lq, 8, seed=1), _rand(2, 2, lk, 8, seed=2), _rand(2, 2, lk, 8, seed=3)
    a = highlevel.attention_fixed_stride(q, k, v, block)
    b = s1.s1_attention(q, k, v, block)
    assert torch.isfinite(a).all()
    assert torch.allclose(a, b, atol=1e-12)


def test_fixed_stride_with_exactly_as_many_buckets_as_blocks():
    # the llama flavour fixes 64 buckets (llama_mem.py:228); 64 blocks just fit.
    block, nb = 4, 6
    L = block * nb
    q, k, v = _rand(1, 1, L, 4, seed=4), _rand(1, 1, L, 4, seed=5), _rand(1, 1, L, 4, seed=6)
    a = highlevel.attention_fixed_stride(q, k, v, block, n_buckets=nb)
    assert torch.allclose(a, s1.s1_attention(q, k, v, block), atol=1e-12)


def test_lm_benchmark_flavour_equals_closed_form():
    # benchmark config 0 in miniature: landmark after every `mem_freq` tokens.
    B, H, T, d, block = 2, 2, 40, 8, 5
    q, k, v = _rand(B, H, T, d, seed=7), _rand(B, H, T, d, seed=8), _rand(B, H, T, d, seed=9)
    is_mem = (torch.arange(T) % block == block - 1)[None].expand(B, T)
    a = highlevel.attention_lm_benchmark(q, k, v, is_mem, n_buckets=T // block + 3)
    assert torch.allclose(a, s1.s1_attention(q, k, v, block), atol=1e-12)


def test_gradients_through_restatement_equal_closed_form():
    block = 4
    q, k, v = _rand(1, 2, 16, 8, seed=10), _rand(1, 2, 16, 8, seed=11), _rand(1, 2, 16, 8, seed=12)
    do = _rand(1, 2, 16, 8, seed=13)
    grads = []
    for fn in (lambda a, b, c: highlevel.attention_fixed_stride(a, b, c, block),
               lambda a, b, c: s1.s1_attention(a, b, c, block)):
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        grads.append(torch.autograd.grad((fn(qq, kk, vv) * do).sum(), [qq, kk, vv]))
    for a, b in zip(*grads):
        assert torch.allclose(a, b, atol=1e-12)


def test_irregular_landmarks_row_sums_and_block_structure():
    # lm_benchmark allows arbitrary landmark positions; rows must still be distributions,
    # and a row in the first section must be plain causal softmax over non-landmark keys.
    B, H, T, d = 1, 1, 12, 4
    q, k = _rand(B, H, T, d, seed=14), _rand(B, H, T, d, seed=15)
    is_mem = torch.zeros(B, T, dtype=torch.bool)
    is_mem[0, [2, 6, 9]] = True          # no two adjacent: an empty block would swallow its landmark's mass
    w = highlevel.attention_lm_benchmark(q, k, torch.eye(T, dtype=torch.float64)[None, None], is_mem, n_buckets=8)
    assert torch.allclose(w.sum(-1), torch.ones(B, H, T, dtype=torch.float64), atol=1e-12)
    s = (q[0, 0, 1] @ k[0, 0, :2].T) / math.sqrt(d)
    assert torch.allclose(w[0, 0, 1, :2], torch.softmax(s, 0), atol=1e-12)
    assert (w[0, 0][:, is_mem[0]] == 0).all()         # landmark columns never carry weight


def test_benchmark_config0_full_size_restatement_equals_closed_form():
    # benchmark config 0 as specified: B2 H8 L510 D128, a landmark at every 51st position, fp32, seed 0,
    # scale 1/sqrt(128); the lm_benchmark flavour with its default 16 buckets (10 blocks need 11) against the
    # closed form.  This is the workload bench.py's CPU baseline times.
    from bench import config0_inputs
    q, k, v, is_mem, block = config0_inputs(0)
    assert q.shape == (2, 8, 510, 128) and q.dtype == torch.float32 and block == 51
    assert is_mem.sum().item() == 2 * 10 and bool(is_mem[0, 50]) and not bool(is_mem[0, 49])
    a = highlevel.attention_lm_benchmark(q, k, v, is_mem, n_buckets=16)
    b = s1.s1_attention(q, k, v, block)
    assert torch.isfinite(a).all()
    assert (a - b).abs().max().item() <= 2e-5
    # and in float64, where both are exact to rounding
    a64 = highlevel.attention_lm_benchmark(q.double(), k.double(), v.double(), is_mem, n_buckets=16)
    assert (a64 - s1.s1_attention(q.double(), k.double(), v.double(), block)).abs().max().item() <= 1e-12
    assert (a64 - a).abs().max().item() <= 2e-5


def test_group_dropout_scales_earlier_blocks_and_leaves_the_landmark_softmax_alone():
    # landmark.py:110-113 with the dropout's outcome supplied as a factor per (row, block): the restated bucketed
    # softmax, the closed form, and the plain statement "weights of a block's normal keys times its factor, every
    # other weight unchanged" must agree (fp64)
    import math
    from oracle import highlevel, s1
    torch.manual_seed(0)
    B, H, L, D, block = 1, 2, 35, 8, 7
    nb = L // block
    q, k, v = (torch.randn(B, H, L, D, dtype=torch.float64) for _ in range(3))
    p_drop = 0.4
    keep = torch.nn.functional.dropout(torch.ones(B, H, nb, L, dtype=torch.float64), p_drop)     # {0, 1/(1-p)}
    assert set(keep.unique().tolist()) <= {0.0, 1.0 / (1.0 - p_drop)} and (keep == 0).any() and (keep > 0).any()
    w_plain, _, _ = s1.s1_weights(q, k, block)
    w_drop, L_drop, M_drop = s1.s1_weights(q, k, block, group_scale=keep)
    # plain statement: key j of an earlier block b (not its landmark) gets factor keep[b, i]; everything else stays
    j = torch.arange(L)
    i = torch.arange(L)
    earlier_normal = ((j // block)[None, :] < (i // block)[:, None]) & ((j % block) != block - 1)[None, :]
    per_key = keep.transpose(-1, -2)[..., j // block]                                   # (B, H, i, j)
    want = torch.where(earlier_normal, w_plain * per_key, w_plain)
    assert torch.allclose(w_drop, want, atol=1e-14)
    _, L_plain, M_plain = s1.s1_weights(q, k, block)
    assert torch.equal(L_drop, L_plain) and torch.equal(M_drop, M_plain)                # the global bucket is untouched
    # the restated high-level path with the same outcome of the dropout
    att = (q @ k.transpose(-2, -1)) / math.sqrt(D)
    causal_masked = ~torch.tril(torch.ones(L, L, dtype=torch.bool))[None, None].expand(B, H, L, L)
    att = att.masked_fill(causal_masked, float("-inf"))
    is_mem = (j % block == block - 1)[None].expand(B, L)
    masked, im, ls = highlevel.masks_from_is_mem(is_mem[:, None, None, :], causal_masked)
    att = att.masked_fill(masked, float("-inf"))
    n_buckets = nb + 3
    keep_b = torch.ones(B, H, L, n_buckets, dtype=torch.float64)
    keep_b[..., :nb] = keep.transpose(-1, -2)
    w_high = highlevel.grouped_softmax(att, im, ls, n_buckets, attn_mask=masked, guard_empty=True, group_keep=keep_b)
    assert torch.allclose(w_high, w_drop, atol=1e-14)


def _irregular_mask(T, seed, tail):
    """Landmarks at irregular positions, never two in a row; `tail` tokens without a landmark at the end."""
    g = torch.Generator().manual_seed(seed)
    marks, j = [False] * T, 0
    while True:
        j += int(torch.randint(2, 7, (1,), generator=g))
        if j >= T - tail:
            break
        marks[j - 1] = True
    if tail == 0:
        marks[T - 1] = True
        if T >= 2 and marks[T - 2]:
            marks[T - 2] = False
    return torch.tensor(marks)


@pytest.mark.parametrize("T,tail,seed", [(23, 0, 1), (23, 3, 2), (40, 1, 3), (9, 0, 4)])
def test_irregular_landmarks_equal_the_row_by_row_evaluation(T, tail, seed):
    # the restatement of the reference's scatter/gather grouped softmax against a literal per-row loop that
    # shares no code with it: blocks of unequal length, with and without a trailing block without landmark
    d = 5
    q, k, v = _rand(1, 1, T, d, seed=20 + seed), _rand(1, 1, T, d, seed=30 + seed), _rand(1, 1, T, d, seed=40 + seed)
    is_mem = _irregular_mask(T, seed, tail)
    got = highlevel.attention_lm_benchmark(q, k, v, is_mem[None], n_buckets=int(is_mem.sum()) + 3)
    want = torch.tensor(s1.s1_rows_python_irregular(q[0, 0], k[0, 0], v[0, 0], is_mem.tolist()), dtype=torch.float64)
    assert torch.allclose(got[0, 0], want, atol=1e-12)


def test_row_by_row_evaluation_for_irregular_landmarks_reduces_to_the_regular_one():
    T, d, block = 24, 4, 6
    q, k, v = _rand(1, 1, 12, d, seed=51)[0, 0], _rand(1, 1, T, d, seed=52)[0, 0], _rand(1, 1, T, d, seed=53)[0, 0]
    is_mem = [(j % block) == block - 1 for j in range(T)]
    want, _, _ = s1.s1_rows_python(q, k, v, block)
    got = s1.s1_rows_python_irregular(q, k, v, is_mem)
    assert torch.allclose(torch.tensor(got), torch.tensor(want), atol=1e-13)
