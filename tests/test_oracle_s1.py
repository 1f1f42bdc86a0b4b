"""Pins oracle/s1.py by mathematics (the reference holds no golden vectors)."""
import math

import pytest
import torch

from oracle import s1

torch.manual_seed(0)


def _rand(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


@pytest.mark.parametrize("lq,lk,block,d", [(12, 12, 4, 8), (8, 16, 4, 4), (11, 11, 4, 8), (6, 14, 4, 8), (16, 16, 8, 4)])
def test_vectorised_equals_python_rows(lq, lk, block, d):
    q, k, v = _rand(lq, d, seed=1), _rand(lk, d, seed=2), _rand(lk, d, seed=3)
    o_ref, l_ref, m_ref = s1.s1_rows_python(q.tolist(), k.tolist(), v.tolist(), block)
    o, L, M = s1.s1_attention(q, k, v, block, return_stats=True)
    assert torch.allclose(o, torch.tensor(o_ref, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(L, torch.tensor(l_ref, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(M, torch.tensor(m_ref, dtype=torch.float64), atol=1e-12)


def test_rows_subset_matches_full():
    q, k, v = _rand(2, 3, 24, 8, seed=4), _rand(2, 3, 40, 8, seed=5), _rand(2, 3, 40, 8, seed=6)
    full = s1.s1_attention(q, k, v, 8)
    rows = [0, 7, 8, 15, 23]
    part = s1.s1_attention(q, k, v, 8, rows=rows)
    assert torch.equal(part, full[..., rows, :])


def test_first_block_is_textbook_causal_attention():
    # block 0 has no earlier landmarks: rows 0..bs-2 are plain causal softmax attention,
    # and the landmark row sees exactly what the row above it sees.
    bs, d = 16, 8
    q, k, v = _rand(1, 2, bs, d, seed=7), _rand(1, 2, bs, d, seed=8), _rand(1, 2, bs, d, seed=9)
    out = s1.s1_attention(q, k, v, bs)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert torch.allclose(out[..., : bs - 1, :], ref[..., : bs - 1, :], atol=1e-12)
    s = (q[..., bs - 1 :, :] @ k[..., : bs - 1, :].transpose(-1, -2)) / math.sqrt(d)
    assert torch.allclose(out[..., bs - 1 :, :], torch.softmax(s, -1) @ v[..., : bs - 1, :], atol=1e-12)


def test_weights_sum_to_one_and_v_ones():
    q, k = _rand(2, 2, 32, 8, seed=10), _rand(2, 2, 48, 8, seed=11)
    w, L, M = s1.s1_weights(q, k, 8)
    assert torch.allclose(w.sum(-1), torch.ones_like(w.sum(-1)), atol=1e-12)
    assert (w >= 0).all()
    out = s1.s1_attention(q, k, torch.ones(2, 2, 48, 8, dtype=torch.float64), 8)
    assert torch.allclose(out, torch.ones_like(out), atol=1e-12)


def test_v_identity_recovers_weights():
    # the reference's own (disabled) check, test_flash_landmark_attention.py:141-143
    lk = 16
    q, k = _rand(1, 1, 16, 8, seed=12), _rand(1, 1, lk, 8, seed=13)
    w, _, _ = s1.s1_weights(q, k, 4)
    out = s1.s1_attention(q, k, torch.eye(lk, dtype=torch.float64)[None, None], 4)
    assert torch.allclose(out, w, atol=1e-14)


def test_landmark_values_never_contribute():
    bs = 8
    q, k, v = _rand(1, 2, 32, 8, seed=14), _rand(1, 2, 32, 8, seed=15), _rand(1, 2, 32, 8, seed=16)
    v.requires_grad_(True)
    k.requires_grad_(True)
    out = s1.s1_attention(q, k, v, bs)
    v2 = v.detach().clone()
    v2[..., bs - 1 :: bs, :] += 100.0
    assert torch.equal(s1.s1_attention(q, k.detach(), v2, bs), out.detach())
    dk, dv = torch.autograd.grad(out.square().sum(), [k, v])
    assert torch.equal(dv[..., bs - 1 :: bs, :], torch.zeros_like(dv[..., bs - 1 :: bs, :]))
    # landmark keys do receive gradient (through the gates), except the last block's
    assert dk[..., bs - 1, :].abs().max() > 0
    assert torch.equal(dk[..., -1, :], torch.zeros_like(dk[..., -1, :]))


def test_permuting_normal_keys_inside_an_earlier_block():
    bs = 8
    q, k, v = _rand(1, 1, 24, 8, seed=17), _rand(1, 1, 24, 8, seed=18), _rand(1, 1, 24, 8, seed=19)
    perm = torch.arange(24)
    perm[:7] = torch.tensor([3, 0, 6, 1, 5, 2, 4])          # shuffle normals of block 0
    out = s1.s1_attention(q, k, v, bs)
    out_p = s1.s1_attention(q, k[..., perm, :], v[..., perm, :], bs)
    # rows of blocks 1,2 only see block 0 through its local softmax -> unchanged
    assert torch.allclose(out[..., 8:, :], out_p[..., 8:, :], atol=1e-13)


def test_two_block_closed_form_by_hand():
    # Lk = 2*bs, a row r in block 1 (not the landmark row):
    #   out = [ e^{s_lm0} * avg0 + sum_{j=bs..r} e^{s_j} v_j ] / [ e^{s_lm0} + sum_{j=bs..r} e^{s_j} ]
    #   avg0 = softmax(s_0..s_{bs-2}) . v_0..v_{bs-2}
    bs, d = 4, 4
    q, k, v = _rand(2 * bs, d, seed=20), _rand(2 * bs, d, seed=21), _rand(2 * bs, d, seed=22)
    out = s1.s1_attention(q, k, v, bs)
    for r in (4, 5, 6):
        s = (k @ q[r]) / math.sqrt(d)
        avg0 = torch.softmax(s[: bs - 1], 0) @ v[: bs - 1]
        e_lm = torch.exp(s[bs - 1])
        e_cur = torch.exp(s[bs : r + 1])
        expect = (e_lm * avg0 + e_cur @ v[bs : r + 1]) / (e_lm + e_cur.sum())
        assert torch.allclose(out[r], expect, atol=1e-13)
    # the landmark row of block 1 (r = 7) sees keys 4..6 of its own block
    s = (k @ q[7]) / math.sqrt(d)
    avg0 = torch.softmax(s[:3], 0) @ v[:3]
    e_lm, e_cur = torch.exp(s[3]), torch.exp(s[4:7])
    assert torch.allclose(out[7], (e_lm * avg0 + e_cur @ v[4:7]) / (e_lm + e_cur.sum()), atol=1e-13)


def test_history_prefix_equals_tail_of_full_problem():
    bs = 4
    q, k, v = _rand(1, 2, 16, 8, seed=23), _rand(1, 2, 16, 8, seed=24), _rand(1, 2, 16, 8, seed=25)
    full = s1.s1_attention(q, k, v, bs)
    tail = s1.s1_attention(q[..., 8:, :], k, v, bs)
    assert torch.allclose(tail, full[..., 8:, :], atol=1e-14)


def test_backward_formulas_equal_autograd_and_finite_differences():
    bs = 4
    q, k, v = _rand(1, 2, 8, 8, seed=26), _rand(1, 2, 12, 8, seed=27), _rand(1, 2, 12, 8, seed=28)
    do = _rand(1, 2, 8, 8, seed=29)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    out = s1.s1_attention(q, k, v, bs)
    gq, gk, gv = torch.autograd.grad((out * do).sum(), [q, k, v])
    dq, dk, dv = s1.s1_backward_formulas(q.detach(), k.detach(), v.detach(), do, bs)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert torch.allclose(a, b, atol=1e-12)
    # central finite differences on a few coordinates pin the sign/index conventions
    f = lambda q_, k_, v_: (s1.s1_attention(q_, k_, v_, bs) * do).sum()
    eps = 1e-6
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    for name, t, g in (("q", qd, gq), ("k", kd, gk), ("v", vd, gv)):
        for idx in [(0, 0, 1, 2), (0, 1, 3, 0), (0, 1, 7, 5)]:
            tp, tm = t.clone(), t.clone()
            tp[idx] += eps
            tm[idx] -= eps
            args_p = {"q": (tp, kd, vd), "k": (qd, tp, vd), "v": (qd, kd, tp)}[name]
            args_m = {"q": (tm, kd, vd), "k": (qd, tm, vd), "v": (qd, kd, tm)}[name]
            fd = (f(*args_p) - f(*args_m)) / (2 * eps)
            assert abs(fd - g[idx]) < 1e-6, (name, idx, fd, g[idx])


def test_fp32_large_block_matches_fp64():
    q, k, v = _rand(1, 2, 128, 64, seed=30), _rand(1, 2, 192, 64, seed=31), _rand(1, 2, 192, 64, seed=32)
    o64 = s1.s1_attention(q, k, v, 32)
    o32 = s1.s1_attention(q.float(), k.float(), v.float(), 32)
    assert (o64 - o32.double()).abs().max() < 1e-5
