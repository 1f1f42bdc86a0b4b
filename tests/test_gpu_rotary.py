"""Rotary embedding kernel against the oracle and against torch's own 16-bit elementwise arithmetic:
bit for bit (llama/llama_mem.py:127-149)."""
import pytest
import torch

from oracle import rotary as orot

pytestmark = pytest.mark.gpu


def _case(B, H, L, D, dtype, seed, n_pos=None):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, L, D, generator=g).to(dtype)
    k = torch.randn(B, H, L, D, generator=g).to(dtype)
    n_pos = n_pos or 4 * L + 7
    cos, sin = orot.rotary_tables(n_pos, D, dtype)
    return q, k, cos, sin, n_pos, g


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,L,D", [(2, 3, 70, 128), (1, 2, 33, 64), (3, 1, 1, 128)])
def test_rotary_bit_exact_against_oracle_and_torch_arithmetic(B, H, L, D, dtype):
    from landmark_hip.rotary import apply_rotary_pos_emb
    print(f"case B{B} H{H} L{L} D{D} {dtype}", flush=True)
    q, k, cos, sin, n_pos, g = _case(B, H, L, D, dtype, seed=B * 100 + L)
    pos = torch.randint(0, n_pos, (B, L), generator=g)
    want_q = orot.apply_rotary(q, cos, sin, pos[:, None, :])
    want_k = orot.apply_rotary(k, cos, sin, pos[:, None, :])
    # the reference's expression evaluated by torch in the model dtype (one rounding per elementwise op)
    c, s = cos[pos].unsqueeze(1), sin[pos].unsqueeze(1)
    assert torch.equal(want_k, (k * c) + (orot.rotate_half(k) * s))
    dev = lambda t: t.cuda()
    gq, gk = apply_rotary_pos_emb(dev(q), dev(k), dev(cos)[None, None], dev(sin)[None, None], dev(pos))
    torch.cuda.synchronize()
    assert torch.equal(gq.cpu(), want_q) and torch.equal(gk.cpu(), want_k)
    # q is optional (llama_mem.py:143-144); one row of positions serves the whole batch
    row = pos[:1]
    none_q, gk1 = apply_rotary_pos_emb(None, dev(k), dev(cos), dev(sin), dev(row))
    assert none_q is None and torch.equal(gk1.cpu(), orot.apply_rotary(k, cos, sin, row[:, None, :]))


def test_rotary_on_projection_layout_and_in_place():
    # (B, L, H, D) memory viewed as (B, H, L, D), as the projections leave it (llama_mem.py:287-289)
    from landmark_hip import _lib
    from landmark_hip.rotary import apply_rotary_pos_emb
    B, H, L, D = 2, 4, 50, 128
    q, k, cos, sin, n_pos, g = _case(B, H, L, D, torch.bfloat16, seed=5)
    pos = torch.arange(13, 13 + L)[None].expand(B, L).contiguous()
    kd = k.permute(0, 2, 1, 3).contiguous().cuda().permute(0, 2, 1, 3)
    assert not kd.is_contiguous()
    _, gk = apply_rotary_pos_emb(None, kd, cos.cuda(), sin.cuda(), pos.cuda())
    want = orot.apply_rotary(k, cos, sin, pos[:, None, :])
    assert gk.stride() == kd.stride() and torch.equal(gk.cpu(), want)
    # out aliasing x through the C ABI
    x = k.cuda()
    cd, sd, pd = cos.cuda(), sin.cuda(), pos.cuda()
    _lib.check(_lib.lib().lmk_apply_rotary(_lib.tensor4(x), _lib.tensor4(x), cd.data_ptr(), sd.data_ptr(), cd.stride(0),
                                           cd.shape[0], pd.data_ptr(), L, B, H, L, D, 0, _lib.current_stream(x.device)))
    torch.cuda.synchronize()
    assert torch.equal(x.cpu(), want)


def test_rotary_feeds_the_fused_attention_like_the_reference_layer():
    # the layer's order of operations (llama_mem.py:287-298, 441-446): rotate q and k, then fused attention
    from landmark_hip.rotary import apply_rotary_pos_emb
    from ltriton.flash_landmark_attention import fused_landmark_attention
    from oracle import s1
    B, H, L, D, block = 1, 2, 96, 128, 32
    q, k, cos, sin, n_pos, g = _case(B, H, L, D, torch.bfloat16, seed=9, n_pos=L)
    q, k = q * 0.5, k * 0.5
    v = (torch.randn(B, H, L, D, generator=g) * 0.5).bfloat16()
    pos = torch.arange(L)[None]
    qr, kr = apply_rotary_pos_emb(q.cuda(), k.cuda(), cos.cuda(), sin.cuda(), pos.cuda())
    is_mem = (torch.arange(L) % block == block - 1)[None].cuda()
    out = fused_landmark_attention(qr, kr, v.cuda(), is_mem, block_size=block)
    pq, pk = orot.apply_rotary(q, cos, sin, pos[:, None, :]), orot.apply_rotary(k, cos, sin, pos[:, None, :])
    for h in range(H):
        ref = s1.s1_attention(pq[0, h].float(), pk[0, h].float(), v[0, h].float(), block)
        assert (out[0, h].float().cpu() - ref).abs().max().item() <= 2e-2


@pytest.mark.parametrize("B,H,Lq,Lk,D,block,dtype", [
    (2, 3, 128, 128, 128, 32, torch.bfloat16),
    (1, 2, 96, 224, 128, 32, torch.bfloat16),       # history: the queries sit at positions 128 ..
    (2, 2, 128, 256, 64, 64, torch.float16),
    (1, 2, 256, 256, 128, 128, torch.bfloat16),
    (1, 2, 70, 70, 64, 32, torch.bfloat16),         # partial last block
])
def test_forward_with_q_rotated_in_the_prologue_is_bit_identical(B, H, Lq, Lk, D, block, dtype):
    # lmk_attn_fwd_rotary_q == lmk_attn_fwd on apply_rotary_pos_emb(q): same output bits, one pass over q less
    from landmark_hip.attention import fused_landmark_attention_rotary_q
    from landmark_hip.rotary import apply_rotary_pos_emb
    from ltriton.flash_landmark_attention import fused_landmark_attention
    print(f"case rope-q B{B} H{H} Lq{Lq} Lk{Lk} D{D} bs{block} {dtype}", flush=True)
    g = torch.Generator().manual_seed(Lq + Lk + D)
    q = (torch.randn(B, H, Lq, D, generator=g) * 0.5).to(dtype).cuda()
    k = (torch.randn(B, H, Lk, D, generator=g) * 0.5).to(dtype).cuda()
    v = (torch.randn(B, H, Lk, D, generator=g) * 0.5).to(dtype).cuda()
    cos, sin = (t.cuda() for t in orot.rotary_tables(Lk + 40, D, dtype))
    pos_q = (torch.arange(Lk - Lq, Lk)[None] + torch.tensor([[0], [7]])[:B]).cuda()      # per-batch offsets
    pos_k = (torch.arange(Lk)[None] + torch.tensor([[0], [7]])[:B]).cuda()
    q_rot, _ = apply_rotary_pos_emb(q, q, cos, sin, pos_q)
    _, k_rot = apply_rotary_pos_emb(None, k, cos, sin, pos_k)
    want = fused_landmark_attention(q_rot, k_rot, v, None, block_size=block)
    got = fused_landmark_attention_rotary_q(q, k_rot, v, cos, sin, pos_q, block_size=block)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # and against the oracle, end to end
    ref = orot.apply_rotary(q.cpu(), cos.cpu(), sin.cpu(), pos_q.cpu()[:, None, :])
    assert torch.equal(q_rot.cpu(), ref)
    with pytest.raises(AssertionError):
        fused_landmark_attention_rotary_q(q.clone().requires_grad_(True), k_rot, v, cos, sin, pos_q, block_size=block)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,L,D,share_pos", [(2, 3, 70, 128, False), (1, 2, 33, 64, True)])
def test_rotary_gradients_match_torch_autograd_of_the_reference_expression(B, H, L, D, share_pos, dtype):
    # apply_rotary_pos_emb is differentiable in q and k (llama_mem.py:134-149 is plain torch arithmetic); the
    # gradient is the transposed rotation, through the same kernel.  Compared with torch's autograd through the
    # reference expression evaluated in the model dtype on the CPU: one rounding per elementwise operation on
    # both sides, so bit for bit.
    from landmark_hip.rotary import apply_rotary_pos_emb
    print(f"case grad B{B} H{H} L{L} D{D} {dtype}", flush=True)
    q, k, cos, sin, n_pos, g = _case(B, H, L, D, dtype, seed=B * 10 + L)
    pos = torch.randint(0, n_pos, (1 if share_pos else B, L), generator=g)
    dq = torch.randn(B, H, L, D, generator=g).to(dtype)
    dk = torch.randn(B, H, L, D, generator=g).to(dtype)
    qc, kc = q.clone().requires_grad_(True), k.clone().requires_grad_(True)
    c, s = cos[pos].unsqueeze(1), sin[pos].unsqueeze(1)
    ref_q = (qc * c) + (orot.rotate_half(qc) * s)
    ref_k = (kc * c) + (orot.rotate_half(kc) * s)
    want_q, want_k = torch.autograd.grad([ref_q, ref_k], [qc, kc], [dq, dk])
    qd, kd = q.cuda().requires_grad_(True), k.cuda().requires_grad_(True)
    out_q, out_k = apply_rotary_pos_emb(qd, kd, cos.cuda(), sin.cuda(), pos.cuda())
    assert out_q.requires_grad and out_k.requires_grad
    got_q, got_k = torch.autograd.grad([out_q, out_k], [qd, kd], [dq.cuda(), dk.cuda()])
    torch.cuda.synchronize()
    assert torch.equal(got_q.cpu(), want_q) and torch.equal(got_k.cpu(), want_k)
    # k alone (q is None), and through the fused attention: the gradient reaches the un-rotated projections
    kd2 = k.cuda().requires_grad_(True)
    _, only_k = apply_rotary_pos_emb(None, kd2, cos.cuda(), sin.cuda(), pos.cuda())
    (g2,) = torch.autograd.grad(only_k, kd2, dk.cuda())
    assert torch.equal(g2.cpu(), want_k)


def test_rotary_q_forward_rejects_block_sizes_it_is_not_built_for():
    # lmk_attn_fwd_rotary_q serves the native block sizes (32, 64, 128); other sizes rotate q with
    # apply_rotary_pos_emb and call fused_landmark_attention
    from landmark_hip.attention import fused_landmark_attention_rotary_q
    B, H, L, D, block = 1, 2, 102, 128, 51
    q, k, v = (torch.zeros(B, H, L, D, dtype=torch.bfloat16, device="cuda") for _ in range(3))
    cos, sin = (t.cuda() for t in orot.rotary_tables(L, D, torch.bfloat16))
    pos = torch.arange(L, device="cuda")[None]
    with pytest.raises(AssertionError):
        fused_landmark_attention_rotary_q(q, k, v, cos, sin, pos, block_size=block)
