"""Landmark blocks of any size up to 128 tokens (the training models use mem_freq + 1 = 51,
lm_benchmark/config/rotary.py:57): such a block is stored in 64 or 128 slots and the kernels mask the
slots in between.  Parity is against the same oracles as for the native block sizes, on the same
16-bit-rounded inputs, max abs error <= 2e-2; the repacking itself is bit-exact.
"""
import pytest
import torch

from tests.util import make_qkv, oracle_forward, oracle_grads

pytestmark = pytest.mark.gpu

TOL = 2e-2
DEV = "cuda:0"


def _expected_padded(x, bs, P):
    B, H, L, D = x.shape
    nb, rem = divmod(L, bs)
    out = torch.zeros(B, H, nb * P + rem, D, dtype=x.dtype)
    for j in range(nb):
        out[:, :, j * P:j * P + bs - 1] = x[:, :, j * bs:j * bs + bs - 1]
        out[:, :, j * P + P - 1] = x[:, :, j * bs + bs - 1]
    out[:, :, nb * P:] = x[:, :, nb * bs:]
    return out


@pytest.mark.parametrize("bs,P,L,D", [(51, 64, 510, 128), (51, 64, 120, 128), (2, 64, 10, 64), (100, 128, 300, 128),
                                       (64, 64, 128, 128), (33, 64, 5, 64)])
def test_repacking_is_bit_exact_both_ways(bs, P, L, D):
    from landmark_hip import _lib
    lib = _lib.lib()
    B, H = 2, 3
    x = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(L + bs)).bfloat16()
    want = _expected_padded(x, bs, P)
    assert lib.lmk_padded_rows(L, bs, P) == want.shape[2]
    xd = x.to(DEV)
    pd = torch.full(want.shape, float("nan"), dtype=x.dtype, device=DEV)       # every row must be written
    _lib.check(lib.lmk_pad_blocks(_lib.tensor4(xd), _lib.tensor4(pd), B, H, L, D, bs, P, _lib.current_stream(xd.device)))
    assert torch.equal(pd.cpu(), want)
    back = torch.full(x.shape, float("nan"), dtype=x.dtype, device=DEV)
    _lib.check(lib.lmk_unpad_blocks(_lib.tensor4(pd), _lib.tensor4(back), B, H, L, D, bs, P, _lib.current_stream(xd.device)))
    assert torch.equal(back.cpu(), x)


def _run(q, k, v, do, block, scale=None):
    from ltriton.flash_landmark_attention import fused_landmark_attention
    qd, kd, vd = (t.to(DEV).requires_grad_(do is not None) for t in (q, k, v))
    is_mem = torch.arange(k.shape[2], device=DEV) % block == block - 1
    out = fused_landmark_attention(qd, kd, vd, is_mem, sm_scale=scale, block_size=block)
    grads = torch.autograd.grad(out, [qd, kd, vd], do.to(DEV)) if do is not None else None
    torch.cuda.synchronize()
    return out, grads


FWD_CASES = [
    # B, H, Lq, Lk, D, block, dtype
    (1, 2, 102, 102, 128, 51, torch.bfloat16),
    (2, 3, 255, 510, 128, 51, torch.bfloat16),      # history of five blocks
    (1, 2, 120, 120, 128, 51, torch.bfloat16),      # partial last block (forward only)
    (1, 2, 5, 107, 128, 51, torch.bfloat16),        # a few new rows behind two blocks of history
    (1, 2, 170, 170, 64, 17, torch.float16),        # narrower than a 32-key tile
    (1, 2, 300, 300, 128, 100, torch.bfloat16),     # stored in 128 slots
    (1, 2, 195, 325, 128, 65, torch.bfloat16),      # one past a native size
    (1, 2, 189, 189, 64, 63, torch.bfloat16),       # one short of a native size: a single padding slot
    (1, 2, 254, 254, 128, 127, torch.float16),
    (1, 4, 40, 40, 128, 2, torch.bfloat16),         # one normal key per block
    (1, 2, 99, 99, 128, 33, torch.bfloat16),
]


@pytest.mark.parametrize("B,H,Lq,Lk,D,block,dtype", FWD_CASES)
def test_forward_matches_oracle(B, H, Lq, Lk, D, block, dtype):
    print(f"case B{B} H{H} Lq{Lq} Lk{Lk} D{D} bs{block} {dtype}", flush=True)
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=Lq + Lk + block, dtype=dtype)
    ref, _, _ = oracle_forward(q, k, v, block)
    out, _ = _run(q, k, v, None, block)
    assert out.shape == q.shape and out.dtype == dtype
    err = (out.float().cpu() - ref).abs().max().item()
    assert err <= TOL, err


BWD_CASES = [c for c in FWD_CASES if c[2] % c[5] == 0] + [
    (1, 2, 561, 561, 128, 51, torch.bfloat16),      # 11 blocks: three workgroups per head
    (1, 2, 153, 255, 64, 51, torch.float16),
]


@pytest.mark.parametrize("B,H,Lq,Lk,D,block,dtype", BWD_CASES)
def test_gradients_match_oracle(B, H, Lq, Lk, D, block, dtype):
    print(f"case B{B} H{H} Lq{Lq} Lk{Lk} D{D} bs{block} {dtype}", flush=True)
    seed = Lq + Lk + D + block
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=seed, dtype=dtype)
    do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(seed + 1)).to(dtype)
    rq, rk, rv = oracle_grads(q, k, v, do, block)
    _, (gq, gk, gv) = _run(q, k, v, do, block)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        assert err <= TOL, (name, err)
        assert g.dtype == dtype and g.shape == r.shape


def test_custom_scale_and_large_magnitudes_with_block_51():
    B, H, L, D, block = 1, 2, 204, 128, 51
    q, k, v = make_qkv(B, H, L, L, D, seed=77, scale=2.0)
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(78)).bfloat16()
    ref, _, _ = oracle_forward(q, k, v, block, scale=0.05)
    rq, rk, rv = oracle_grads(q, k, v, do, block, scale=0.05)
    out, (gq, gk, gv) = _run(q, k, v, do, block, scale=0.05)
    assert (out.float().cpu() - ref).abs().max().item() <= TOL * max(1.0, ref.abs().max().item())
    for g, r in ((gq, rq), (gk, rk), (gv, rv)):
        assert (g.float().cpu() - r).abs().max().item() <= TOL * max(1.0, r.abs().max().item())


def test_benchmark_config0_full_size():
    """B=2 H=8 L=510 D=128, block 51, N(0,1) inputs of seed 0 (the case the reference's CPU path runs),
    rounded to bf16 for the kernels and the oracle alike: forward against the restated high-level path
    (lm_benchmark/models/landmark.py:196-236, 16 buckets), gradients against autograd through the closed form."""
    from oracle import highlevel
    B, H, L, D, block = 2, 8, 510, 128, 51
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(B, H, L, D, generator=g).bfloat16() for _ in range(3))
    is_mem = (torch.arange(L) % block == block - 1)[None].expand(B, L)
    ref = highlevel.attention_lm_benchmark(q.float(), k.float(), v.float(), is_mem, n_buckets=16)
    do = torch.randn(B, H, L, D, generator=g).bfloat16()
    out, (gq, gk, gv) = _run(q, k, v, do, block)
    err = (out.float().cpu() - ref).abs().max().item()
    assert err <= TOL, err
    rq, rk, rv = oracle_grads(q, k, v, do, block)
    for name, a, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        e = (a.float().cpu() - r).abs().max().item()
        assert e <= TOL * max(1.0, r.abs().max().item()), (name, e)


def test_padded_entry_points_reject_what_the_kernels_do_not_cover():
    from landmark_hip import _lib
    lib = _lib.lib()
    B, H, L, D = 1, 1, 64, 128
    x = torch.zeros(B, H, L, D, dtype=torch.bfloat16, device=DEV)
    st = torch.zeros(B * H, L, device=DEV)
    t4 = _lib.tensor4(x)

    def fwd(block, real):
        return lib.lmk_attn_fwd_padded(t4, t4, t4, t4, st.data_ptr(), st.data_ptr(), B, H, L, L, D, 0.1, block, real, 0, 0,
                                       _lib.current_stream(x.device))
    assert fwd(32, 17) == -3            # the block-32 kernels carry no padding mask
    assert fwd(64, 1) == -2 and fwd(64, 65) == -2
    assert fwd(64, 64) == 0 and fwd(64, 51) == 0 and fwd(32, 32) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("D,block", [(32, 32), (16, 64), (32, 51)])
def test_head_dims_16_and_32(D, block):
    # the reference accepts head dims 16 and 32 as well (flash_landmark_attention.py:321)
    B, H, L = 1, 3, 4 * block
    q, k, v = make_qkv(B, H, L, L, D, seed=D + block)
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(5)).bfloat16()
    ref, _, _ = oracle_forward(q, k, v, block)
    rq, rk, rv = oracle_grads(q, k, v, do, block)
    out, (gq, gk, gv) = _run(q, k, v, do, block)
    assert out.shape == q.shape
    assert (out.float().cpu() - ref).abs().max().item() <= TOL
    for g, r in ((gq, rq), (gk, rk), (gv, rv)):
        assert g.shape == r.shape and (g.float().cpu() - r).abs().max().item() <= TOL


@pytest.mark.parametrize("block,D,L,P", [(51, 128, 204, 1), (100, 64, 300, 0), (17, 128, 136, 2)])
def test_token_layout_equals_the_repacked_path_bit_for_bit(block, D, L, P):
    # the kernels reading the tensors as they are (lmk_attn_*_blocks) against the same kernels on repacked copies
    # (lmk_pad_blocks + lmk_attn_*_padded + lmk_unpad_blocks): same arithmetic on the same values, so the same bits;
    # and the autograd function keeps the caller's tensors, not padded copies
    from landmark_hip import attention
    from ltriton.flash_landmark_attention import fused_landmark_attention
    B, H = 1, 2
    Lk = L + P * block
    q, k, v = (t.to(DEV) for t in make_qkv(B, H, L, Lk, D, seed=block + L))
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(3)).bfloat16().to(DEV)
    scale = D ** -0.5
    slots = attention.storage_block(block)
    o, Ls, M = attention._launch_fwd_blocks(q, k, v, P, scale, block)
    dq, dk, dv = attention._launch_bwd_blocks(q, k, v, o, do, Ls, M, P, scale, block)
    qp, kp, vp, dop = (attention._repack(t, block, slots) for t in (q, k, v, do))
    op, Lp, Mp = attention._launch_fwd(qp, kp, vp, P, scale, slots, block)
    dqp, dkp, dvp = attention._launch_bwd(qp, kp, vp, op, dop, Lp, Mp, P, scale, slots, block)
    torch.cuda.synchronize()
    assert torch.equal(o, attention._repack(op, block, slots, unpad=True, rows=L))
    assert torch.equal(dq, attention._repack(dqp, block, slots, unpad=True, rows=L))
    assert torch.equal(dk, attention._repack(dkp, block, slots, unpad=True, rows=Lk))
    assert torch.equal(dv, attention._repack(dvp, block, slots, unpad=True, rows=Lk))
    r = torch.arange(L, device=DEV)
    r = r // block * slots + torch.where(r % block == block - 1, slots - 1, r % block)
    assert torch.equal(Ls, Lp[:, r]) and torch.equal(M, Mp[:, r])
    qg = q.clone().requires_grad_(True)
    out = fused_landmark_attention(qg, k, v, None, block_size=block)
    assert all(t.shape[2] in (L, Lk) for t in out.grad_fn.saved_tensors[:4])


def test_token_layout_ignores_what_lies_in_rows_it_does_not_own():
    # the padded entry points need finite values in their padding rows; the token-layout ones have no such rows:
    # NaNs around the tensors (strided views of a larger, poisoned buffer) must not reach any result
    from landmark_hip import attention
    B, H, L, D, block = 1, 2, 153, 128, 51
    big = [torch.full((B, H, L + 64, D), float("nan"), dtype=torch.bfloat16, device=DEV) for _ in range(4)]
    q, k, v, do = (make_qkv(B, H, L, L, D, seed=9)[i].to(DEV) if i < 3 else
                   torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(1)).bfloat16().to(DEV) for i in range(4))
    views = []
    for buf, t in zip(big, (q, k, v, do)):
        buf[:, :, 32:32 + L] = t
        views.append(buf[:, :, 32:32 + L])
    qv, kv, vv, dov = views
    scale = D ** -0.5
    o, Ls, M = attention._launch_fwd_blocks(qv, kv, vv, 0, scale, block)
    grads = attention._launch_bwd_blocks(qv, kv, vv, o, dov, Ls, M, 0, scale, block)
    o2, L2, M2 = attention._launch_fwd_blocks(q, k, v, 0, scale, block)
    grads2 = attention._launch_bwd_blocks(q, k, v, o2, do, L2, M2, 0, scale, block)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.equal(o, o2)
    for a, b_ in zip(grads, grads2):
        assert torch.isfinite(a.float()).all() and torch.equal(a, b_)
