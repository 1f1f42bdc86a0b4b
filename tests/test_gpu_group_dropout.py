"""Group dropout on the fused path (lm_benchmark/models/landmark.py:110-113): the caller supplies the outcome of the
dropout as a factor per (query row, earlier block); forward against the restated high-level grouped softmax with the
same factors and against the closed form, gradients against autograd through the closed form.  Tolerance 2e-2 max
abs on 16-bit-rounded inputs, as for the other attention tests."""
import math

import pytest
import torch

from oracle import highlevel, s1
from tests.util import make_qkv

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-2


def _keep(B, H, nb, Lq, p, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(B, H, nb, Lq, generator=g) >= p).float() / (1.0 - p)       # what F.dropout(ones, p) yields


@pytest.mark.parametrize("B,H,Lq,Lk,D,block,dtype", [
    (2, 3, 204, 204, 128, 51, torch.bfloat16),       # the benchmark models' block
    (1, 2, 255, 357, 64, 51, torch.bfloat16),        # two history blocks, head dim 64
    (1, 2, 256, 256, 128, 32, torch.bfloat16),       # block 32 runs in 64 slots here
    (1, 2, 256, 384, 128, 64, torch.float16),
    (1, 2, 512, 512, 64, 128, torch.bfloat16),
    (1, 2, 300, 300, 128, 100, torch.bfloat16),
])
def test_group_dropout_forward_and_gradients(B, H, Lq, Lk, D, block, dtype):
    from ltriton.flash_landmark_attention import fused_landmark_attention
    print(f"case group dropout B{B} H{H} Lq{Lq} Lk{Lk} D{D} bs{block} {dtype}", flush=True)
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=Lq + block, dtype=dtype)
    do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(2)).to(dtype)
    keep = _keep(B, H, Lk // block, Lq, 0.3, seed=block)
    qc, kc, vc = (t.float().requires_grad_(True) for t in (q, k, v))
    ref = s1.s1_attention(qc, kc, vc, block, group_scale=keep)
    rq, rk, rv = torch.autograd.grad(ref, [qc, kc, vc], do.float())
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = fused_landmark_attention(qd, kd, vd, None, block_size=block, group_scale=keep.to(DEV))
    gq, gk, gv = torch.autograd.grad(out, [qd, kd, vd], do.to(DEV))
    torch.cuda.synchronize()
    assert (out.float().cpu() - ref.detach()).abs().max().item() <= TOL
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        assert err <= TOL, (name, err)
    # a dropped block must change the result: the same call without factors differs
    plain = fused_landmark_attention(qd, kd, vd, None, block_size=block)
    assert (plain.float() - out.float()).abs().max().item() > 1e-2
    # all factors 1: the plain kernels' result to the last bit when they are the same kernels (blocks other than 32)
    ones = torch.ones_like(keep).to(DEV)
    same = fused_landmark_attention(qd, kd, vd, None, block_size=block, group_scale=ones)
    if block != 32:
        assert torch.equal(same, plain)
    else:
        assert (same.float() - plain.float()).abs().max().item() <= 1e-2


def test_group_dropout_against_the_high_level_path_of_the_benchmark():
    # forward of CausalSelfAttention with softmax_func = mem_opt and p_group_dropout (landmark.py:196-236, :110-113),
    # restated in oracle/highlevel.py, with the dropout's outcome fixed
    from ltriton.flash_landmark_attention import fused_landmark_attention
    B, H, L, D, block = 2, 4, 255, 128, 51
    nb = L // block
    q, k, v = make_qkv(B, H, L, L, D, seed=5)
    keep = _keep(B, H, nb, L, 0.5, seed=6)
    att = (q.float() @ k.float().transpose(-2, -1)) / math.sqrt(D)
    causal_masked = ~torch.tril(torch.ones(L, L, dtype=torch.bool))[None, None].expand(B, H, L, L)
    att = att.masked_fill(causal_masked, float("-inf"))
    is_mem = (torch.arange(L) % block == block - 1)[None].expand(B, L)
    masked, im, ls = highlevel.masks_from_is_mem(is_mem[:, None, None, :], causal_masked)
    att = att.masked_fill(masked, float("-inf"))
    n_buckets = 16
    keep_b = torch.ones(B, H, L, n_buckets)
    keep_b[..., :nb] = keep.transpose(-1, -2)
    ref = highlevel.grouped_softmax(att, im, ls, n_buckets, attn_mask=masked, guard_empty=True, group_keep=keep_b) @ v.float()
    out = fused_landmark_attention(q.to(DEV), k.to(DEV), v.to(DEV), is_mem[0].to(DEV), block_size=block,
                                   group_scale=keep.to(DEV))
    assert (out.float().cpu() - ref).abs().max().item() <= TOL
