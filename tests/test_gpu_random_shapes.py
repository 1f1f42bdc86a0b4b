"""Seeded random sweep over shapes, block sizes, dtypes, layouts and history lengths: forward and gradients
of the attention against the fp32 oracle, and both retrieval modes against the model-dtype restatement.
Every case prints its parameters before it runs, so a failure (or a fault) names its case."""
import random

import pytest
import torch

from oracle import retrieval as oret
from oracle import rotary as orot
from tests.util import make_qkv, oracle_forward, oracle_grads

pytestmark = pytest.mark.gpu

TOL = 2e-2


@pytest.mark.parametrize("sweep_seed", [1, 2])
def test_attention_random_shapes(sweep_seed):
    from ltriton.flash_landmark_attention import fused_landmark_attention
    rnd = random.Random(sweep_seed)
    dev = torch.device("cuda:0")
    for it in range(24):
        block = rnd.choice([32, 32, 32, 64, 128])
        D = rnd.choice([128, 128, 64])
        dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        n_blocks, n_hist = rnd.randint(1, 12), rnd.choice([0, 0, 1, 2, 3, 5, 9])
        B, H = rnd.choice([1, 2]), rnd.choice([1, 2, 3, 8])
        Lq = n_blocks * block
        Lk = Lq + n_hist * block
        backward = True
        if rnd.random() < 0.25:                          # partial last block: forward only
            cut = rnd.randint(1, block - 1)
            Lq, Lk, backward = Lq - cut, Lk - cut, False
        layout = rnd.choice(["bhld", "blhd"])
        print(f"case {sweep_seed}.{it} B{B} H{H} Lq{Lq} Lk{Lk} D{D} bs{block} {dtype} {layout} bwd={backward}", flush=True)
        q, k, v = make_qkv(B, H, Lq, Lk, D, seed=1000 * sweep_seed + it, dtype=dtype, layout=layout)
        ref, _, _ = oracle_forward(q, k, v, block)
        qd, kd, vd = (t.to(dev).requires_grad_(backward) for t in (q, k, v))
        out = fused_landmark_attention(qd, kd, vd, None, block_size=block)
        assert (out.float().cpu() - ref).abs().max().item() <= TOL, it
        if backward:
            do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(77 + it)).to(dtype)
            want = oracle_grads(q, k, v, do, block)
            got = torch.autograd.grad(out, [qd, kd, vd], do.to(dev))
            for g, r in zip(got, want):
                assert (g.float().cpu() - r).abs().max().item() <= TOL, it


@pytest.mark.parametrize("sweep_seed", [3])
def test_retrieval_random_shapes(sweep_seed):
    from landmark_hip.retrieval import retrieve_and_attend
    rnd = random.Random(sweep_seed)
    D = 128
    for it in range(30):
        block = rnd.choice([32, 64, 128])
        n_mems, top_k = rnd.choice([1, 2, 3, 5, 17, 40, 130]), rnd.choice([1, 2, 4, 5, 8])
        dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        if rnd.random() < 0.5:                           # cache ends in an incomplete block
            inc = rnd.randint(1, block - 1)
            T = rnd.randint(1, block - inc)
        else:
            inc, T = 0, rnd.choice([1, 3, block, block + 5, 3 * block])
        B, H = rnd.choice([1, 2]), rnd.choice([1, 2, 3])
        aggregate = rnd.choice([None, "max_over_tokens"])
        S = n_mems * block + inc
        print(f"case {sweep_seed}.{it} B{B} H{H} T{T} n_mems{n_mems} inc{inc} bs{block} k{top_k} {dtype} {aggregate}", flush=True)
        g = torch.Generator().manual_seed(3000 + it)
        mk = lambda *s: (torch.randn(*s, generator=g) * 0.5).to(dtype)
        q, kc, vc, kl, vl = mk(B, H, T, D), mk(B, H, S, D), mk(B, H, S, D), mk(B, H, T, D), mk(B, H, T, D)
        cos, sin = orot.rotary_tables(S + T, D, dtype)
        is_mem = ((torch.arange(T) + inc) % block == block - 1)[None].expand(B, T)
        oracle = oret.retrieve_and_attend_shared if aggregate else oret.retrieve_and_attend
        want, want_idx = oracle(q, kc, vc, kl, vl, is_mem, cos, sin, block, top_k, n_buckets=max(64, top_k + T // block + 3))
        dev = lambda t: t.cuda()
        out, idx = retrieve_and_attend(dev(q), (dev(kc), dev(vc)), dev(kl), dev(vl), dev(cos), dev(sin), block, top_k,
                                       aggregate=aggregate)
        torch.cuda.synchronize()
        assert torch.equal(idx.cpu(), want_idx), it
        assert (out.float().cpu() - want.float()).abs().max().item() <= TOL, it
