"""Writes the golden fixtures in this directory from the CPU oracle's slowest, most literal paths.

    python tests/golden/make_fixtures.py

The reference holds no golden vectors for this path (its only test draws unseeded random inputs,
llama/ltriton/test_flash_landmark_attention.py:91-94), so these are the build's own: inputs drawn
from a seeded generator and rounded to bf16, expected values from
  * attention:  the per-row Python-float loop ``oracle.s1.s1_rows_python`` (out, L, M) and float64
                autograd through the closed form (dq, dk, dv);
  * retrieval:  the sequential-accumulation score contract and (score desc, index asc) selection of
                ``oracle.retrieval`` (indices), and a float64 evaluation of the attend step written
                out per query in this file (out), for a cache that ends in an incomplete block;
  * per-head selection (``max_over_tokens``): the softmax contract written out lane by lane in
                numpy scalars (the head's vector of 16-bit probabilities and its top-k), and a
                float64 evaluation of the attention over [selected blocks | tail | new tokens].
They pin the oracle against silent changes (tests/test_golden.py, CPU) and are a second target for
the HIP kernels (tests/test_gpu_golden.py).  Values are stored as float32 / int64 in .npz files.
"""
import math
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import retrieval, rotary, s1  # noqa: E402


def _bf16(*shape, gen, scale=0.5):
    return (torch.randn(*shape, generator=gen) * scale).bfloat16().float()


def attention_fixture():
    g = torch.Generator().manual_seed(1234)
    H, Lq, Lk, D, block = 1, 64, 96, 64, 32                  # one history block, two query blocks
    q, k, v = _bf16(H, Lq, D, gen=g), _bf16(H, Lk, D, gen=g), _bf16(H, Lk, D, gen=g)
    do = _bf16(H, Lq, D, gen=g, scale=1.0)
    out, L, M = [], [], []
    for h in range(H):
        o, ell, m = s1.s1_rows_python(q[h], k[h], v[h], block)
        out.append(o), L.append(ell), M.append(m)
    qd, kd, vd = (t.double().requires_grad_(True) for t in (q, k, v))
    o64 = s1.s1_attention(qd, kd, vd, block)
    dq, dk, dv = torch.autograd.grad(o64, [qd, kd, vd], do.double())
    assert (o64.detach() - torch.tensor(out, dtype=torch.float64)).abs().max() < 1e-12
    np.savez_compressed(os.path.join(HERE, "attention_h1_lq64_lk96_d64_b32.npz"),
                        q=q.numpy(), k=k.numpy(), v=v.numpy(), do=do.numpy(), block=np.int64(block),
                        out=np.asarray(out, np.float32), L=np.asarray(L, np.float32), M=np.asarray(M, np.float32),
                        dq=dq.float().numpy(), dk=dk.float().numpy(), dv=dv.float().numpy())


def retrieval_fixture():
    g = torch.Generator().manual_seed(4321)
    H, T, D, block, n_mems, inc, top_k = 1, 3, 128, 32, 6, 5, 2
    S = n_mems * block + inc
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.5).bfloat16()
    q, kc, vc, kl, vl = mk(1, H, T, D), mk(1, H, S, D), mk(1, H, S, D), mk(1, H, T, D), mk(1, H, T, D)
    cos, sin = rotary.rotary_tables(S + T, D, torch.bfloat16)
    geo = retrieval.retrieval_geometry(S, block, top_k)
    idx = retrieval.select_topk(retrieval.landmark_scores(q, kc, cos, sin, block, top_k), geo["k"])
    out = np.zeros((1, H, T, D), np.float64)
    for h in range(H):
        for t in range(T):
            qq = q[0, h, t].double()
            sel = idx[0, h, t]
            pos = retrieval.gather_positions(sel, geo["num_mems"], geo["k"], block, geo["prefix_len"])
            blocks = [(rotary.apply_rotary(kc[0, h, b * block:(b + 1) * block], cos, sin, pos[j]).double(),
                       vc[0, h, b * block:(b + 1) * block].double()) for j, b in enumerate(sel.tolist())]
            tail_pos = torch.arange(geo["full_len"], S)
            wk = torch.cat((rotary.apply_rotary(kc[0, h, geo["full_len"]:], cos, sin, tail_pos), kl[0, h])).double()
            wv = torch.cat((vc[0, h, geo["full_len"]:], vl[0, h])).double()
            last = inc + t - (1 if (inc + t) % block == block - 1 else 0)
            z = torch.cat((torch.stack([(kb[block - 1] @ qq) / math.sqrt(D) for kb, _ in blocks]),
                           (wk[: last + 1] @ qq) / math.sqrt(D)))
            w = torch.softmax(z, 0)
            o = w[geo["k"]:] @ wv[: last + 1]
            for j, (kb, vb) in enumerate(blocks):
                o = o + w[j] * (torch.softmax((kb[: block - 1] @ qq) / math.sqrt(D), 0) @ vb[: block - 1])
            out[0, h, t] = o.numpy()
    np.savez_compressed(os.path.join(HERE, "retrieval_h1_t3_s197_d128_b32_k2.npz"),
                        q=q.float().numpy(), k_cache=kc.float().numpy(), v_cache=vc.float().numpy(),
                        k_loc=kl.float().numpy(), v_loc=vl.float().numpy(), block=np.int64(block),
                        top_k=np.int64(top_k), idx=idx.numpy(), out=out.astype(np.float32))


def shared_selection_fixture():
    g = torch.Generator().manual_seed(2468)
    H, T, D, block, n_mems, inc, top_k = 1, 4, 64, 32, 66, 3, 3         # 66 blocks: lanes 0 and 1 sum two terms
    S = n_mems * block + inc
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.5).bfloat16()
    q, kc, vc, kl, vl = mk(1, H, T, D), mk(1, H, S, D), mk(1, H, S, D), mk(1, H, T, D), mk(1, H, T, D)
    cos, sin = rotary.rotary_tables(S + T, D, torch.bfloat16)
    geo = retrieval.retrieval_geometry(S, block, top_k)
    sc = retrieval.landmark_scores(q, kc, cos, sin, block, top_k).float().numpy()   # (1,H,T,n_mems)
    f32 = np.float32
    coef = [f32(c) for c in (1.0, 0.6931471805599453, 0.2402265069591007, 0.05550410866482158,
                             0.009618129107628477, 0.0013333558146428443, 0.00015403530393381608)]
    probs = np.zeros((1, H, n_mems), np.float32)
    for h in range(H):
        for t in range(T):
            x = sc[0, h, t]
            mx = x.max()
            e = []
            for m in range(n_mems):                                     # 2^t by the fixed polynomial
                tt = f32(f32(x[m] - mx) * f32(1.4426950408889634))
                n = np.rint(tt)
                fr = f32(tt - n)
                p = coef[6]
                for c in coef[5::-1]:
                    p = f32(f32(p * fr) + c)
                e.append(f32(0.0) if tt < f32(-126.0) else f32(np.ldexp(p, int(n))))
            lanes = [f32(0.0)] * 64
            for m in range(n_mems):                                     # lane m % 64 adds its terms in order
                lanes[m % 64] = f32(lanes[m % 64] + e[m])
            w = 32
            while w:                                                    # fold by halves
                lanes = [f32(lanes[i] + lanes[i + w]) for i in range(w)]
                w //= 2
            row = torch.tensor([f32(v / lanes[0]) for v in e]).bfloat16().float().numpy()
            probs[0, h] = np.maximum(probs[0, h], row)                  # amax over the queries
    idx = np.zeros((1, H, 1, geo["k"]), np.int64)
    for h in range(H):
        order = sorted(range(n_mems), key=lambda m: (-probs[0, h, m], m))   # value desc, index asc
        idx[0, h, 0] = sorted(order[: geo["k"]])
    idx_t = torch.from_numpy(idx)
    out = np.zeros((1, H, T, D), np.float64)
    for h in range(H):
        sel = idx_t[0, h, 0]
        pos = retrieval.gather_positions(sel, geo["num_mems"], geo["k"], block, geo["prefix_len"])
        blocks = [(rotary.apply_rotary(kc[0, h, b * block:(b + 1) * block], cos, sin, pos[j]).double(),
                   vc[0, h, b * block:(b + 1) * block].double()) for j, b in enumerate(sel.tolist())]
        tail_pos = torch.arange(geo["full_len"], S)
        wk = torch.cat((rotary.apply_rotary(kc[0, h, geo["full_len"]:], cos, sin, tail_pos), kl[0, h])).double()
        wv = torch.cat((vc[0, h, geo["full_len"]:], vl[0, h])).double()
        for t in range(T):
            qq = q[0, h, t].double()
            last = inc + t - (1 if (inc + t) % block == block - 1 else 0)
            z = torch.cat((torch.stack([(kb[block - 1] @ qq) / math.sqrt(D) for kb, _ in blocks]),
                           (wk[: last + 1] @ qq) / math.sqrt(D)))
            w = torch.softmax(z, 0)
            o = w[geo["k"]:] @ wv[: last + 1]
            for j, (kb, vb) in enumerate(blocks):
                o = o + w[j] * (torch.softmax((kb[: block - 1] @ qq) / math.sqrt(D), 0) @ vb[: block - 1])
            out[0, h, t] = o.numpy()
    bits = lambda t: t.view(torch.int16).numpy()                        # bf16 bit patterns: half the bytes of float32
    np.savez_compressed(os.path.join(HERE, "shared_selection_h1_t4_s2115_d64_b32_k3.npz"),
                        q_bf16bits=bits(q), k_cache_bf16bits=bits(kc), v_cache_bf16bits=bits(vc),
                        k_loc_bf16bits=bits(kl), v_loc_bf16bits=bits(vl), block=np.int64(block),
                        top_k=np.int64(top_k), block_probs=probs, idx=idx, out=out.astype(np.float32))


if __name__ == "__main__":
    attention_fixture()
    retrieval_fixture()
    shared_selection_fixture()
    print("fixtures written to", HERE)
