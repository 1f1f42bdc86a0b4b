"""The committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py from the
oracle's most literal paths) against the oracle's vectorised paths: guards the checker itself."""
import os

import numpy as np
import torch

from oracle import retrieval, rotary, s1

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLDEN, name)) as z:       # plain arrays, no pickles
        return {k: torch.from_numpy(np.asarray(z[k])) for k in z.files}


def test_attention_fixture_matches_closed_form_and_autograd():
    f = load("attention_h1_lq64_lk96_d64_b32.npz")
    block = int(f["block"])
    q, k, v = (f[n].clone().requires_grad_(True) for n in ("q", "k", "v"))
    w, L, M = s1.s1_weights(q.detach(), k.detach(), block)
    out = s1.s1_attention(q, k, v, block)
    assert (out.detach() - f["out"]).abs().max() < 1e-5
    assert ((L - f["L"]).abs() / f["L"]).max() < 1e-5 and (M - f["M"]).abs().max() < 1e-5
    dq, dk, dv = torch.autograd.grad(out, [q, k, v], f["do"])
    for got, name in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert (got - f[name]).abs().max() < 2e-5, name
    # inputs are exactly representable in bf16, as the kernels will see them
    for n in ("q", "k", "v", "do"):
        assert torch.equal(f[n].bfloat16().float(), f[n])


def test_retrieval_fixture_matches_restated_reference_path():
    f = load("retrieval_h1_t3_s197_d128_b32_k2.npz")
    block, top_k = int(f["block"]), int(f["top_k"])
    q, kc, vc, kl, vl = (f[n].bfloat16() for n in ("q", "k_cache", "v_cache", "k_loc", "v_loc"))
    S, T, D = kc.shape[2], q.shape[2], q.shape[3]
    cos, sin = rotary.rotary_tables(S + T, D, torch.bfloat16)
    inc = S % block
    is_mem = ((torch.arange(T) + inc) % block == block - 1)[None]
    out, idx = retrieval.retrieve_and_attend(q, kc, vc, kl, vl, is_mem, cos, sin, block, top_k)
    assert torch.equal(idx, f["idx"])
    assert (out.float() - f["out"]).abs().max() < 2e-2           # the restatement rounds to bf16 where the reference does
    out32, _ = retrieval.retrieve_and_attend(q.float(), kc.float(), vc.float(), kl.float(), vl.float(), is_mem,
                                             cos.float(), sin.float(), block, top_k, idx=f["idx"])
    assert (out32 - f["out"]).abs().max() < 2e-2                 # fp32 tables differ from the bf16 ones the fixture used


def test_shared_selection_fixture_matches_vectorised_contract():
    f = load("shared_selection_h1_t4_s2115_d64_b32_k3.npz")
    block, top_k = int(f["block"]), int(f["top_k"])
    q, kc, vc, kl, vl = (f[n + "_bf16bits"].view(torch.bfloat16) for n in ("q", "k_cache", "v_cache", "k_loc", "v_loc"))
    S, T, D = kc.shape[2], q.shape[2], q.shape[3]
    cos, sin = rotary.rotary_tables(S + T, D, torch.bfloat16)
    agg = retrieval.aggregate_max_over_tokens(retrieval.landmark_scores(q, kc, cos, sin, block, top_k))
    assert torch.equal(agg[:, :, 0].float(), f["block_probs"])    # the head's vector, bit for bit
    inc = S % block
    is_mem = ((torch.arange(T) + inc) % block == block - 1)[None]
    out, idx = retrieval.retrieve_and_attend_shared(q, kc, vc, kl, vl, is_mem, cos, sin, block, top_k)
    assert torch.equal(idx, f["idx"])
    assert (out.float() - f["out"]).abs().max() < 2e-2
    ref32 = retrieval.retrieve_and_attend_shared_s1(q, kc, vc, kl, vl, cos, sin, block, top_k, f["idx"])
    assert (ref32 - f["out"]).abs().max() < 2e-3
