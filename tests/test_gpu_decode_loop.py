"""A decode loop over the growing cache: every step's block indices bit for bit and its attention within
2e-2 of the oracle, across a landmark boundary and a reallocation of the cache buffers
(llama/llama_mem.py:318-430: attend against the cache, then append)."""
import pytest
import torch

from oracle import retrieval as oret
from oracle import rotary as orot

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("aggregate", [None, "max_over_tokens"])
def test_decode_steps_match_the_oracle(aggregate):
    from landmark_hip.cache import LandmarkKVCache
    B, H, D, block, top_k = 1, 2, 128, 32, 2
    chunks = [3 * block, 5] + [1] * 27 + [block, 7, 1]          # prefill, then chunks and single tokens
    total = sum(chunks)
    g = torch.Generator().manual_seed(11)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.5).bfloat16()
    q_all, k_all, v_all = mk(B, H, total, D), mk(B, H, total, D), mk(B, H, total, D)     # before rotary
    cos, sin = orot.rotary_tables(total, D, torch.bfloat16)
    pos = torch.arange(total)
    q_rot, k_rot = orot.apply_rotary(q_all, cos, sin, pos), orot.apply_rotary(k_all, cos, sin, pos)
    dev = torch.device("cuda:0")
    cache = LandmarkKVCache(B, H, D, torch.bfloat16, dev, capacity=64)             # forces two reallocations
    cd, sd = cos.to(dev), sin.to(dev)
    S = 0
    for step, T in enumerate(chunks):
        sl = slice(S, S + T)
        if step == 0:
            cache.append(k_all[:, :, sl].to(dev), v_all[:, :, sl].to(dev))
        else:
            inc = S % block
            print(f"step {step} S{S} T{T} inc{inc} {aggregate}", flush=True)
            is_mem = ((torch.arange(T) + inc) % block == block - 1)[None]
            ref = oret.retrieve_and_attend_shared if aggregate else oret.retrieve_and_attend
            want, want_idx = ref(q_rot[:, :, sl], k_all[:, :, :S], v_all[:, :, :S], k_rot[:, :, sl], v_all[:, :, sl],
                                 is_mem, cos, sin, block, top_k)
            out, idx = cache.step(q_rot[:, :, sl].to(dev), k_rot[:, :, sl].to(dev), k_all[:, :, sl].to(dev),
                                  v_all[:, :, sl].to(dev), cd, sd, block, top_k, aggregate=aggregate)
            torch.cuda.synchronize()
            assert torch.equal(idx.cpu(), want_idx), step
            assert (out.float().cpu() - want.float()).abs().max().item() <= 2e-2, step
        S += T
        pk, pv = cache.past_key_value
        assert pk.shape[2] == S
    assert torch.equal(cache.past_key_value[0].cpu(), k_all) and torch.equal(cache.past_key_value[1].cpu(), v_all)
