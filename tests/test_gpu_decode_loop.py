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


def test_offloaded_cache_equals_the_device_cache_step_for_step():
    """offload_cache_to_cpu (llama_mem.py:326-328,344-356): blocks in pinned host memory, landmark keys on the GPU,
    one selection per head.  Same indices and bit-identical attention as the device-resident cache with
    aggregate="max_over_tokens", over chunks and single tokens that cross landmarks and one regrowth of the buffers."""
    from landmark_hip.cache import LandmarkKVCache, OffloadedLandmarkCache
    from landmark_hip.rotary import apply_rotary_pos_emb
    from oracle import rotary as orot
    B, H, D, block, top_k = 2, 3, 128, 32, 3
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(11)
    cos, sin = (t.to(dev) for t in orot.rotary_tables(4096, D, torch.bfloat16))
    dcache = LandmarkKVCache(B, H, D, torch.bfloat16, dev, capacity=64)
    ocache = OffloadedLandmarkCache(B, H, D, block, torch.bfloat16, dev, capacity=64)
    prompt = 3 * block + 5
    k0 = (torch.randn(B, H, prompt, D, generator=g) * 0.5).bfloat16().to(dev)
    v0 = (torch.randn(B, H, prompt, D, generator=g) * 0.5).bfloat16().to(dev)
    dcache.append(k0, v0)
    ocache.append(k0, v0)
    assert ocache.n_blocks == 3 and torch.equal(ocache.landmark_keys.cpu(), k0[:, :, block - 1::block].cpu())
    for step, T in enumerate([1, 1, 20, 5, 1, 27, 4, 1, 1, 30, 2, 32 - 30]):
        S = dcache.length
        inc = S % block
        assert inc == 0 or T + inc <= block
        print(f"offload step {step}: S{S} T{T}", flush=True)
        q = (torch.randn(B, H, T, D, generator=g) * 0.5).bfloat16().to(dev)
        kn = (torch.randn(B, H, T, D, generator=g) * 0.5).bfloat16().to(dev)
        v = (torch.randn(B, H, T, D, generator=g) * 0.5).bfloat16().to(dev)
        pos = torch.arange(S, S + T, device=dev)[None]
        q_rot, k_rot = apply_rotary_pos_emb(q, kn, cos, sin, pos)
        want, want_idx = dcache.step(q_rot, k_rot, kn, v, cos, sin, block, top_k, aggregate="max_over_tokens")
        got, got_idx = ocache.step(q_rot, k_rot, kn, v, cos, sin, top_k)
        torch.cuda.synchronize()
        assert torch.equal(got_idx, want_idx)
        assert torch.equal(got, want)
        assert ocache.length == dcache.length
    kd, vd = dcache.past_key_value
    kh, vh = ocache.host_key_value
    assert torch.equal(kh, kd.cpu()) and torch.equal(vh, vd.cpu())
    assert torch.equal(ocache.landmark_keys.cpu(), kd[:, :, block - 1::block].cpu())
    assert ocache.n_blocks == dcache.length // block
