"""Host logic of the growing KV cache (CPU tensors; no kernel is launched)."""
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "landmark-attention_amd"))


def test_append_equals_torch_cat_and_views_share_storage():
    from landmark_hip.cache import LandmarkKVCache
    g = torch.Generator().manual_seed(0)
    B, H, D = 2, 3, 16
    cache = LandmarkKVCache(B, H, D, torch.float32, "cpu", capacity=8)
    ks, vs = [], []
    for t in (5, 1, 1, 9, 40, 1):                       # crosses the capacity several times
        k, v = torch.randn(B, H, t, D, generator=g), torch.randn(B, H, t, D, generator=g)
        ks.append(k)
        vs.append(v)
        cache.append(k, v)
        pk, pv = cache.past_key_value
        assert torch.equal(pk, torch.cat(ks, dim=2)) and torch.equal(pv, torch.cat(vs, dim=2))   # llama_mem.py:424-425
        assert pk.stride(3) == 1 and pk.stride(2) == D and pk.stride(1) == cache.capacity * D
    assert cache.length == 57 and cache.capacity >= 57
    # a view, not a copy: rows appended later land in the same buffer
    pk, _ = cache.past_key_value
    before = pk.data_ptr()
    cache.append(torch.zeros(B, H, 1, D), torch.zeros(B, H, 1, D))
    assert cache.past_key_value[0].data_ptr() == before
