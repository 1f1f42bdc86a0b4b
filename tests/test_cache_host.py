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


def test_ring_storage_bookkeeping_matches_the_restated_store_in_cache():
    # MemLMCacheStorage.store_in_cache on CPU tensors against oracle/mem_cache.RingStore
    # (lm_benchmark/models/caches/mem_cache.py:111-158): counters and buffer contents after every chunk
    from landmark_hip.mem_cache import MemLMCacheStorage
    from oracle import mem_cache as omc
    for cap, block, chunks in [(4, 3, [3, 3, 6, 3, 9]), (4, 3, [5, 2, 8, 1, 1, 1, 13]), (3, 4, [40]), (3, 4, [4, 20, 4]),
                               (5, 2, [2] * 7)]:
        B, nh, hs = 2, 3, 8
        s = MemLMCacheStorage(B, cap, block - 1, nh, hs, dtype=torch.float32, device="cpu")
        r = omc.RingStore(B, cap, block, nh, hs)
        g = torch.Generator().manual_seed(cap)
        seen = 0
        for T in chunks:
            k, v = torch.randn(B, nh, T, hs, generator=g), torch.randn(B, nh, T, hs, generator=g)
            im = ((torch.arange(T) + seen) % block == block - 1)[None].expand(B, T)
            s.store_in_cache(k, {"v": v, "is_mem": im})
            r.store(k, v, im)
            seen += T
            n = r.filled
            assert (s.cache_iter, s.cache_size, s.last_incomplete_len, s.filled) == \
                (r.cache_iter, r.cache_size, r.last_incomplete_len, n)
            assert torch.equal(s.cache_mem_k[:, :n], r.cache_k[:, :n]) and torch.equal(s.cache_mem_v[:, :n], r.cache_v[:, :n])
            assert torch.equal(s.last_incomplete_k[:, :, :s.last_incomplete_len], r.pending_k)
            assert s.oldest_slot == (int(omc.slot_ages(n, r.cache_iter).argmin()) if n else 0)
        s.clear_state()
        assert (s.cache_iter, s.cache_size, s.last_incomplete_len) == (0, 0, 0)


def test_transposed_rotation_table_gives_the_gradient_of_the_rotary_expression():
    # the gradient of y = x*cos + rotate_half(x)*sin with respect to x is the same expression on dy with the
    # table landmark_hip.rotary._transposed_sin(sin); checked in fp64 against torch autograd with tables whose
    # two halves differ (LLaMA's are equal, which would hide a wrong swap)
    import torch

    from landmark_hip.rotary import _transposed_sin
    from oracle import rotary as orot
    g = torch.Generator().manual_seed(3)
    n, D = 9, 16
    cos, sin = (torch.randn(n, D, generator=g, dtype=torch.float64) for _ in range(2))
    x = torch.randn(2, n, D, generator=g, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(2, n, D, generator=g, dtype=torch.float64)
    y = x * cos + orot.rotate_half(x) * sin
    (want,) = torch.autograd.grad(y, x, dy)
    got = dy * cos + orot.rotate_half(dy) * _transposed_sin(sin)
    assert torch.allclose(got, want, rtol=0, atol=1e-14)
    # LLaMA's tables: the transposed rotation is the rotation by the opposite angle
    c2, s2 = orot.rotary_tables(n, D, torch.float64)
    assert torch.equal(_transposed_sin(s2), -s2)
