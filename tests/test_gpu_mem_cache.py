"""Ring cache of landmark blocks on the GPU (lm_benchmark/models/caches/mem_cache.py:41-158): the HIP
selection against oracle/mem_cache.py, slot for slot (int64, bit-exact; rows with a tie at the k-th
place are compared too, the tie rule being part of the contract), for the three selection methods,
wrapped and unwrapped rings, and the storage bookkeeping against the oracle's RingStore."""
import pytest
import torch

from oracle import mem_cache as omc
from oracle import rotary

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _fill(storage, ring, B, nh, hs, block, chunks, g, dtype):
    seen = 0
    for T in chunks:
        k = torch.randn(B, nh, T, hs, generator=g).to(dtype)
        v = torch.randn(B, nh, T, hs, generator=g).to(dtype)
        im = ((torch.arange(T) + seen) % block == block - 1)[None].expand(B, T)
        ring.store(k, v, im)
        storage.store_in_cache(k.to(DEV), {"v": v.to(DEV), "is_mem": im.to(DEV)})
        seen += T


CASES = [
    # capacity, mem_freq, hs, nh, chunks, top_k, T, dtype
    (6, 50, 64, 4, [51 * 4], 2, 5, torch.bfloat16),                 # not yet full
    (6, 50, 64, 4, [51 * 4, 51 * 4], 2, 5, torch.bfloat16),         # wrapped: oldest block at slot 2
    (6, 50, 64, 4, [51 * 6], 3, 3, torch.bfloat16),                 # filled exactly: next write at slot 0
    (5, 31, 128, 2, [100, 100, 100, 37], 4, 7, torch.bfloat16),     # ragged chunks
    (40, 50, 64, 12, [51 * 64], 4, 250, torch.bfloat16),            # the benchmark's shape: chunk larger than the ring
    (8, 15, 128, 3, [16 * 11], 8, 4, torch.float16),                # top_k == filled blocks
    (200, 3, 64, 2, [4 * 333], 5, 9, torch.bfloat16),               # many small blocks, several turns of the ring
    (4, 50, 64, 2, [51 * 5], 1, 6, torch.bfloat16),                 # top_k 1: no reordering (mem_cache.py:73)
]


@pytest.mark.parametrize("method", omc.METHODS)
@pytest.mark.parametrize("capacity,mem_freq,hs,nh,chunks,top_k,T,dtype", CASES)
def test_selection_matches_oracle(method, capacity, mem_freq, hs, nh, chunks, top_k, T, dtype):
    from landmark_hip.mem_cache import MemLMCacheStorage
    print(f"case cap{capacity} freq{mem_freq} hs{hs} nh{nh} chunks{chunks[:3]} k{top_k} T{T} {method}", flush=True)
    B, block = 2, mem_freq + 1
    g = torch.Generator().manual_seed(capacity + mem_freq + top_k)
    storage = MemLMCacheStorage(B, capacity, mem_freq, nh, hs, dtype=dtype, device=DEV, cache_topk=top_k,
                                cache_selection_method=method)
    ring = omc.RingStore(B, capacity, block, nh, hs, dtype=dtype)
    _fill(storage, ring, B, nh, hs, block, chunks, g, dtype)
    assert (storage.cache_iter, storage.cache_size, storage.last_incomplete_len) == \
        (ring.cache_iter, ring.cache_size, ring.last_incomplete_len)
    n = ring.filled
    assert storage.filled == n
    assert torch.equal(storage.cache_mem_k[:, :n].cpu(), ring.cache_k[:, :n])
    assert torch.equal(storage.cache_mem_v[:, :n].cpu(), ring.cache_v[:, :n])
    assert torch.equal(storage.last_incomplete_k[:, :, :ring.last_incomplete_len].cpu(), ring.pending_k)

    q = torch.randn(B, nh, T, hs, generator=g).to(dtype)
    cos, sin = rotary.rotary_tables((top_k + 1) * block, hs, dtype)
    scores = omc.ring_scores(q, ring.cache_k, n, ring.cache_iter, top_k, cos, sin)
    want = omc.select_blocks(scores, ring.cache_iter, top_k, method)                # (B, nh, T, k)
    got = storage.select_blocks(q.to(DEV), cos.to(DEV), sin.to(DEV)).cpu()
    if method == "max_over_heads":
        assert got.shape == (B, T, top_k)
        got = got[:, None].expand(B, nh, T, top_k)
    elif method == "max_over_tokens":
        assert got.shape == (B, nh, top_k)
        got = got[:, :, None].expand(B, nh, T, top_k)
    assert got.dtype == torch.int64
    assert torch.equal(got, want)
    # positions of the gathered keys (mem_cache.py:95-97)
    pos = storage.key_positions(got.to(DEV)).cpu()
    assert torch.equal(pos, omc.gathered_key_positions(want, n, ring.cache_iter, top_k, block))


def test_selection_errors():
    from landmark_hip import _lib
    from landmark_hip.mem_cache import MemLMCacheStorage
    storage = MemLMCacheStorage(1, 4, 3, 2, 64, device=DEV, cache_topk=3)
    q = torch.zeros(1, 2, 1, 64, dtype=torch.bfloat16, device=DEV)
    cos, sin = (t.to(DEV) for t in rotary.rotary_tables(64, 64, torch.bfloat16))
    with pytest.raises(ValueError):
        storage.select_blocks(q, cos, sin)                                  # empty cache
    k = torch.randn(1, 2, 8, 64).bfloat16().to(DEV)
    im = (torch.arange(8) % 4 == 3)[None].to(DEV)
    storage.store_in_cache(k, {"v": k, "is_mem": im})
    with pytest.raises(_lib.LmkError) as e:                                 # two blocks cached, three asked for
        storage.select_blocks(q, cos, sin)
    assert e.value.code == -10
    with pytest.raises(NotImplementedError):
        MemLMCacheStorage(1, 4, 3, 2, 64, device=DEV, cache_selection_method="mean")
    with pytest.raises(AssertionError):
        storage.store_in_cache(k[:, :, :4], {"v": k[:, :, :4], "is_mem": torch.zeros(1, 4, dtype=torch.bool, device=DEV)})
