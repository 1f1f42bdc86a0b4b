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


# ------------------------------------------------- gather + attend over the ring (mem_cache.py:86-109, landmark.py:192-240)
ATTEND_CASES = [
    # capacity, mem_freq, hs, nh, chunks, top_k, T, dtype
    (40, 50, 64, 12, [51 * 64 + 13], 4, 250, torch.bfloat16),       # the benchmark's shape; tail of 13 tokens in front of the chunk
    (40, 50, 64, 12, [51 * 41], 4, 250, torch.bfloat16),            # the same without a tail, ring wrapped by one block
    (6, 50, 64, 4, [51 * 4 + 50], 2, 5, torch.bfloat16),            # the chunk's first token is the tail's landmark
    (6, 31, 128, 2, [32 * 9 + 7], 3, 70, torch.bfloat16),           # blocks of 32 (native slots), head dim 128, wrapped
    (5, 99, 64, 2, [100 * 7 + 40], 2, 130, torch.float16),          # blocks of 100 in 128 slots, f16
    (8, 15, 128, 3, [16 * 11 + 3], 8, 20, torch.bfloat16),          # every filled slot picked
    (4, 63, 64, 2, [64 * 3], 1, 64, torch.bfloat16),                # blocks of 64, top_k 1, ring not yet full
]


@pytest.mark.parametrize("method", omc.METHODS)
@pytest.mark.parametrize("capacity,mem_freq,hs,nh,chunks,top_k,T,dtype", ATTEND_CASES)
def test_attention_over_the_ring_matches_oracle(method, capacity, mem_freq, hs, nh, chunks, top_k, T, dtype):
    # tolerance 2e-2 max abs against the fp32 restatement of retrieve_for_query + CausalSelfAttention.forward on the
    # same 16-bit inputs, with the slots the HIP selection returned (their equality with the oracle's is the test above)
    from landmark_hip.mem_cache import MemLMCacheStorage
    print(f"case attend cap{capacity} freq{mem_freq} hs{hs} nh{nh} chunks{chunks} k{top_k} T{T} {method}", flush=True)
    B, block = 2, mem_freq + 1
    g = torch.Generator().manual_seed(capacity + mem_freq + top_k + T)
    storage = MemLMCacheStorage(B, capacity, mem_freq, nh, hs, dtype=dtype, device=DEV, cache_topk=top_k,
                                cache_selection_method=method)
    ring = omc.RingStore(B, capacity, block, nh, hs, dtype=dtype)
    _fill(storage, ring, B, nh, hs, block, chunks, g, dtype)
    tail = ring.last_incomplete_len
    start = (top_k + 1) * block + tail                              # what MemLMCache.forward hands out (mem_cache.py:188)
    cos, sin = rotary.rotary_tables(start + T, hs, dtype)
    pos = torch.arange(start, start + T)
    q = rotary.apply_rotary((torch.randn(B, nh, T, hs, generator=g) * 0.5).to(dtype), cos, sin, pos)
    k = rotary.apply_rotary((torch.randn(B, nh, T, hs, generator=g) * 0.5).to(dtype), cos, sin, pos)
    v = (torch.randn(B, nh, T, hs, generator=g) * 0.5).to(dtype)
    is_mem = ((torch.arange(T) + tail) % block == block - 1)[None].expand(B, T)
    y, slots = storage.attend(q.to(DEV), k.to(DEV), v.to(DEV), is_mem.to(DEV), cos.to(DEV), sin.to(DEV), start)
    torch.cuda.synchronize()
    assert y.shape == (B, nh, T, hs) and y.dtype == dtype
    slots = omc.expand_slots(slots.cpu(), method, B, nh, T)
    ring32 = omc.RingStore(B, capacity, block, nh, hs)
    ring32.cache_k, ring32.cache_v = ring.cache_k.float(), ring.cache_v.float()
    ring32.pending_k, ring32.pending_v, ring32.pending_is_mem = ring.pending_k.float(), ring.pending_v.float(), ring.pending_is_mem
    ring32.cache_iter, ring32.cache_size = ring.cache_iter, ring.cache_size
    want, _ = omc.attention_with_cache(ring32, q.float(), k.float(), v.float(), is_mem, cos.float(), sin.float(), top_k,
                                       method, start, n_buckets=top_k + (tail + T) // block + 3, slots=slots)
    err = (y.float().cpu() - want).abs().max().item()
    print("   max abs err", err, flush=True)
    assert err <= 2e-2, err


def test_attention_without_cached_blocks_is_the_chunk_behind_its_tail():
    from landmark_hip.mem_cache import MemLMCacheStorage
    B, nh, hs, mem_freq, T = 1, 2, 64, 50, 60
    block = mem_freq + 1
    g = torch.Generator().manual_seed(3)
    storage = MemLMCacheStorage(B, 4, mem_freq, nh, hs, device=DEV, cache_topk=2)
    ring = omc.RingStore(B, 4, block, nh, hs, dtype=torch.bfloat16)
    _fill(storage, ring, B, nh, hs, block, [20], g, torch.bfloat16)
    cos, sin = rotary.rotary_tables(20 + T, hs, torch.bfloat16)
    pos = torch.arange(20, 20 + T)
    q = rotary.apply_rotary((torch.randn(B, nh, T, hs, generator=g) * 0.5).bfloat16(), cos, sin, pos)
    k = rotary.apply_rotary((torch.randn(B, nh, T, hs, generator=g) * 0.5).bfloat16(), cos, sin, pos)
    v = (torch.randn(B, nh, T, hs, generator=g) * 0.5).bfloat16()
    is_mem = ((torch.arange(T) + 20) % block == block - 1)[None]
    y, slots = storage.attend(q.to(DEV), k.to(DEV), v.to(DEV), is_mem.to(DEV), cos.to(DEV), sin.to(DEV), 20)
    assert slots is None
    ring32 = omc.RingStore(B, 4, block, nh, hs)
    ring32.pending_k, ring32.pending_v, ring32.pending_is_mem = ring.pending_k.float(), ring.pending_v.float(), ring.pending_is_mem
    want, _ = omc.attention_with_cache(ring32, q.float(), k.float(), v.float(), is_mem, cos.float(), sin.float(), 2,
                                       "per_token_and_head", 20, n_buckets=6)
    assert (y.float().cpu() - want).abs().max().item() <= 2e-2
    with pytest.raises(AssertionError):                                     # a landmark in the wrong place
        storage.attend(q.to(DEV), k.to(DEV), v.to(DEV), torch.zeros(1, T, dtype=torch.bool, device=DEV), cos.to(DEV),
                       sin.to(DEV), 20)
