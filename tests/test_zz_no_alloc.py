"""The selection entry point that allocates nothing (``lmk_retrieve_topk_static``): its workspace is a
fixed array of device memory inside the library.  Called through the C ABI, its indices must equal, bit for
bit, those of ``lmk_retrieve_topk`` with a caller-owned workspace -- on two calls in a row, the second with
a smaller input (the array keeps the first call's contents), and then once more at the first size."""
import pytest
import torch

from oracle import retrieval as oret
from oracle import rotary as orot

pytestmark = pytest.mark.gpu


def _case(B, H, T, S, D, block, top_k, seed):
    from landmark_hip import _lib
    lib = _lib.lib()
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, H, T, D, generator=g) * 0.5).bfloat16()
    kc = (torch.randn(B, H, S, D, generator=g) * 0.5).bfloat16()
    cos, sin = orot.rotary_tables(S + T, D, torch.bfloat16)
    want = oret.select_topk(oret.landmark_scores(q, kc, cos, sin, block, top_k), min(top_k, S // block))
    qd, kd, cd, sd = q.cuda(), kc.cuda(), cos.cuda(), sin.cuda()
    k = min(top_k, S // block)
    stream = _lib.current_stream(qd.device)
    head = (_lib.tensor4(qd), _lib.tensor4(kd), cd.data_ptr(), sd.data_ptr(), cd.stride(0), cd.shape[0])
    tail = (B, H, T, S, D, block, top_k, 0, stream)
    nbytes = lib.lmk_retrieve_workspace_bytes(B, H, T, S, D, block)
    assert nbytes <= lib.lmk_retrieve_static_max_bytes()
    ws = torch.empty(nbytes, device=qd.device, dtype=torch.uint8)
    ref = torch.full((B, H, T, k), -1, device=qd.device, dtype=torch.int64)
    _lib.check(lib.lmk_retrieve_topk(*head, ref.data_ptr(), ws.data_ptr(), nbytes, *tail))
    got = torch.full((B, H, T, k), -1, device=qd.device, dtype=torch.int64)
    _lib.check(lib.lmk_retrieve_topk_static(*head, got.data_ptr(), *tail))
    torch.cuda.synchronize()
    assert torch.equal(got, ref), "static-scratch entry point differs from lmk_retrieve_topk"
    assert torch.equal(got.cpu(), want), "indices differ from the oracle"


def test_static_scratch_selection_matches_the_workspace_entry_point():
    print("no-alloc: decode-sized call, smaller call, first size again", flush=True)
    _case(1, 32, 1, 1024 * 32 + 7, 128, 32, 4, seed=1)      # one token per head against 1024 blocks and a tail
    _case(1, 4, 3, 200 * 32, 128, 32, 5, seed=2)            # smaller: reads and writes a prefix of the same array
    _case(1, 32, 1, 1024 * 32 + 7, 128, 32, 4, seed=3)
    _case(2, 2, 40, 300 * 16, 64, 16, 3, seed=4)            # a chunk of queries: the fused score + select kernel


def test_static_scratch_rejects_sizes_beyond_its_array():
    from landmark_hip import _lib
    lib = _lib.lib()
    B, H, T, S, D, block, top_k = 1, 32, 256, 32768, 128, 32, 4       # benchmark config 4: two 33.5 MB score planes
    assert lib.lmk_retrieve_workspace_bytes(B, H, T, S, D, block) > lib.lmk_retrieve_static_max_bytes()
    q = torch.zeros(B, H, T, D, dtype=torch.bfloat16, device="cuda")
    kc = torch.zeros(B, H, S, D, dtype=torch.bfloat16, device="cuda")
    cos = torch.zeros(S + T, D, dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros(B, H, T, top_k, dtype=torch.int64, device="cuda")
    rc = lib.lmk_retrieve_topk_static(_lib.tensor4(q), _lib.tensor4(kc), cos.data_ptr(), cos.data_ptr(), D, S + T,
                                      idx.data_ptr(), B, H, T, S, D, block, top_k, 0, None)
    assert rc == -8
    with pytest.raises(_lib.LmkError):
        _lib.check(rc)


def test_static_scratch_selection_replays_from_a_graph():
    # the array's address is resolved before the capture (lmk_retrieve_static_init); the captured call must then
    # reproduce lmk_retrieve_topk on every replay, with eager work and new inputs in between
    from landmark_hip import _lib
    lib = _lib.lib()
    _lib.check(lib.lmk_retrieve_static_init())
    B, H, T, S, D, block, top_k = 1, 8, 1, 64 * 32 + 5, 128, 32, 4
    g = torch.Generator().manual_seed(11)
    mk = lambda *s_: (torch.randn(*s_, generator=g) * 0.5).bfloat16().cuda()
    q, kc = mk(B, H, T, D), mk(B, H, S, D)
    cos, sin = (t.cuda() for t in orot.rotary_tables(S + T, D, torch.bfloat16))
    nbytes = lib.lmk_retrieve_workspace_bytes(B, H, T, S, D, block)
    ws = torch.empty(nbytes, device="cuda", dtype=torch.uint8)
    ref = torch.empty((B, H, T, top_k), device="cuda", dtype=torch.int64)
    got = torch.empty_like(ref)

    def eager_ref():
        _lib.check(lib.lmk_retrieve_topk(_lib.tensor4(q), _lib.tensor4(kc), cos.data_ptr(), sin.data_ptr(), cos.stride(0),
                                         cos.shape[0], ref.data_ptr(), ws.data_ptr(), nbytes, B, H, T, S, D, block, top_k, 0,
                                         _lib.current_stream(q.device)))

    def static_call():
        _lib.check(lib.lmk_retrieve_topk_static(_lib.tensor4(q), _lib.tensor4(kc), cos.data_ptr(), sin.data_ptr(),
                                                cos.stride(0), cos.shape[0], got.data_ptr(), B, H, T, S, D, block, top_k, 0,
                                                _lib.current_stream(q.device)))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        static_call()                                            # kernel attributes are set outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call()
    for rep in range(4):
        if rep:
            q.copy_(mk(B, H, T, D))                              # new queries in the captured buffer
        eager_ref()
        got.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, ref), rep
