"""Retrieval parity: top-k block indices bit-exact against the oracle's score/selection
contract, and gather+attend output within 2e-2 of the oracle (both the model-dtype
restatement of the reference and the fp32 closed form)."""
import pytest
import torch

from oracle import retrieval as oret
from oracle import rotary as orot

pytestmark = pytest.mark.gpu


def _inputs(B, H, T, S, D, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.5).to(dtype)
    q, kc, vc, kl, vl = mk(B, H, T, D), mk(B, H, S, D), mk(B, H, S, D), mk(B, H, T, D), mk(B, H, T, D)
    cos, sin = orot.rotary_tables(S + T, D, dtype)
    return q, kc, vc, kl, vl, cos, sin


CASES = [
    # B, H, T, S, D, block, top_k
    (1, 2, 8, 64 * 32, 128, 32, 4),
    (2, 3, 40, 20 * 32, 128, 32, 5),
    (1, 2, 16, 3 * 32, 128, 32, 5),        # fewer cached blocks than top_k
    (1, 2, 130, 33 * 32, 128, 32, 1),      # ragged landmark tile, ragged query tile
    (1, 2, 64, 40 * 64, 128, 64, 4),
    (1, 2, 32, 50 * 32, 64, 32, 4),
    (1, 2, 16, 70 * 16, 128, 16, 3),       # selection does not depend on the block size set of the attend kernels
    (1, 2, 40, 2500 * 32, 128, 32, 5),     # more than 1024 cached blocks: three segments, the last one ragged
    (1, 1, 3, 2048 * 16, 128, 16, 64),     # two full segments, the longest list to merge
    (1, 2, 1, 3000 * 32, 64, 32, 4),       # one query against a long cache
    (1, 2, 3, 1024 * 32, 128, 32, 64),     # few rows: four slices of 256 blocks, 256 candidates to merge
    (1, 1, 5, 4100 * 16, 128, 16, 60),     # few rows, 17 slices x 60 > 1024 candidates: back on the fused kernel
    (36, 32, 1, 20 * 32, 128, 32, 4),      # batched decoding: more than 1024 rows but one per head: still by slices
    (20, 32, 2, 300 * 32, 64, 32, 5),      # two per head, two slices
    # more than 1024 query rows (B * H * T): the fused score + select kernel
    (1, 2, 530, 33 * 32, 128, 32, 1),
    (2, 3, 200, 20 * 32, 128, 32, 5),
    (1, 2, 520, 50 * 32, 64, 32, 4),
    (1, 2, 520, 2500 * 32, 128, 32, 5),
    (1, 1, 1030, 2048 * 16, 128, 16, 64),
]


@pytest.mark.parametrize("B,H,T,S,D,block,top_k", CASES)
def test_topk_indices_bit_exact(B, H, T, S, D, block, top_k):
    from landmark_hip.retrieval import retrieve_topk
    print(f"case B{B} H{H} T{T} S{S} D{D} bs{block} k{top_k}", flush=True)
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=S + T)
    sc = oret.landmark_scores(q, kc, cos, sin, block, top_k)
    want = oret.select_topk(sc, min(top_k, S // block))
    got = retrieve_topk(q.cuda(), kc.cuda(), cos.cuda(), sin.cuda(), block, top_k)
    torch.cuda.synchronize()
    assert got.dtype == torch.int64 and got.shape == want.shape
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("T", [8, 520])                             # few rows: sliced kernel; many: fused kernel
def test_topk_with_massive_ties(T):
    # identical landmark keys in many blocks: every score ties, the lowest indices must win
    from landmark_hip.retrieval import retrieve_topk
    B, H, S, D, block, top_k = 1, 2, 2100 * 32, 128, 32, 4          # > 1024 landmarks: two list sweeps / nine slices
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=3)
    kc[:, :, block - 1::block] = kc[:, :, block - 1:block]
    sc = oret.landmark_scores(q, kc, cos, sin, block, top_k)
    want = oret.select_topk(sc, top_k)
    got = retrieve_topk(q.cuda(), kc.cuda(), cos.cuda(), sin.cuda(), block, top_k)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("T", [40, 520])                            # few rows: sliced kernel; many: fused kernel
@pytest.mark.parametrize("n_mems,top_k", [(700, 4), (1024, 64), (130, 7)])
def test_topk_ties_inside_one_workgroup(n_mems, top_k, T):
    # at most 1024 landmarks: scores stay on the CU; identical landmark keys make every block a
    # contender, so the contender list is flushed several times, and a large top_k runs many rounds
    from landmark_hip.retrieval import retrieve_topk
    B, H, D, block = 1, 2, 128, 32
    S = n_mems * block
    print(f"case ties n_mems{n_mems} k{top_k}", flush=True)
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=n_mems)
    kc[:, :, block - 1::block] = kc[:, :, block - 1:block]
    if n_mems == 1024:                                   # half tied, half distinct
        kc[:, :, block - 1::2 * block] = (torch.randn(B, H, n_mems // 2, D) * 0.5).to(kc.dtype)
    sc = oret.landmark_scores(q, kc, cos, sin, block, top_k)
    want = oret.select_topk(sc, top_k)
    got = retrieve_topk(q.cuda(), kc.cuda(), cos.cuda(), sin.cuda(), block, top_k)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("T", [24, 520])
def test_fp16_indices_bit_exact(T):
    from landmark_hip.retrieval import retrieve_topk
    B, H, S, D, block, top_k = 1, 2, 48 * 32, 128, 32, 4
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=4, dtype=torch.float16)
    want = oret.select_topk(oret.landmark_scores(q, kc, cos, sin, block, top_k), top_k)
    got = retrieve_topk(q.cuda(), kc.cuda(), cos.cuda(), sin.cuda(), block, top_k)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,H,T,S,block,top_k", [(1, 2, 64, 24 * 32, 32, 4), (1, 2, 128, 12 * 64, 64, 3),
                                                  (2, 2, 96, 3 * 32, 32, 5),
                                                  (1, 2, 1, 24 * 32, 32, 4),      # decode: first token of a new block
                                                  (1, 2, 5, 12 * 64, 64, 3),
                                                  (1, 2, 160, 9 * 128, 128, 3), (2, 2, 7, 2 * 128, 128, 4)])
def test_gather_attend_matches_oracle(B, H, T, S, block, top_k, D):
    from landmark_hip.retrieval import retrieve_and_attend
    print(f"case gather B{B} H{H} T{T} S{S} bs{block} k{top_k} D{D}", flush=True)
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=S + T + 1)
    is_mem = (torch.arange(T) % block == block - 1)[None].expand(B, T)
    ref_bf16, idx_ref = oret.retrieve_and_attend(q, kc, vc, kl, vl, is_mem, cos, sin, block, top_k)
    dev = lambda t: t.cuda()
    out, idx = retrieve_and_attend(dev(q), (dev(kc), dev(vc)), dev(kl), dev(vl), dev(cos), dev(sin), block, top_k)
    torch.cuda.synchronize()
    assert torch.equal(idx.cpu(), idx_ref)
    out = out.float().cpu()
    assert (out - ref_bf16.float()).abs().max().item() <= 2e-2
    ref32 = oret.retrieve_and_attend_s1(q, kc, vc, kl, vl, cos, sin, block, top_k, idx_ref,
                                        heads=[0, H - 1],
                                        tokens=sorted({t for t in (0, 1, block - 2, block - 1, block, T - 1) if 0 <= t < T}))
    for (b, h, t), o in ref32.items():
        assert (out[b, h, t] - o).abs().max().item() <= 2e-2, (b, h, t)


# cache ending in an incomplete block: the state between two landmarks while decoding
# (llama_mem.py:321-342).  inc = S % block cached tail tokens, T new tokens, T + inc <= block.
@pytest.mark.parametrize("n_mems,inc,T,block,top_k", [
    (20, 7, 1, 32, 4),          # decode by one token
    (20, 31, 1, 32, 4),         # the new token is the block's landmark: it does not see itself
    (20, 1, 31, 32, 4),         # a chunk that completes the block
    (20, 10, 12, 32, 4),
    (3, 5, 2, 32, 5),           # fewer complete blocks than top_k
    (12, 40, 24, 64, 3),        # block 64, ends on the landmark
    (12, 17, 1, 64, 3),
    (7, 100, 28, 128, 2),       # block 128, ends on the landmark
    (7, 5, 1, 128, 4),
])
@pytest.mark.parametrize("D", [128, 64])
def test_incomplete_cached_block(n_mems, inc, T, block, top_k, D):
    from landmark_hip.retrieval import retrieve_and_attend
    B, H = 2, 3
    S = n_mems * block + inc
    print(f"case tail n_mems{n_mems} inc{inc} T{T} bs{block} k{top_k} D{D}", flush=True)
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=S + T + 2)
    is_mem = ((torch.arange(T) + inc) % block == block - 1)[None].expand(B, T)
    ref_bf16, idx_ref = oret.retrieve_and_attend(q, kc, vc, kl, vl, is_mem, cos, sin, block, top_k)
    dev = lambda t: t.cuda()
    out, idx = retrieve_and_attend(dev(q), (dev(kc), dev(vc)), dev(kl), dev(vl), dev(cos), dev(sin), block, top_k)
    torch.cuda.synchronize()
    assert torch.equal(idx.cpu(), idx_ref)
    out = out.float().cpu()
    assert (out - ref_bf16.float()).abs().max().item() <= 2e-2
    ref32 = oret.retrieve_and_attend_s1(q, kc, vc, kl, vl, cos, sin, block, top_k, idx_ref,
                                        heads=[0, H - 1], tokens=sorted({0, T // 2, T - 1}))
    for (b, h, t), o in ref32.items():
        assert (out[b, h, t] - o).abs().max().item() <= 2e-2, (b, h, t)


# A handful of new tokens whose window stays inside one block: the gather kernel attends to the window itself
# (no window, no forward launch).  Window filling the block with the last new token its landmark; a fresh block;
# one block per row (no split over waves); more than 1024 rows (a wave per row); fp16; head dim 64.
# Blocks of 64 (the reference's default) and 128: the window is one or two chunks of 64 keys.
@pytest.mark.parametrize("n_mems,inc,T,top_k,B,H,D,dtype,block", [
    (20, 28, 4, 4, 2, 3, 128, torch.bfloat16, 32),
    (20, 0, 4, 4, 2, 3, 128, torch.bfloat16, 32),
    (10, 29, 3, 1, 2, 3, 128, torch.bfloat16, 32),
    (10, 13, 3, 4, 12, 32, 128, torch.bfloat16, 32),
    (20, 30, 2, 4, 1, 2, 128, torch.float16, 32),
    (20, 27, 4, 5, 2, 3, 64, torch.bfloat16, 32),
    (12, 60, 4, 3, 2, 3, 128, torch.bfloat16, 64),     # fills the block: the last new token is its landmark
    (12, 0, 2, 3, 2, 3, 128, torch.bfloat16, 64),
    (12, 33, 1, 3, 12, 32, 64, torch.float16, 64),     # a wave per row
    (300, 41, 1, 4, 1, 4, 128, torch.bfloat16, 64),    # two slices to merge
    (7, 125, 3, 2, 2, 3, 128, torch.bfloat16, 128),    # second chunk of the window, ends on the landmark
    (7, 40, 2, 4, 1, 2, 64, torch.bfloat16, 128),      # window inside the first chunk
])
def test_decode_rows_attend_to_their_local_window_inside_the_gather(n_mems, inc, T, top_k, B, H, D, dtype, block):
    from landmark_hip.retrieval import gather_attend, retrieve_and_attend
    S = n_mems * block + inc
    print(f"case local n_mems{n_mems} inc{inc} T{T} k{top_k} B{B} H{H} D{D} {dtype} bs{block}", flush=True)
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=S + T + 5, dtype=dtype)
    is_mem = ((torch.arange(T) + inc) % block == block - 1)[None].expand(B, T)
    ref, idx_ref = oret.retrieve_and_attend(q, kc, vc, kl, vl, is_mem, cos, sin, block, top_k)
    dev = lambda t: t.cuda()
    out, idx = retrieve_and_attend(dev(q), (dev(kc), dev(vc)), dev(kl), dev(vl), dev(cos), dev(sin), block, top_k)
    out2 = gather_attend(dev(q), dev(kc), dev(vc), idx, dev(kl), dev(vl), dev(cos), dev(sin), block, top_k)
    torch.cuda.synchronize()
    assert torch.equal(idx.cpu(), idx_ref)
    assert (out.float().cpu() - ref.float()).abs().max().item() <= 2e-2
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))     # the attend step by itself: same kernel
    ref32 = oret.retrieve_and_attend_s1(q, kc, vc, kl, vl, cos, sin, block, top_k, idx_ref,
                                        heads=[0, H - 1], tokens=sorted({0, T - 1}))
    for (b, h, t), o in ref32.items():
        assert (out.float().cpu()[b, h, t] - o).abs().max().item() <= 2e-2, (b, h, t)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_local_window_rows_bit_exact(dtype):
    # the window builder alone: rotated tail keys bit for bit, values and new rows copied, zero query rows
    from landmark_hip import _lib
    B, H, T, D, block, inc = 1, 2, 3, 128, 32, 6
    S = 4 * block + inc
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=77, dtype=dtype)
    k_ref, v_ref = oret.local_window(kc, vc, kl, vl, cos, sin, block)
    dev = lambda t: t.cuda()
    qd, kcd, vcd, kld, vld, cd, sd = map(dev, (q, kc, vc, kl, vl, cos, sin))
    qw, kw, vw = (torch.full((B, H, inc + T, D), 3.0, device="cuda:0", dtype=q.dtype) for _ in range(3))
    T4 = _lib.tensor4
    _lib.check(_lib.lib().lmk_local_window(T4(qd), T4(kcd), T4(vcd), T4(kld), T4(vld), cd.data_ptr(), sd.data_ptr(),
                                           cd.stride(0), cd.shape[0], T4(qw), T4(kw), T4(vw), B, H, T, S, D, block,
                                           _lib.DTYPE_CODES[dtype], _lib.current_stream(qd.device)))
    torch.cuda.synchronize()
    assert torch.equal(kw.cpu(), k_ref) and torch.equal(vw.cpu(), v_ref)
    assert torch.equal(qw.cpu()[:, :, inc:], q) and (qw.cpu()[:, :, :inc] == 0).all()


SHARED_CASES = [
    # B, H, T, n_mems, inc, D, block, top_k, dtype, scale
    (1, 2, 8, 64, 0, 128, 32, 4, torch.bfloat16, 0.5),
    (2, 3, 40, 20, 0, 128, 32, 5, torch.bfloat16, 0.5),
    (1, 2, 16, 3, 0, 128, 32, 5, torch.bfloat16, 0.5),       # fewer cached blocks than top_k
    (1, 2, 100, 1500, 0, 128, 32, 4, torch.bfloat16, 0.5),   # more blocks than one sweep of 1024, ragged lanes
    (1, 2, 64, 40, 0, 128, 64, 3, torch.bfloat16, 0.5),
    (1, 2, 32, 50, 0, 64, 32, 4, torch.bfloat16, 0.5),
    (1, 2, 24, 70, 0, 128, 32, 4, torch.float16, 0.5),       # fp16 probabilities reach the subnormal range
    (1, 2, 24, 300, 0, 128, 32, 8, torch.bfloat16, 6.0),     # peaked softmax: probabilities down to subnormals and zero
    (1, 2, 1, 300, 0, 128, 32, 8, torch.bfloat16, 6.0),      # one query: the head's vector is that query's probabilities
    (1, 2, 5, 17, 9, 128, 32, 4, torch.bfloat16, 0.5),       # cache ends in an incomplete block
    (1, 3, 1, 33, 31, 128, 32, 2, torch.bfloat16, 0.5),      # decode step that lands on the landmark
    (1, 2, 20, 12, 40, 128, 64, 3, torch.float16, 0.5),
    (1, 1, 70, 1100, 0, 64, 32, 4, torch.bfloat16, 0.5),     # 32 probabilities per lane; a second, partial group of 64 queries
    (1, 1, 5, 2100, 0, 64, 32, 4, torch.float16, 0.5),       # more blocks than a wave holds in registers
    (1, 2, 140, 40, 0, 128, 32, 4, torch.float16, 0.5),      # enough queries for the fp32 copy of the keys (as the 70 above)
    (2, 2, 200, 70, 0, 128, 64, 4, torch.bfloat16, 0.5),
]


@pytest.mark.parametrize("B,H,T,n_mems,inc,D,block,top_k,dtype,scale", SHARED_CASES)
def test_selection_shared_by_the_queries_of_a_head(B, H, T, n_mems, inc, D, block, top_k, dtype, scale):
    # aggregate == "max_over_tokens" (llama_mem.py:373-377): indices bit for bit, attention within 2e-2 of the
    # fp32 closed form with the selected blocks as history and of the model-dtype high-level restatement
    from landmark_hip.retrieval import retrieve_and_attend
    S = n_mems * block + inc
    print(f"case B{B} H{H} T{T} n_mems{n_mems} inc{inc} D{D} bs{block} k{top_k} {dtype} x{scale}", flush=True)
    g = torch.Generator().manual_seed(S + T)
    mk = lambda *s, a=0.5: (torch.randn(*s, generator=g) * a).to(dtype)
    q, kc, vc, kl, vl = mk(B, H, T, D, a=scale), mk(B, H, S, D, a=scale), mk(B, H, S, D), mk(B, H, T, D), mk(B, H, T, D)
    cos, sin = orot.rotary_tables(S + T, D, dtype)
    k = min(top_k, n_mems)
    sc = oret.landmark_scores(q, kc, cos, sin, block, top_k)
    agg = oret.aggregate_max_over_tokens(sc)
    want = oret.select_topk(agg, k)
    dev = lambda t: t.cuda()
    out, idx = retrieve_and_attend(dev(q), (dev(kc), dev(vc)), dev(kl), dev(vl), dev(cos), dev(sin), block, top_k,
                                   aggregate="max_over_tokens")
    torch.cuda.synchronize()
    assert idx.shape == (B, H, 1, k) and idx.dtype == torch.int64
    assert torch.equal(idx.cpu(), want)
    # the vector the selection ran on, bit for bit (exponential, order of the sum, division, rounding, maximum)
    from landmark_hip.retrieval import retrieve_topk
    idx2, probs = retrieve_topk(dev(q), dev(kc), dev(cos), dev(sin), block, top_k, aggregate="max_over_tokens",
                                return_block_probs=True)
    assert torch.equal(idx2, idx) and torch.equal(probs.cpu().view(torch.int16), agg.view(torch.int16))
    # the library expression agrees on heads where its values equal the contract's and the k-th place is not tied
    lib = torch.softmax(sc, dim=-1, dtype=torch.float32).to(dtype).amax(dim=2, keepdim=True)
    ok = ~oret.boundary_tie_rows(lib, k) & (lib == agg).all(-1)
    assert torch.equal(idx.cpu()[ok], lib.topk(k, dim=-1).indices.sort(-1).values[ok])
    ref32 = oret.retrieve_and_attend_shared_s1(q, kc, vc, kl, vl, cos, sin, block, top_k, want)
    assert (out.float().cpu() - ref32).abs().max().item() <= 2e-2
    if scale > 1:            # scores of magnitude 100: their 16-bit rounding alone moves the high-level path's weights
        return
    is_mem = ((torch.arange(T) + inc) % block == block - 1)[None].expand(B, T)
    ref16, _ = oret.retrieve_and_attend_shared(q, kc, vc, kl, vl, is_mem, cos, sin, block, top_k, idx=want,
                                               n_buckets=max(64, k + T // block + 2))
    assert (out.float().cpu() - ref16.float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gather_window_rows_bit_exact(dtype):
    # the builder alone: selected keys rotated at their slot positions bit for bit, values copied, then tail and chunk
    from landmark_hip import _lib
    B, H, T, D, block, inc, top_k, n_mems = 1, 2, 3, 128, 32, 6, 3, 9
    S = n_mems * block + inc
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=78, dtype=dtype)
    idx = torch.tensor([[0, 6, 8], [2, 3, 7]]).view(B, H, 1, top_k)      # 6.. are among the newest three: bumped
    k_ref, v_ref = oret.shared_window(kc, vc, kl, vl, idx, cos, sin, block, top_k)
    dev = lambda t: t.cuda()
    qd, kcd, vcd, kld, vld, cd, sd, idxd = map(dev, (q, kc, vc, kl, vl, cos, sin, idx))
    W = top_k * block + inc + T
    qw = torch.full((B, H, inc + T, D), 3.0, device="cuda:0", dtype=q.dtype)
    kw, vw = (torch.full((B, H, W, D), 3.0, device="cuda:0", dtype=q.dtype) for _ in range(2))
    T4 = _lib.tensor4
    _lib.check(_lib.lib().lmk_gather_window(T4(qd), T4(kcd), T4(vcd), idxd.data_ptr(), T4(kld), T4(vld), cd.data_ptr(),
                                            sd.data_ptr(), cd.stride(0), cd.shape[0], T4(qw), T4(kw), T4(vw), B, H, T, S,
                                            D, block, top_k, _lib.DTYPE_CODES[dtype], _lib.current_stream(qd.device)))
    torch.cuda.synchronize()
    assert torch.equal(kw.cpu(), k_ref) and torch.equal(vw.cpu(), v_ref)
    assert torch.equal(qw.cpu()[:, :, inc:], q) and (qw.cpu()[:, :, :inc] == 0).all()


def test_reusing_rotated_landmark_keys_between_landmarks():
    # decode steps between two landmarks: the number of complete blocks, hence every landmark position, stays
    # put, and the second call may skip the rotation (other queries, another T, a longer tail)
    from landmark_hip import _lib
    from landmark_hip.retrieval import retrieve_topk
    B, H, D, block, top_k = 1, 3, 128, 32, 4
    S = 50 * block + 3
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, 5, S + 8, D, seed=91)
    dev = lambda t: t.cuda()
    kcd, cd, sd = dev(kc), dev(cos), dev(sin)
    ws = torch.empty(_lib.lib().lmk_retrieve_workspace_bytes(B, H, 5, S + 8, D, block), device="cuda:0", dtype=torch.uint8)
    first = retrieve_topk(dev(q), kcd[:, :, :S], cd, sd, block, top_k, workspace=ws)
    assert torch.equal(first.cpu(), oret.select_topk(oret.landmark_scores(q, kc[:, :, :S], cos, sin, block, top_k), top_k))
    q2 = q[:, :, :2] * 1.5
    again = retrieve_topk(dev(q2), kcd[:, :, : S + 8], cd, sd, block, top_k, workspace=ws, reuse_landmark_keys=True)
    want = oret.select_topk(oret.landmark_scores(q2, kc[:, :, : S + 8], cos, sin, block, top_k), top_k)
    assert torch.equal(again.cpu(), want)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_baseline_config4_full_size(seed):
    # benchmark config 4: H32 D128, 32768 cached tokens = 1024 blocks of 32, 256 queries, top-4
    # (seed 0 is the benchmark's, 1 and 2 for robustness)
    from landmark_hip.retrieval import retrieve_and_attend
    B, H, T, S, D, block, top_k = 1, 32, 256, 32768, 128, 32, 4
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=seed)
    sc = oret.landmark_scores(q, kc, cos, sin, block, top_k)
    want = oret.select_topk(sc, top_k)
    ties = oret.boundary_tie_rows(sc, top_k)
    dev = lambda t: t.cuda()
    out, idx = retrieve_and_attend(dev(q), (dev(kc), dev(vc)), dev(kl), dev(vl), dev(cos), dev(sin), block, top_k)
    torch.cuda.synchronize()
    print("config4 rows", ties.numel(), "rows with a tie at the 4th place", int(ties.sum()), flush=True)
    assert torch.equal(idx.cpu(), want)
    # torch.topk agrees wherever the k-th place is not tied
    tk = sc.float().topk(top_k, dim=-1).indices.sort(-1).values
    assert torch.equal(idx.cpu()[~ties], tk[~ties])
    # attend: fp32 closed form on sampled (head, token) pairs
    ref32 = oret.retrieve_and_attend_s1(q, kc, vc, kl, vl, cos, sin, block, top_k, want,
                                        heads=[0, 13, 31], tokens=[0, 30, 31, 32, 100, 255])
    out = out.float().cpu()
    for (b, h, t), o in ref32.items():
        assert (out[b, h, t] - o).abs().max().item() <= 2e-2, (b, h, t)


@pytest.mark.parametrize("T,n_mems", [(8, 64), (520, 64), (40, 2500)])   # sliced, fused, segmented selection
def test_nan_queries_keep_indices_inside_the_cache(T, n_mems):
    # a NaN score wins no comparison, so a row of NaN scores picks nothing: the indices written must still
    # be block numbers of the cache (the gather follows them), and the output is NaN rather than a fault
    from landmark_hip.retrieval import retrieve_and_attend
    B, H, D, block, top_k = 1, 2, 128, 32, 4
    S = n_mems * block
    print(f"case nan T{T} n_mems{n_mems}", flush=True)
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=11)
    q[:, 0] = float("nan")                                           # head 0: every score NaN; head 1 untouched
    out, idx = retrieve_and_attend(q.cuda(), (kc.cuda(), vc.cuda()), kl.cuda(), vl.cuda(), cos.cuda(), sin.cuda(),
                                   block, top_k)
    torch.cuda.synchronize()
    idx = idx.cpu()
    assert int(idx.min()) >= 0 and int(idx.max()) < n_mems
    assert torch.isnan(out[:, 0].float()).all()
    sc = oret.landmark_scores(q[:, 1:], kc[:, 1:], cos, sin, block, top_k)
    assert torch.equal(idx[:, 1:], oret.select_topk(sc, top_k))
    assert torch.isfinite(out[:, 1].float()).all()


def test_gather_clamps_indices_outside_the_cache():
    # idx is a caller's array at the C ABI: values outside 0 .. num_mems-1 are read as the nearest block
    from landmark_hip.retrieval import gather_attend
    B, H, T, n_mems, D, block, top_k = 1, 2, 16, 40, 128, 32, 4
    S = n_mems * block
    q, kc, vc, kl, vl, cos, sin = _inputs(B, H, T, S, D, seed=12)
    dev = [t.cuda() for t in (q, kc, vc)]
    bad = torch.tensor([-7, 3, n_mems + 5, 2 ** 31 - 1]).expand(B, H, T, top_k).contiguous()
    clamped = bad.clamp(0, n_mems - 1)
    got = gather_attend(*dev, bad.cuda(), kl.cuda(), vl.cuda(), cos.cuda(), sin.cuda(), block, top_k)
    want = gather_attend(*dev, clamped.cuda(), kl.cuda(), vl.cuda(), cos.cuda(), sin.cuda(), block, top_k)
    torch.cuda.synchronize()
    assert torch.isfinite(got.float()).all()
    assert torch.equal(got, want)


# The one-call step of a decode loop runs the selection's slice step and lets the gather pick a row's k best from the
# slices' candidates (and attend to the row's local window); the separate calls run slice step, merge and gather as
# three launches.  Same indices, same output bits -- with a candidate per lane (<= 64) and with several per lane.
@pytest.mark.parametrize("n_mems,inc,T,top_k,reuse", [(1024, 7, 1, 4, True), (1024, 0, 3, 32, False),
                                                      (700, 31, 1, 40, True), (40, 5, 2, 4, False)])
def test_one_call_decode_step_equals_the_separate_calls(n_mems, inc, T, top_k, reuse):
    from landmark_hip import _lib
    from landmark_hip.retrieval import gather_attend, retrieve_and_attend, retrieve_topk
    B, H, D, block = 1, 3, 128, 32
    S = n_mems * block + inc
    print(f"case one-call n_mems{n_mems} inc{inc} T{T} k{top_k} reuse{reuse}", flush=True)
    q, kc, vc, kl, vl, cos, sin = (t.cuda() for t in _inputs(B, H, T, S, D, seed=n_mems + top_k))
    ws = torch.empty(_lib.lib().lmk_retrieve_workspace_bytes(B, H, T, S, D, block), device="cuda", dtype=torch.uint8)
    idx2 = retrieve_topk(q, kc, cos, sin, block, top_k, workspace=ws)
    out2 = gather_attend(q, kc, vc, idx2, kl, vl, cos, sin, block, top_k)
    out1, idx1 = retrieve_and_attend(q, (kc, vc), kl, vl, cos, sin, block, top_k, workspace=ws, reuse_landmark_keys=reuse)
    torch.cuda.synchronize()
    assert torch.equal(idx1, idx2)
    assert torch.equal(out1.view(torch.int16), out2.view(torch.int16))
