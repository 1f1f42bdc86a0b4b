"""Landmarks at irregular positions: blocks of unequal length on the fused kernels.

The reference's fused path rejects such masks (flash_landmark_attention.py:393-394); its high-level path takes
them (llama/llama_mem.py:222-243, lm_benchmark/models/landmark.py:88-119).  Parity is against the fp32
restatement of that path (oracle/highlevel.py, itself pinned against a literal per-row loop in
tests/test_oracle_highlevel.py) on the same 16-bit-rounded inputs: max abs error <= 2e-2 for the output and
for the gradients (autograd through the restatement).
"""
import math

import pytest
import torch

from oracle import highlevel, s1

pytestmark = pytest.mark.gpu

TOL = 2e-2
DEV = "cuda:0"


def _mask(T, seed, lo, hi, tail=0):
    """Blocks of lo..hi tokens, each ending in its landmark; `tail` tokens without one at the end."""
    g = torch.Generator().manual_seed(seed)
    marks, j = [False] * T, 0
    while T - tail - j >= lo:
        n = int(torch.randint(lo, hi + 1, (1,), generator=g))
        n = min(n, T - tail - j)
        if T - tail - (j + n) in range(1, lo):          # what is left would be too short for a block: take it along
            n = T - tail - j
            if n > hi:
                n = n - lo                              # ... or leave a block of lo behind
        j += n
        marks[j - 1] = True
    assert j == T - tail, (j, T, tail)
    return torch.tensor(marks)


def _oracle(q, k, v, is_mem, do=None):
    """fp32 restatement on the 16-bit inputs; with history the queries are the last rows of a full-length run."""
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    qf, kf, vf = (t.float().clone().requires_grad_(do is not None) for t in (q, k, v))
    q_full = torch.cat((torch.zeros(B, H, Lk - Lq, D), qf), dim=2)
    out = highlevel.attention_lm_benchmark(q_full, kf, vf, is_mem[None].expand(B, Lk), n_buckets=int(is_mem.sum()) + 3)
    out = out[:, :, Lk - Lq:]
    if do is None:
        return out.detach()
    return (out.detach(),) + torch.autograd.grad((out * do.float()).sum(), [qf, kf, vf])


CASES = [
    # Lq, Lk, D, lo, hi, tail
    (200, 200, 128, 2, 64, 0),        # blocks of 2..64 tokens in 64 slots
    (300, 300, 128, 20, 128, 0),      # up to 128: 128 slots
    (150, 150, 64, 3, 40, 0),         # head dim 64
    (260, 260, 128, 30, 64, 17),      # a trailing block without landmark (forward only)
    (64, 64, 128, 64, 64, 0),         # one block that fills its slots
]


@pytest.mark.parametrize("Lq,Lk,D,lo,hi,tail", CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_forward_matches_the_high_level_path(Lq, Lk, D, lo, hi, tail, dtype):
    from ltriton.flash_landmark_attention import fused_landmark_attention
    B, H = 2, 3
    print(f"case irregular fwd L{Lk} D{D} blocks {lo}..{hi} tail {tail} {dtype}", flush=True)
    g = torch.Generator().manual_seed(Lk + D + hi)
    q, k, v = ((torch.randn(B, H, L, D, generator=g) * 0.5).to(dtype) for L in (Lq, Lk, Lk))
    is_mem = _mask(Lk, Lk + hi, lo, hi, tail)
    want = _oracle(q, k, v, is_mem)
    with torch.no_grad():
        got = fused_landmark_attention(q.to(DEV), k.to(DEV), v.to(DEV), is_mem.to(DEV), block_size=hi)
    torch.cuda.synchronize()
    assert got.shape == q.shape and got.dtype == dtype
    assert (got.float().cpu() - want).abs().max().item() <= TOL


def test_forward_with_history_blocks():
    from ltriton.flash_landmark_attention import fused_landmark_attention
    B, H, D, Lk = 1, 2, 128, 330
    g = torch.Generator().manual_seed(5)
    is_mem = _mask(Lk, 77, 5, 50)
    ends = [j + 1 for j, m in enumerate(is_mem.tolist()) if m]
    hist = ends[3]                                       # four blocks of history
    Lq = Lk - hist
    q, k, v = ((torch.randn(B, H, L, D, generator=g) * 0.5).bfloat16() for L in (Lq, Lk, Lk))
    want = _oracle(q, k, v, is_mem)
    with torch.no_grad():
        got = fused_landmark_attention(q.to(DEV), k.to(DEV), v.to(DEV), is_mem[None].to(DEV))
        with pytest.raises(AssertionError, match="whole blocks"):
            fused_landmark_attention(q[:, :, 1:].to(DEV), k.to(DEV), v.to(DEV), is_mem[None].to(DEV))
    torch.cuda.synchronize()
    assert (got.float().cpu() - want).abs().max().item() <= TOL


def test_tiny_case_against_the_row_by_row_evaluation():
    from ltriton.flash_landmark_attention import fused_landmark_attention
    D, T = 64, 29
    g = torch.Generator().manual_seed(9)
    q, k, v = ((torch.randn(1, 1, T, D, generator=g) * 0.5).bfloat16() for _ in range(3))
    is_mem = torch.zeros(T, dtype=torch.bool)
    is_mem[[2, 9, 11, 20, 25]] = True                    # blocks of 3, 7, 2, 9, 5 and a tail of 3
    want = torch.tensor(s1.s1_rows_python_irregular(q[0, 0].float(), k[0, 0].float(), v[0, 0].float(), is_mem.tolist()))
    with torch.no_grad():
        got = fused_landmark_attention(q.to(DEV), k.to(DEV), v.to(DEV), is_mem.to(DEV))
    torch.cuda.synchronize()
    assert (got[0, 0].float().cpu() - want).abs().max().item() <= TOL


@pytest.mark.parametrize("Lq,Lk,D,lo,hi", [(200, 200, 128, 2, 64), (256, 256, 128, 20, 128), (150, 150, 64, 3, 40),
                                            (100, 100, 128, 2, 6), (0, 330, 128, 5, 50)])
def test_gradients_match_autograd_through_the_high_level_path(Lq, Lk, D, lo, hi):
    from ltriton.flash_landmark_attention import fused_landmark_attention
    B, H = 2, 2
    print(f"case irregular bwd L{Lk} D{D} blocks {lo}..{hi}", flush=True)
    g = torch.Generator().manual_seed(Lk + D + lo)
    is_mem = _mask(Lk, Lk + lo, lo, hi)
    if Lq == 0:                                          # with history: three blocks in front of the queries
        Lq = Lk - [j + 1 for j, m in enumerate(is_mem.tolist()) if m][2]
    q, k, v = ((torch.randn(B, H, L, D, generator=g) * 0.5).bfloat16() for L in (Lq, Lk, Lk))
    do = torch.randn(B, H, Lq, D, generator=g).bfloat16()
    out_ref, dq_ref, dk_ref, dv_ref = _oracle(q, k, v, is_mem, do)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = fused_landmark_attention(qd, kd, vd, is_mem.to(DEV))
    dq, dk, dv = torch.autograd.grad(out, [qd, kd, vd], do.to(DEV))
    torch.cuda.synchronize()
    assert (out.float().cpu() - out_ref).abs().max().item() <= TOL
    for name, a, b in (("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
        err = (a.float().cpu() - b).abs().max().item()
        assert err <= TOL, (name, err)
    # a landmark's value row never contributes: its gradient is exactly zero
    assert (dv.float().cpu()[:, :, is_mem] == 0).all()


def test_regular_mask_through_the_table_gives_the_bits_of_the_plain_path():
    # the same geometry described twice: blocks of 51 tokens as a block size and as a table of blocks
    from landmark_hip import attention
    B, H, L, D, block = 1, 2, 51 * 6, 128, 51
    g = torch.Generator().manual_seed(3)
    q, k, v = ((torch.randn(B, H, L, D, generator=g) * 0.5).bfloat16().to(DEV) for _ in range(3))
    is_mem = (torch.arange(L) % block == block - 1)
    seg = attention.LandmarkSegments(is_mem.tolist(), torch.device(DEV))
    with torch.no_grad():
        plain = attention.fused_landmark_attention(q, k, v, is_mem.to(DEV), block_size=block)
        table = attention.FusedLandmarkAttentionSegments.apply(q, k, v, seg, 1.0 / math.sqrt(D))
    torch.cuda.synchronize()
    assert torch.equal(plain.view(torch.int16), table.view(torch.int16))
