"""Backward parity: dQ, dK, dV of the HIP kernels against autograd through the fp32
closed form on the CPU, same 16-bit-rounded inputs.

Tolerance: max abs error <= 2e-2 (the bound the task states; the reference compares its
own gradients at rtol=atol=4e-2 and only prints, test_flash_landmark_attention.py:156-165).
"""
import pytest
import torch

from tests.util import make_qkv, oracle_grads

pytestmark = pytest.mark.gpu

TOL = 2e-2


@pytest.fixture(params=["recompute", "handover"])
def bwd_path(request, monkeypatch):
    """Both backward paths of block 32: the kernels that form dS twice, and the hand-over of dS tiles from the
    dQ kernel to the dK/dV kernel (chosen by the size of the workspace the shim allocates)."""
    from landmark_hip import attention
    monkeypatch.setattr(attention, "HANDOVER_MAX_BYTES", 0 if request.param == "recompute" else 1 << 40)
    monkeypatch.setattr(attention, "HANDOVER_MIN_KEYS", 0)
    return request.param


def _grads(q, k, v, do, block, scale=None):
    from ltriton.flash_landmark_attention import fused_landmark_attention
    dev = torch.device("cuda:0")
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    is_mem = torch.arange(k.shape[2], device=dev) % block == block - 1
    out = fused_landmark_attention(qd, kd, vd, is_mem, sm_scale=scale, block_size=block)
    gq, gk, gv = torch.autograd.grad(out, [qd, kd, vd], do.to(dev))
    torch.cuda.synchronize()
    return gq, gk, gv


CASES = [
    (1, 2, 32, 32, 128, 32, torch.bfloat16),
    (1, 2, 64, 64, 128, 32, torch.bfloat16),
    (2, 3, 256, 256, 128, 32, torch.bfloat16),
    (1, 8, 384, 384, 128, 32, torch.bfloat16),
    (1, 2, 128, 256, 128, 32, torch.bfloat16),     # history prefix
    (1, 2, 96, 160, 128, 32, torch.bfloat16),      # ragged workgroup tails
    (1, 2, 64, 96, 128, 32, torch.bfloat16),       # odd history (1 block)
    (1, 2, 160, 256, 128, 32, torch.bfloat16),     # odd history (3 blocks), 5 query blocks
    (1, 2, 544, 544, 128, 32, torch.bfloat16),     # 17 blocks: the LDS rings wrap at every phase
    (1, 2, 544, 544, 64, 32, torch.float16),
    # blocks in front of a workgroup run in a loop of their own, in whole turns of the 4-slot ring: history of
    # 5, 6, 7 and 9 blocks leaves 1, 2, 3 and 1 of them to the general path, over two and three query tiles
    (1, 2, 512, 672, 128, 32, torch.bfloat16),
    (1, 2, 288, 480, 128, 32, torch.bfloat16),
    (1, 1, 640, 864, 128, 32, torch.bfloat16),
    (1, 2, 320, 608, 64, 32, torch.bfloat16),
    (1, 2, 256, 256, 128, 64, torch.bfloat16),
    (1, 2, 128, 320, 128, 64, torch.bfloat16),
    (1, 2, 512, 512, 128, 128, torch.bfloat16),
    (1, 2, 256, 512, 128, 128, torch.bfloat16),
    (1, 2, 576, 576, 128, 64, torch.bfloat16),     # 9 blocks of two tiles: ring wraps inside and between blocks
    (1, 2, 384, 640, 128, 128, torch.bfloat16),    # two history blocks of four tiles
    (2, 3, 192, 320, 128, 64, torch.float16),
    (1, 2, 256, 256, 64, 32, torch.bfloat16),
    (1, 2, 256, 256, 64, 64, torch.bfloat16),
    (1, 2, 256, 256, 64, 128, torch.bfloat16),
    (1, 2, 256, 256, 128, 32, torch.float16),
]


@pytest.mark.parametrize("B,H,Lq,Lk,D,block,dtype", CASES)
def test_gradients_match_oracle(B, H, Lq, Lk, D, block, dtype, bwd_path):
    if block != 32 and bwd_path == "handover":
        pytest.skip("the hand-over exists for block 32 only; other sizes always recompute")
    print(f"case B{B} H{H} Lq{Lq} Lk{Lk} D{D} bs{block} {dtype} {bwd_path}", flush=True)
    seed = Lq + Lk + D + block
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=seed, dtype=dtype)
    do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(seed + 1)).to(dtype)
    rq, rk, rv = oracle_grads(q, k, v, do, block)
    gq, gk, gv = _grads(q, k, v, do, block)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        assert err <= TOL, (name, err)
        assert g.dtype == dtype and g.shape == r.shape


def test_landmark_value_rows_get_zero_gradient_and_last_landmark_key_too():
    B, H, L, D, block = 1, 2, 256, 128, 32
    q, k, v = make_qkv(B, H, L, L, D, seed=3)
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(4)).bfloat16()
    gq, gk, gv = _grads(q, k, v, do, block)
    assert (gv[:, :, block - 1::block] == 0).all()
    assert (gk[:, :, -1] == 0).all()
    assert gk[:, :, block - 1].abs().max() > 0


@pytest.mark.parametrize("block", [64, 32])
def test_reference_script_loss_and_blhd_layout(block):
    # the reference's own check: grads of (out**2).sum() on (B,L,H,D)-backed views
    # (test_flash_landmark_attention.py:91-94,156-157)
    from ltriton.flash_landmark_attention import fused_landmark_attention
    from oracle import s1
    B, H, L, D = 2, 4, 256, 128
    q, k, v = make_qkv(B, H, L, L, D, seed=11, layout="blhd")
    dev = torch.device("cuda:0")
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    is_mem = torch.arange(L, device=dev) % block == block - 1
    out = fused_landmark_attention(qd, kd, vd, is_mem, block_size=block)
    g = torch.autograd.grad((out.float() ** 2).sum(), [qd, kd, vd])
    qc, kc, vc = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    r = torch.autograd.grad((s1.s1_attention(qc, kc, vc, block) ** 2).sum(), [qc, kc, vc])
    for a, b_ in zip(g, r):
        assert (a.float().cpu() - b_).abs().max().item() <= 4e-2
        assert a.transpose(1, 2).is_contiguous()             # gradients come back in their input's layout


def test_broadcast_upstream_gradient_and_activation_checkpointing():
    # out.sum().backward() hands the backward an expanded scalar (all strides 0); the reference's layers call the
    # op under torch.utils.checkpoint (llama_mem.py:847-859), which re-runs the forward inside the backward
    from torch.utils.checkpoint import checkpoint
    from ltriton.flash_landmark_attention import fused_landmark_attention
    from oracle import s1
    B, H, L, D, block = 1, 2, 128, 128, 32
    q, k, v = make_qkv(B, H, L, L, D, seed=21)
    dev = torch.device("cuda:0")
    is_mem = torch.arange(L, device=dev) % block == block - 1
    qc, kc, vc = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    r = torch.autograd.grad(s1.s1_attention(qc, kc, vc, block).sum(), [qc, kc, vc])
    for use_checkpoint in (False, True):
        qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
        fn = lambda a, b_, c: fused_landmark_attention(a, b_, c, is_mem, block_size=block)
        out = checkpoint(fn, qd, kd, vd, use_reentrant=False) if use_checkpoint else fn(qd, kd, vd)
        out.sum().backward()
        for a, b_ in zip((qd.grad, kd.grad, vd.grad), r):
            assert (a.float().cpu() - b_).abs().max().item() <= TOL, use_checkpoint


def test_partial_block_backward_is_rejected():
    from ltriton.flash_landmark_attention import fused_landmark_attention
    q, k, v = make_qkv(1, 2, 100, 100, 128, seed=12)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = fused_landmark_attention(qd, kd, vd, None, block_size=32)
    with pytest.raises(AssertionError):
        out.sum().backward()


def test_backward_deterministic_bitwise(bwd_path):
    B, H, L, D, block = 2, 8, 512, 128, 32
    q, k, v = make_qkv(B, H, L, L, D, seed=13)
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(14)).bfloat16()
    a = _grads(q, k, v, do, block)
    b_ = _grads(q, k, v, do, block)
    for x, y in zip(a, b_):
        assert torch.equal(x, y)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_baseline_config2_full_size(seed, bwd_path):
    if bwd_path == "handover" and seed != 0:
        pytest.skip("the hand-over path runs the full size once")
    # benchmark config 2: B2 H32 L2048 D128 block 32, dO ~ N(0,1); seed 0 is the benchmark's, 1 and 2 for robustness
    B, H, L, D, block = 2, 32, 2048, 128, 32
    q, k, v = make_qkv(B, H, L, L, D, seed=seed)
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(100 + seed)).bfloat16()
    gq, gk, gv = _grads(q, k, v, do, block)
    rq, rk, rv = oracle_grads(q, k, v, do, block, chunk=4)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        print("config2", name, "max abs err", err, flush=True)
        assert err <= TOL, (name, err)


@pytest.mark.parametrize("scale", [0.05, 0.3])
@pytest.mark.parametrize("block,Lq,Lk", [(32, 256, 384), (64, 256, 384), (128, 256, 512)])
def test_gradients_with_a_custom_softmax_scale(scale, block, Lq, Lk):
    # sm_scale enters the backward twice: through the exponent (scale * log2 e) and as the factor of dQ and dK
    B, H, D = 1, 2, 128
    print(f"case scale{scale} bs{block} Lq{Lq} Lk{Lk}", flush=True)
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=int(1000 * scale) + block)
    do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(7)).bfloat16()
    rq, rk, rv = oracle_grads(q, k, v, do, block, scale=scale)
    gq, gk, gv = _grads(q, k, v, do, block, scale=scale)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        assert err <= TOL, (name, err)


@pytest.mark.parametrize("Lq,Lk", [(256, 4352), (4608, 4608)])
def test_gradients_beyond_64_blocks(Lq, Lk, bwd_path):
    # 136 and 144 landmark blocks of 32: long history in front of few queries, and a long square problem
    B, H, D, block = 1, 2, 128, 32
    print(f"case long Lq{Lq} Lk{Lk}", flush=True)
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=Lq + Lk)
    do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(8)).bfloat16()
    rq, rk, rv = oracle_grads(q, k, v, do, block, chunk=1)
    gq, gk, gv = _grads(q, k, v, do, block)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        print("long", name, "max abs err", err, flush=True)
        assert err <= TOL, (name, err)


@pytest.mark.parametrize("block", [32, 64])
def test_large_magnitude_inputs_forward_and_backward(block):
    # inputs four times the benchmark's spread: scores reach +-25, far from the fixed reference maximum the
    # block-32 forward takes from the landmark scores alone.  Tolerance: 2e-2 of the largest reference value
    # (16-bit outputs carry a relative rounding error, so the absolute bound scales with the magnitude).
    from tests.util import oracle_forward
    from ltriton.flash_landmark_attention import fused_landmark_attention
    B, H, Lq, Lk, D = 1, 4, 512, 640, 128
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=40 + block, scale=2.0)
    do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(9)).bfloat16()
    ref, _, _ = oracle_forward(q, k, v, block)
    out = fused_landmark_attention(q.cuda(), k.cuda(), v.cuda(), None, block_size=block)
    err = (out.float().cpu() - ref).abs().max().item()
    assert torch.isfinite(out.float()).all()
    assert err <= TOL * max(1.0, ref.abs().max().item()), ("out", err)
    rq, rk, rv = oracle_grads(q, k, v, do, block)
    gq, gk, gv = _grads(q, k, v, do, block)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        bound = TOL * max(1.0, r.abs().max().item())
        print("large magnitude", name, "max abs err", err, "bound", bound, flush=True)
        assert torch.isfinite(g.float()).all()
        assert err <= bound, (name, err, bound)


def test_reference_script_case():
    # the reference's own parity script: B2 H8 L1024 D128, mem_freq 63 -> block 64, bf16, torch.rand inputs on
    # (B,L,H,D)-backed views (test_flash_landmark_attention.py:84-102); forward asserted at rtol=atol=1e-2 (:147),
    # gradients of (out**2).sum() compared at rtol=atol=4e-2 (:156-165; printed there, asserted here)
    from ltriton.flash_landmark_attention import fused_landmark_attention
    from oracle import s1
    B, H, L, D, block = 2, 8, 1024, 128, 64
    g = torch.Generator().manual_seed(1234)
    q, k, v = (torch.rand(B, L, H, D, generator=g).bfloat16().transpose(1, 2) for _ in range(3))
    dev = torch.device("cuda:0")
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    is_mem = torch.arange(L, device=dev) % block == block - 1
    out = fused_landmark_attention(qd, kd, vd, is_mem, block_size=block)
    grads = torch.autograd.grad((out ** 2).sum(), [qd, kd, vd])
    qc, kc, vc = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    exact = s1.s1_attention(qc, kc, vc, block)
    exact_grads = torch.autograd.grad((exact ** 2).sum(), [qc, kc, vc])
    assert torch.allclose(out.float().cpu(), exact.detach(), rtol=1e-2, atol=1e-2)
    for name, a, b_ in zip("qkv", grads, exact_grads):
        assert torch.allclose(a.float().cpu(), b_, rtol=4e-2, atol=4e-2), f"d{name}"


# Many heads: the dK/dV kernel then gives one workgroup several 128-key tiles of a head in a row (its requests
# run on into the next tile while the current one finishes), in zig-zag order over the head's tiles.
@pytest.mark.parametrize("B,H,Lq,Lk,D,block,dtype", [
    (8, 32, 512, 512, 64, 32, torch.bfloat16),       # four tiles per workgroup, one workgroup per head
    (8, 32, 384, 640, 64, 32, torch.bfloat16),       # history; five tiles over two workgroups (3 + 2)
    (4, 32, 768, 768, 64, 64, torch.float16),        # three tiles per workgroup, blocks of two tiles
    (8, 32, 512, 512, 128, 128, torch.bfloat16),     # blocks of four tiles
    (6, 32, 416, 416, 128, 32, torch.bfloat16),      # last tile of a head partly empty (13 key tiles of 32)
])
def test_gradients_with_several_key_tiles_per_workgroup(B, H, Lq, Lk, D, block, dtype, bwd_path):
    if block != 32 and bwd_path == "handover":
        pytest.skip("the hand-over exists for block 32 only")
    print(f"case multi-item B{B} H{H} Lq{Lq} Lk{Lk} D{D} bs{block} {dtype}", flush=True)
    seed = B + Lq + Lk + D + block
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=seed, dtype=dtype)
    do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(seed + 1)).to(dtype)
    rq, rk, rv = oracle_grads(q, k, v, do, block, chunk=16)
    gq, gk, gv = _grads(q, k, v, do, block)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        assert err <= TOL, (name, err)


def test_workspace_size_selects_the_backward_path():
    # lmk_attn_bwd picks the hand-over kernels when the workspace reaches lmk_attn_bwd_handover_workspace_bytes and
    # the recomputing kernels one byte below; both sides of the threshold give the oracle's gradients, and the two
    # paths are different code (their dK differs in the last bits)
    import math
    from landmark_hip import _lib
    from landmark_hip.attention import _launch_fwd
    lib, T4 = _lib.lib(), _lib.tensor4
    B, H, Lq, Lk, D, block = 1, 4, 256, 384, 128, 32
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=77)
    do = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(78)).bfloat16()
    rq, rk, rv = oracle_grads(q, k, v, do, block)
    dev = torch.device("cuda:0")
    qd, kd, vd, dod = (t.to(dev) for t in (q, k, v, do))
    scale = 1.0 / math.sqrt(D)
    n_prefix = (Lk - Lq) // block
    o, Ls, M = _launch_fwd(qd, kd, vd, n_prefix, scale, block)
    small = lib.lmk_attn_bwd_workspace_bytes(B, H, Lq, Lk, block)
    big = lib.lmk_attn_bwd_handover_workspace_bytes(B, H, Lq, Lk, block)
    rows, nb, nq = B * H * Lq, Lk // block, Lq // block
    tiles = nq * (n_prefix + 1) + nq * (nq - 1) // 2
    assert big == ((4 * (2 * rows + rows * nb) + 2047) // 2048) * 2048 + B * H * tiles * 2048 and big > small
    assert lib.lmk_attn_bwd_handover_workspace_bytes(B, H, Lq, Lk, 64) == 0
    ws = torch.empty(big, device=dev, dtype=torch.uint8)
    got = {}
    for name, nbytes in (("below", big - 1), ("at", big), ("small", small)):
        dq, dk, dv = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
        ws.fill_(0xFF)                                        # NaN patterns: nothing may be read that was not written
        _lib.check(lib.lmk_attn_bwd(T4(qd), T4(kd), T4(vd), T4(o), T4(dod), Ls.data_ptr(), M.data_ptr(), T4(dq), T4(dk),
                                    T4(dv), ws.data_ptr(), nbytes, B, H, Lq, Lk, D, scale, block, n_prefix, 0,
                                    _lib.current_stream(dev)))
        torch.cuda.synchronize()
        for nm, g, r in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
            assert (g.float().cpu() - r).abs().max().item() <= TOL, (name, nm)
        got[name] = (dq, dk, dv)
    assert all(torch.equal(a, b_) for a, b_ in zip(got["below"], got["small"]))
    assert not torch.equal(got["at"][1], got["small"][1])


def test_gradients_at_8192_tokens():
    # B1 H2 L8192, block 32: 256 landmark blocks, 32 query tiles per head.  The hand-over workspace (1.1 GB for two
    # heads) is above the shim's default limit, so this is the recomputing pair, the path that serves this length
    B, H, L, D, block = 1, 2, 8192, 128, 32
    print("case L8192", flush=True)
    q, k, v = make_qkv(B, H, L, L, D, seed=8192)
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(8193)).bfloat16()
    rq, rk, rv = oracle_grads(q, k, v, do, block, chunk=1)
    gq, gk, gv = _grads(q, k, v, do, block)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        print("L8192", name, "max abs err", err, flush=True)
        assert err <= TOL, (name, err)


@pytest.mark.parametrize("L,block,D", [(8960, 64, 64), (6885, 51, 64)])
def test_gradients_beyond_128_blocks_of_64_slots(L, block, D):
    # 140 blocks of 64 / 135 blocks of 51 in 64 slots: the 64-slot forward's first pass takes its landmark keys in
    # two rounds, and the dQ kernel's straight-line stages run for most of the sequence
    B, H = 1, 1
    print(f"case L{L} block{block}", flush=True)
    q, k, v = make_qkv(B, H, L, L, D, seed=L)
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(L + 1)).bfloat16()
    rq, rk, rv = oracle_grads(q, k, v, do, block, chunk=1)
    gq, gk, gv = _grads(q, k, v, do, block)
    for name, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        err = (g.float().cpu() - r).abs().max().item()
        print(f"L{L} block{block}", name, "max abs err", err, flush=True)
        assert err <= TOL, (name, err)
