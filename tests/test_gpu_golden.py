"""HIP kernels against the committed fixtures (tests/golden/*.npz), through the C ABI."""
import pytest
import torch

from tests.test_golden import load

pytestmark = pytest.mark.gpu

TOL = 2e-2


def test_attention_fixture_forward_and_backward():
    from landmark_hip.attention import _launch_fwd
    from ltriton.flash_landmark_attention import fused_landmark_attention
    f = load("attention_h1_lq64_lk96_d64_b32.npz")
    block = int(f["block"])
    dev = torch.device("cuda:0")
    q, k, v = (f[n][None].bfloat16().to(dev).requires_grad_(True) for n in ("q", "k", "v"))
    is_mem = torch.arange(k.shape[2], device=dev) % block == block - 1
    out = fused_landmark_attention(q, k, v, is_mem, block_size=block)
    assert (out.float().cpu()[0] - f["out"]).abs().max().item() <= TOL
    dq, dk, dv = torch.autograd.grad(out, [q, k, v], f["do"][None].bfloat16().to(dev))
    for got, name in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert (got.float().cpu()[0] - f[name]).abs().max().item() <= TOL, name
    _, L, M = _launch_fwd(q.detach(), k.detach(), v.detach(), (k.shape[2] - q.shape[2]) // block,
                          1.0 / q.shape[-1] ** 0.5, block)
    torch.cuda.synchronize()
    assert (M.cpu() - f["M"]).abs().max() < 1e-3 and ((L.cpu() - f["L"]).abs() / f["L"]).max() < 1e-3


def test_retrieval_fixture_indices_and_output():
    from landmark_hip.retrieval import retrieve_and_attend
    from oracle import rotary
    f = load("retrieval_h1_t3_s197_d128_b32_k2.npz")
    block, top_k = int(f["block"]), int(f["top_k"])
    dev = torch.device("cuda:0")
    q, kc, vc, kl, vl = (f[n].bfloat16().to(dev) for n in ("q", "k_cache", "v_cache", "k_loc", "v_loc"))
    cos, sin = rotary.rotary_tables(kc.shape[2] + q.shape[2], q.shape[3], torch.bfloat16)
    out, idx = retrieve_and_attend(q, (kc, vc), kl, vl, cos.to(dev), sin.to(dev), block, top_k)
    torch.cuda.synchronize()
    assert torch.equal(idx.cpu(), f["idx"])
    assert (out.float().cpu() - f["out"]).abs().max().item() <= TOL


def test_shared_selection_fixture_probabilities_indices_and_output():
    from landmark_hip.retrieval import attend_shared, retrieve_topk
    from oracle import rotary
    f = load("shared_selection_h1_t4_s2115_d64_b32_k3.npz")
    block, top_k = int(f["block"]), int(f["top_k"])
    dev = torch.device("cuda:0")
    q, kc, vc, kl, vl = (f[n + "_bf16bits"].view(torch.bfloat16).to(dev)
                         for n in ("q", "k_cache", "v_cache", "k_loc", "v_loc"))
    cos, sin = (t.to(dev) for t in rotary.rotary_tables(kc.shape[2] + q.shape[2], q.shape[3], torch.bfloat16))
    idx, probs = retrieve_topk(q, kc, cos, sin, block, top_k, aggregate="max_over_tokens", return_block_probs=True)
    torch.cuda.synchronize()
    assert torch.equal(probs.float().cpu()[:, :, 0], f["block_probs"])
    assert torch.equal(idx.cpu(), f["idx"])
    out = attend_shared(q, kc, vc, idx, kl, vl, cos, sin, block, top_k)
    assert (out.float().cpu() - f["out"]).abs().max().item() <= TOL
