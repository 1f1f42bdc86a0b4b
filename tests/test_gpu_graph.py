"""The entry points only launch kernels on the stream they are given, so a step can be recorded into a
HIP graph: every replay must reproduce the eager result bit for bit, with eager work in between."""
import pytest
import torch

from oracle import rotary as orot

pytestmark = pytest.mark.gpu


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fn()                                                 # first calls: attributes set, allocator warmed
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        res = fn()
    return g, res


@pytest.mark.parametrize("aggregate", [None, "max_over_tokens"])
def test_decode_step_replays_from_a_graph(aggregate):
    from landmark_hip.retrieval import retrieve_and_attend
    B, H, D, block, top_k, T = 1, 4, 128, 32, 4, 1
    S = 40 * block + 9                                           # cache with an incomplete block
    gen = torch.Generator().manual_seed(5)
    mk = lambda *s: (torch.randn(*s, generator=gen) * 0.5).bfloat16().cuda()
    q, kc, vc, kl, vl = mk(B, H, T, D), mk(B, H, S, D), mk(B, H, S, D), mk(B, H, T, D), mk(B, H, T, D)
    cos, sin = (t.cuda() for t in orot.rotary_tables(S + T, D, torch.bfloat16))
    step = lambda: retrieve_and_attend(q, (kc, vc), kl, vl, cos, sin, block, top_k, aggregate=aggregate)
    out_e, idx_e = step()
    torch.cuda.synchronize()
    out_e, idx_e = out_e.clone(), idx_e.clone()
    g, (out_g, idx_g) = _capture(step)
    for rep in range(4):
        out_g.zero_()
        idx_g.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e) and torch.equal(idx_g, idx_e), rep
        step()                                                   # eager work between the replays
    # new inputs in the captured buffers: the replay follows them
    q2 = mk(B, H, T, D)
    out2, idx2 = retrieve_and_attend(q2, (kc, vc), kl, vl, cos, sin, block, top_k, aggregate=aggregate)
    torch.cuda.synchronize()
    out2, idx2 = out2.clone(), idx2.clone()
    q.copy_(q2)
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(out_g, out2) and torch.equal(idx_g, idx2)


@pytest.mark.parametrize("path", ["recompute", "handover"])
def test_forward_backward_replays_from_a_graph(path, monkeypatch):
    from landmark_hip import attention
    from landmark_hip.attention import _launch_bwd, _launch_fwd
    monkeypatch.setattr(attention, "HANDOVER_MAX_BYTES", 0 if path == "recompute" else 1 << 40)
    monkeypatch.setattr(attention, "HANDOVER_MIN_KEYS", 0)
    B, H, L, D, block = 1, 4, 256, 128, 32
    gen = torch.Generator().manual_seed(6)
    mk = lambda: (torch.randn(B, H, L, D, generator=gen) * 0.5).bfloat16().cuda()
    q, k, v, do = mk(), mk(), mk(), mk()
    sc = D ** -0.5

    def step():
        o, Ls, M = _launch_fwd(q, k, v, 0, sc, block)
        return (o,) + tuple(_launch_bwd(q, k, v, o, do, Ls, M, 0, sc, block))

    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    g, res = _capture(step)
    for rep in range(3):
        for t in res:
            t.zero_()
        g.replay()
        torch.cuda.synchronize()
        for a, b in zip(res, eager):
            assert torch.equal(a, b), rep
        step()
