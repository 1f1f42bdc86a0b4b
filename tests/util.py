"""Shared helpers for the GPU parity tests: seeded inputs built on the CPU (so the
oracle and the kernels see identical bits) and oracle evaluation in head chunks."""
import torch

from oracle import s1


def make_qkv(B, H, Lq, Lk, D, seed=0, dtype=torch.bfloat16, scale=0.5, layout="bhld"):
    """q (B,H,Lq,D), k, v (B,H,Lk,D) ~ N(0,1)*scale, generated in fp32 on the CPU then cast.
    layout "blhd" backs the tensors by (B,L,H,D) storage and returns transposed views, the
    way the reference's callers hand them over (llama_mem.py:287-289)."""
    g = torch.Generator().manual_seed(seed)

    def one(L):
        if layout == "blhd":
            return (torch.randn(B, L, H, D, generator=g) * scale).to(dtype).transpose(1, 2)
        return (torch.randn(B, H, L, D, generator=g) * scale).to(dtype)

    return one(Lq), one(Lk), one(Lk)


def oracle_forward(q, k, v, block, scale=None, chunk=8):
    """fp32 S1 on the CPU from the (already rounded) 16-bit inputs; returns out, L, M."""
    B, H = q.shape[:2]
    qf, kf, vf = (t.float().flatten(0, 1) for t in (q, k, v))
    outs, Ls, Ms = [], [], []
    for i in range(0, B * H, chunk):
        o, L, M = s1.s1_attention(qf[i:i + chunk], kf[i:i + chunk], vf[i:i + chunk], block, scale, return_stats=True)
        outs.append(o), Ls.append(L), Ms.append(M)
    out = torch.cat(outs).unflatten(0, (B, H))
    return out, torch.cat(Ls), torch.cat(Ms)


def oracle_grads(q, k, v, do, block, scale=None, chunk=4):
    """Autograd through fp32 S1 on the CPU; returns dq, dk, dv (fp32)."""
    B, H = q.shape[:2]
    qf, kf, vf, dof = (t.float().flatten(0, 1) for t in (q, k, v, do))
    gq, gk, gv = [], [], []
    for i in range(0, B * H, chunk):
        a, b, c = (t[i:i + chunk].clone().requires_grad_(True) for t in (qf, kf, vf))
        o = s1.s1_attention(a, b, c, block, scale)
        x, y, z = torch.autograd.grad((o * dof[i:i + chunk]).sum(), [a, b, c])
        gq.append(x), gk.append(y), gv.append(z)
    unf = lambda ts: torch.cat(ts).unflatten(0, (B, H))
    return unf(gq), unf(gk), unf(gv)
