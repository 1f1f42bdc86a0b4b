"""CPU-side checks of the C ABI: the shared library loads without a GPU, exports every
symbol include/lmk.h declares, and rejects bad arguments on the host before any launch."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lmk.h")


@pytest.fixture(scope="module")
def lib():
    from landmark_hip import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import importlib.util
        spec = importlib.util.spec_from_file_location("lmk_build", os.path.join(ROOT, "landmark-attention_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build()
    return _lib.lib()


def _declared():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(lmk_[a-z_0-9]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = _declared()
    assert {"lmk_attn_fwd", "lmk_attn_bwd", "lmk_retrieve_topk", "lmk_gather_attend", "lmk_local_window", "lmk_ring_local_window",
            "lmk_retrieve_topk_shared", "lmk_retrieve_topk_reuse", "lmk_gather_window", "lmk_apply_rotary", "lmk_attend", "lmk_retrieve_and_attend", "lmk_retrieve_topk_static", "lmk_retrieve_static_max_bytes",
            "lmk_ring_retrieve_topk", "lmk_ring_gather_attend", "lmk_attn_bwd_handover_workspace_bytes", "lmk_retrieve_topk_shared_landmarks", "lmk_attn_fwd_rotary_q", "lmk_apply_rotary_qk", "lmk_padded_rows", "lmk_pad_blocks", "lmk_unpad_blocks", "lmk_attn_fwd_padded", "lmk_attn_bwd_padded", "lmk_attn_fwd_blocks", "lmk_attn_bwd_blocks", "lmk_attn_fwd_segments", "lmk_attn_bwd_segments", "lmk_attn_fwd_group_scale", "lmk_attn_bwd_group_scale",
            "lmk_strerror"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n


def test_version_and_strerror(lib):
    assert b"gfx950" in lib.lmk_version()
    assert lib.lmk_strerror(0) == b"ok"
    for code in range(-11, 0):
        assert lib.lmk_strerror(code) not in (b"", b"unknown error")


def _t4(ptr=0x1000, sb=0, sh=0, sr=128):
    from landmark_hip._lib import Tensor4
    return Tensor4(ptr, sb, sh, sr)


def _fwd(lib, q=None, k=None, v=None, o=None, L=0x2000, M=0x3000, B=1, H=1, Lq=64, Lk=64, D=128, scale=0.1,
         block=32, n_prefix=0, dtype=0):
    t = _t4()
    return lib.lmk_attn_fwd(q or t, k or t, v or t, o or t, L, M, B, H, Lq, Lk, D, scale, block, n_prefix, dtype, None)


def test_forward_argument_errors(lib):
    # every call here fails validation, so nothing is launched and no GPU is needed
    assert _fwd(lib, q=_t4(ptr=0)) == -1                      # NULL
    assert _fwd(lib, L=0) == -1
    assert _fwd(lib, q=_t4(ptr=0x1008)) == -4                 # misaligned pointer
    assert _fwd(lib, q=_t4(sr=-128)) == -2                    # rows are walked forwards
    assert _fwd(lib, k=_t4(sr=1 << 26), Lq=64, Lk=64) == -3   # 64 rows x 2^26 elements x 2 bytes = 8 GiB per slice
    assert _fwd(lib, k=_t4(sr=130)) == -4                     # misaligned row stride
    assert _fwd(lib, B=0) == -2
    assert _fwd(lib, D=96) == -3
    assert _fwd(lib, block=48) == -3
    assert _fwd(lib, dtype=7) == -3
    assert _fwd(lib, Lq=64, Lk=96, n_prefix=0) == -5          # history not declared
    assert _fwd(lib, Lq=64, Lk=80, n_prefix=1) == -5          # history not whole blocks
    assert _fwd(lib, Lq=96, Lk=64) == -5
    assert _fwd(lib, scale=0.0) == -7
    assert _fwd(lib, scale=float("nan")) == -7


def test_backward_argument_errors(lib):
    t = _t4()
    args = lambda **kw: dict(dict(ws=0x4000, wsb=1 << 30, B=1, H=1, Lq=64, Lk=64, D=128, scale=0.1, block=32,
                                  n_prefix=0, dtype=0), **kw)

    def call(**kw):
        a = args(**kw)
        return lib.lmk_attn_bwd(t, t, t, t, t, 0x2000, 0x3000, t, t, t, a["ws"], a["wsb"], a["B"], a["H"], a["Lq"],
                                a["Lk"], a["D"], a["scale"], a["block"], a["n_prefix"], a["dtype"], None)

    assert call(ws=0) == -1
    assert call(Lq=48, Lk=48) == -6                           # partial blocks
    assert call(wsb=16) == -8                                 # workspace too small
    assert call(block=16) == -3
    need = lib.lmk_attn_bwd_workspace_bytes(2, 32, 2048, 2048, 32)
    assert need == 4 * (2 * 2 * 32 * 2048 + 3 * 2 * 32 * 2048 * 64)
    assert lib.lmk_attn_bwd_workspace_bytes(0, 1, 1, 1, 1) == 0
    # hand-over workspace: row terms + one plane, rounded up to 2 KB, + one 2 KB tile per visible (query tile, block)
    ho = lib.lmk_attn_bwd_handover_workspace_bytes(2, 32, 2048, 2048, 32)
    assert ho == 4 * (2 * 2 * 32 * 2048 + 2 * 32 * 2048 * 64) + 64 * (64 * 65 // 2) * 2048
    assert lib.lmk_attn_bwd_handover_workspace_bytes(1, 2, 64, 128, 32) == 4096 + 2 * (2 * 3 + 1) * 2048
    assert lib.lmk_attn_bwd_handover_workspace_bytes(2, 32, 2048, 2048, 64) == 0     # block 32 only
    assert lib.lmk_attn_bwd_handover_workspace_bytes(1, 1, 48, 48, 32) == 0          # whole blocks only


def test_retrieval_argument_errors(lib):
    t = _t4()

    def topk(S=64, block=32, top_k=4, n_pos=4096, ws=0x4000, wsb=1 << 30, cos=0x5000, D=128):
        return lib.lmk_retrieve_topk(t, t, cos, 0x6000, 128, n_pos, 0x7000, ws, wsb, 1, 1, 8, S, D, block, top_k, 0, None)

    assert topk(cos=0) == -1
    assert lib.lmk_retrieve_topk_reuse(t, t, 0x5000, 0x6000, 128, 4096, 0x7000, 0x4000, 64, 1, 1, 8, 64, 128, 32, 4, 0,
                                       None) == -8      # the workspace is still checked for this call's size
    assert topk(S=16) == -9                                   # less than one complete block
    assert topk(top_k=0) == -10 and topk(top_k=65) == -10
    assert topk(n_pos=32) == -11
    assert topk(wsb=64) == -8
    assert topk(D=96) == -3
    assert lib.lmk_retrieve_workspace_bytes(1, 32, 256, 32768, 128, 32) >= 32 * 1024 * 128 * 2 + 2 * 32 * 256 * 1024 * 4
    # the entry point whose workspace is a fixed array inside the library: same checks, all of them on the host
    # before the array is looked up, and a size limit instead of a workspace argument
    def static(S=64, T=8, H=1, top_k=4, cos=0x5000, idx=0x7000):
        return lib.lmk_retrieve_topk_static(t, t, cos, 0x6000, 128, 1 << 20, idx, 1, H, T, S, 128, 32, top_k, 0, None)

    assert lib.lmk_retrieve_static_max_bytes() == 16 << 20
    assert static(cos=0) == -1 and static(idx=0) == -1 and static(S=16) == -9 and static(top_k=0) == -10
    assert static(S=32768, T=256, H=32) == -8                 # benchmark config 4 needs 75 MB of workspace
    assert lib.lmk_retrieve_workspace_bytes(1, 32, 1, 32768 + 7, 128, 32) < 16 << 20      # a decode step fits
    # gather+attend is built for head dims 64 and 128 and blocks of 32/64/128
    ga = lambda D, block: lib.lmk_gather_attend(t, t, t, 0x7000, 0x5000, 0x6000, 128, 4096, t, 0x2000, 0x3000, 8, t, 1, 1,
                                                8, 64, D, 0.1, block, 4, 0, None)
    assert ga(96, 32) == -3 and ga(128, 16) == -3 and ga(64, 16) == -3

    # window of an incomplete cached block: needs a tail, and tail + new chunk within one block (llama_mem.py:330)
    def window(S, T):
        return lib.lmk_local_window(t, t, t, t, t, 0x5000, 0x6000, 128, 4096, t, t, t, 1, 1, T, S, 128, 32, 0, None)

    assert window(64, 4) == -9
    assert window(70, 27) == -2
    assert window(20, 4) == -9

    # the ring cache's window: the tail lives outside the ring and is rotated at positions the caller names
    def ring_window(tail=5, pos=100, D=128, kt=None):
        return lib.lmk_ring_local_window(t, kt or t, t, t, t, 0x5000, 0x6000, 128, 4096, t, t, t, 1, 1, 8, tail, pos, D,
                                         0, None)

    assert ring_window(tail=0) == -2 and ring_window(pos=-1) == -11 and ring_window(pos=4092) == -11
    assert ring_window(D=96) == -3 and ring_window(kt=_t4(ptr=0)) == -1

    # the attend step as one call: workspace and tail are checked before anything is launched
    def attend(S=64, T=8, ws=0x4000, wsb=1 << 30):
        return lib.lmk_attend(t, t, t, 0x7000, t, t, 0x5000, 0x6000, 128, 4096, t, ws, wsb, 1, 1, T, S, 128, 0.1, 32, 4,
                              0, None)

    assert attend(ws=None) == -1
    assert attend(wsb=64) == -8
    assert attend(S=70, T=27) == -2
    a256 = lambda x: (x + 255) & ~255
    assert lib.lmk_attend_workspace_bytes(1, 32, 256, 32768, 128, 32) == a256(32 * 256 * 128 * 2) + 2 * a256(32 * 256 * 4)
    assert lib.lmk_attend_workspace_bytes(1, 32, 1, 32768 + 7, 128, 32) == 4 * a256(32 * 8 * 128 * 2) + 2 * a256(32 * 8 * 4)

    # selection + attend in one call: the attend workspace and the tail are checked before the selection is enqueued
    def both(S=64, T=8, aws=0x4000, awsb=1 << 30, wsb=1 << 30):
        return lib.lmk_retrieve_and_attend(t, t, t, t, t, 0x5000, 0x6000, 128, 4096, 0x7000, t, 0x8000, wsb, 0, aws, awsb,
                                           1, 1, T, S, 128, 0.1, 32, 4, 0, None)

    assert both(aws=None) == -1
    assert both(awsb=64) == -8
    assert both(wsb=64) == -8
    assert both(S=70, T=27) == -2
    assert both(S=20, T=4) == -9

    # what a later stage of the fused entry points would reject is rejected before the first launch
    def both_x(D=128, block=32, out=t, idx=0x7000, scale=0.1):
        return lib.lmk_retrieve_and_attend(t, t, t, t, t, 0x5000, 0x6000, 128, 4096, idx, out, 0x8000, 1 << 30, 0, 0x4000,
                                           1 << 30, 1, 1, 8, 64, D, scale, block, 4, 0, None)

    def attend_x(D=128, block=32, out=t, idx=0x7000, scale=0.1):
        return lib.lmk_attend(t, t, t, idx, t, t, 0x5000, 0x6000, 128, 4096, out, 0x4000, 1 << 30, 1, 1, 8, 64, D, scale,
                              block, 4, 0, None)

    for f in (both_x, attend_x):
        assert f(D=96) == -3                                    # head dims 64 and 128
        assert f(block=16) == -3                                # the fused forward for blocks of 32, 64, 128
        assert f(out=None) == -1
        assert f(idx=0) == -1
        assert f(scale=0.0) == -7

    # one selection per head: same argument contract as the per-token entry point
    def shared(S=64, top_k=4, n_pos=4096, wsb=1 << 30, idx=0x7000):
        return lib.lmk_retrieve_topk_shared(t, t, 0x5000, 0x6000, 128, n_pos, idx, None, 0x4000, wsb, 1, 1, 8, S, 128, 32, top_k,
                                            0, None)

    assert shared(idx=0) == -1 and shared(S=16) == -9 and shared(top_k=0) == -10 and shared(n_pos=32) == -11
    assert shared(wsb=64) == -8

    # selected blocks + local window: padded queries are required only when there is a tail
    def gwin(S, T, idx=0x7000, q_win=t):
        return lib.lmk_gather_window(t, t, t, idx, t, t, 0x5000, 0x6000, 128, 4096, q_win, t, t, 1, 1, T, S, 128, 32, 4, 0,
                                     None)

    assert gwin(64, 4, idx=0) == -1
    assert gwin(70, 27) == -2                                  # llama_mem.py:330
    assert gwin(70, 4, q_win=None) == -1
    assert gwin(20, 4) == -9

    # rotary of a whole tensor
    def rot(pos=0x7000, D=128, n_pos=64, stride=8, L=8, dtype=0):
        return lib.lmk_apply_rotary(t, t, 0x5000, 0x6000, 128, n_pos, pos, stride, 1, 1, L, D, dtype, None)

    assert rot(pos=0) == -1 and rot(D=96) == -3 and rot(n_pos=0) == -11 and rot(stride=-1) == -2 and rot(L=0) == -2
    assert rot(dtype=5) == -3


def test_python_shim_rejects_what_the_reference_rejects():
    import torch
    from ltriton.flash_landmark_attention import FusedLandmarkAttention, fused_landmark_attention
    q = torch.zeros(1, 1, 32, 128, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):                       # CPU tensors (flash_landmark_attention.py:324)
        fused_landmark_attention(q, q, q, None, block_size=32)
    with pytest.raises(AssertionError):                       # history not whole blocks (:397)
        fused_landmark_attention(q, torch.zeros(1, 1, 40, 128, dtype=torch.bfloat16), q, None, block_size=32)
    assert issubclass(FusedLandmarkAttention, torch.autograd.Function)


def test_blocks_of_any_size_host_side(lib):
    # a narrower block is stored in the next of 64 / 128 slots; whole blocks widen, a partial tail keeps its length
    import torch
    from landmark_hip import _lib, attention
    L = _lib.lib()
    assert L.lmk_padded_rows(510, 51, 64) == 640 and L.lmk_padded_rows(120, 51, 64) == 2 * 64 + 18
    assert L.lmk_padded_rows(64, 64, 64) == 64 and L.lmk_padded_rows(0, 51, 64) == 0
    assert L.lmk_padded_rows(10, 1, 64) == -1 and L.lmk_padded_rows(10, 65, 64) == -1 and L.lmk_padded_rows(-1, 51, 64) == -1
    assert [attention.storage_block(b) for b in (2, 17, 32, 33, 51, 64, 65, 100, 128)] == [64, 64, 32, 64, 64, 64, 128, 128, 128]
    for bad in (1, 0, 129, 256):
        with pytest.raises(ValueError):
            attention.storage_block(bad)
    t = _lib.Tensor4(0x1000, 0, 0, 128)

    def pad(fn=L.lmk_pad_blocks, src=t, rows=102, D=128, real=51, block=64):
        return fn(src, t, 1, 1, rows, D, real, block, None)
    assert pad(src=None) == -1 and pad(rows=0) == -2 and pad(real=1) == -2 and pad(real=65) == -2 and pad(D=96) == -3
    assert pad(fn=L.lmk_unpad_blocks, rows=0) == -2 and pad(rows=1 << 31) == -3

    def fwd(block, real, L_=128):
        return L.lmk_attn_fwd_padded(t, t, t, t, 0x2000, 0x3000, 1, 1, L_, L_, 128, 0.1, block, real, 0, 0, None)
    assert fwd(32, 17) == -3 and fwd(64, 1) == -2 and fwd(64, 65) == -2 and fwd(16, 16) == -3

    def bwd(block, real, ws=1 << 30):
        return L.lmk_attn_bwd_padded(t, t, t, t, t, 0x2000, 0x3000, t, t, t, 0x4000, ws, 1, 1, 128, 128, 128, 0.1, block,
                                     real, 0, 0, None)
    assert bwd(32, 17) == -3 and bwd(128, 1) == -2 and bwd(64, 51, ws=16) == -8


def test_token_layout_entry_points_argument_errors(lib):
    # lmk_attn_fwd_blocks / lmk_attn_bwd_blocks: blocks of 2..128 tokens on tensors that are not repacked
    from landmark_hip import _lib
    L = _lib.lib()
    t = _lib.Tensor4(0x1000, 0, 0, 128)

    def fwd(Lq=102, Lk=102, block=51, n_prefix=0, D=128):
        return L.lmk_attn_fwd_blocks(t, t, t, t, 0x2000, 0x3000, 1, 1, Lq, Lk, D, 0.1, block, n_prefix, 0, None)

    def bwd(Lq=102, Lk=102, block=51, n_prefix=0, ws=1 << 30):
        return L.lmk_attn_bwd_blocks(t, t, t, t, t, 0x2000, 0x3000, t, t, t, 0x4000, ws, 1, 1, Lq, Lk, 128, 0.1, block,
                                     n_prefix, 0, None)
    assert fwd(block=1) == -3 and fwd(block=129) == -3 and fwd(D=96) == -3
    assert fwd(Lk=153, n_prefix=0) == -5 and fwd(Lq=102, Lk=51) == -2        # history must be whole blocks; Lk >= Lq
    assert bwd(Lq=100, Lk=100) == -6                                          # the backward needs whole blocks
    assert bwd(Lk=153, n_prefix=2) == -5 and bwd(ws=16) == -8
    # the workspace is indexed by slots: 51 tokens in 64 slots
    assert L.lmk_attn_bwd_blocks_workspace_bytes(2, 8, 510, 510, 51) == L.lmk_attn_bwd_workspace_bytes(2, 8, 640, 640, 64)
    assert L.lmk_attn_bwd_blocks_workspace_bytes(2, 8, 512, 512, 64) == L.lmk_attn_bwd_workspace_bytes(2, 8, 512, 512, 64)
    assert L.lmk_attn_bwd_blocks_workspace_bytes(1, 1, 10, 10, 200) == 0


def test_group_scale_and_rotary_q_argument_errors(lib):
    from landmark_hip import _lib
    L = _lib.lib()
    t = _lib.Tensor4(0x1000, 0, 0, 128)

    def fwd(gs=0x9000, Lq=102, Lk=102, block=51, n_prefix=0):
        return L.lmk_attn_fwd_group_scale(t, t, t, t, 0x2000, 0x3000, gs, 1, 1, Lq, Lk, 128, 0.1, block, n_prefix, 0, None)

    def bwd(gs=0x9000, Lq=102, Lk=102, block=51, ws=1 << 30):
        return L.lmk_attn_bwd_group_scale(t, t, t, t, t, 0x2000, 0x3000, gs, t, t, t, 0x4000, ws, 1, 1, Lq, Lk, 128, 0.1,
                                          block, 0, 0, None)
    assert fwd(gs=None) == -1 and fwd(block=129) == -3 and fwd(Lk=150) == -5
    assert bwd(gs=None) == -1 and bwd(Lq=100, Lk=100) == -6 and bwd(ws=8) == -8
    # block 32 runs in 64 slots when group factors are given: the workspace is sized for that
    assert L.lmk_attn_bwd_group_scale_workspace_bytes(1, 2, 64, 64, 32) == L.lmk_attn_bwd_workspace_bytes(1, 2, 128, 128, 64)
    # the forward that rotates q in its prologue exists for the native block sizes only
    rc = L.lmk_attn_fwd_rotary_q(t, t, t, t, 0x2000, 0x3000, 0x5000, 0x6000, 128, 4096, 0x7000, 0, 1, 1, 102, 102, 128, 0.1,
                                 51, 0, 0, None)
    assert rc == -3


def test_ring_selection_argument_errors(lib):
    from landmark_hip import _lib
    L = _lib.lib()
    t = _lib.Tensor4(0x1000, 0, 0, 64)

    def sel(q=t, idx=0x7000, ws=0x8000, nbytes=1 << 30, T=1, n=4, D=64, block=51, k=2, start=0, method=0, n_pos=1 << 20):
        return L.lmk_ring_retrieve_topk(q, t, 0x5000, 0x6000, 64, n_pos, idx, ws, nbytes, 1, 2, T, n, D, block, k, start,
                                        method, 0, None)
    assert sel(q=None) == -1 and sel(idx=None) == -1 and sel(ws=None) == -1
    assert sel(n=0) == -9 and sel(T=0) == -2 and sel(D=96) == -3 and sel(block=1) == -3 and sel(method=3) == -3
    assert sel(k=5) == -10 and sel(k=0) == -10                    # more blocks asked for than cached: torch.topk raises
    assert sel(start=4) == -2 and sel(start=-1) == -2
    assert sel(n_pos=3 * 51 - 1) == -11 and sel(nbytes=16) == -8


def test_ring_attention_argument_errors(lib):
    from landmark_hip import _lib
    L = _lib.lib()
    t = _lib.Tensor4(0x1000, 0, 0, 64)

    def att(q=t, idx=0x7000, Ls=0x8000, T=1, n=4, D=64, block=51, k=2, start=0, method=0, n_pos=1 << 20, stride=1, scale=0.1):
        return L.lmk_ring_gather_attend(q, t, t, idx, 0x5000, 0x6000, 64, n_pos, t, Ls, 0x9000, stride, t, 1, 2, T, n, D,
                                        scale, block, k, start, method, 0, None)
    assert att(q=None) == -1 and att(idx=None) == -1 and att(Ls=None) == -1
    assert att(n=0) == -9 and att(T=0) == -2 and att(D=96) == -3 and att(method=3) == -3
    assert att(block=1) == -3 and att(block=129) == -3           # blocks of 2..128 tokens
    assert att(k=5) == -10 and att(k=0) == -10
    assert att(start=4) == -2 and att(T=3, stride=2) == -2
    assert att(n_pos=3 * 51 - 1) == -11 and att(scale=0.0) == -7


def test_irregular_landmark_positions_are_rejected_with_a_message():
    # landmarks anywhere but at the end of every block are rejected where the caller has not asked for them
    # (the rotary-q forward, the ring cache, group dropout), as in the reference (flash_landmark_attention.py:393-394)
    import torch
    from landmark_hip import attention
    attention._VALIDATED_MASKS.clear()
    mask = torch.arange(102) % 51 == 50
    attention._check_is_mem(mask, 51)
    dropped = mask.clone()
    dropped[50] = False
    with pytest.raises(AssertionError, match="last token of every block"):
        attention._check_is_mem(dropped, 51)
    with pytest.raises(AssertionError, match="last token of every block"):
        attention._check_is_mem(torch.arange(102) % 51 == 49, 51)


def test_is_mem_is_validated_once_per_mask_state():
    # the reference compares the mask with the expected pattern on every call (one device->host sync each,
    # flash_landmark_attention.py:393-394); the shim remembers masks that passed and re-checks a tensor only
    # after an in-place write to it
    import torch
    from landmark_hip import attention
    attention._VALIDATED_MASKS.clear()
    mask = torch.arange(128) % 32 == 31
    attention._check_is_mem(mask, 32)
    attention._check_is_mem(mask, 32)
    assert len(attention._VALIDATED_MASKS) == 1
    with pytest.raises(AssertionError):
        attention._check_is_mem(mask, 64)                      # same tensor, other block size: checked again
    mask[5] = True                                             # bumps the version counter
    with pytest.raises(AssertionError):
        attention._check_is_mem(mask, 32)
    with pytest.raises(AssertionError):
        attention._check_is_mem(torch.zeros(128, dtype=torch.bool), 32)


def test_is_mem_built_under_inference_mode_is_checked_without_a_version_counter():
    # inference tensors track no version counter (reading it raises); such masks are validated on every call
    import torch
    from landmark_hip import attention
    attention._VALIDATED_MASKS.clear()
    with torch.inference_mode():
        mask = torch.arange(128) % 32 == 31
        bad = torch.zeros(128, dtype=torch.bool)
    assert mask.is_inference()
    attention._check_is_mem(mask, 32)
    attention._check_is_mem(mask, 32)
    assert len(attention._VALIDATED_MASKS) == 0
    with pytest.raises(AssertionError):
        attention._check_is_mem(bad, 32)
    with torch.inference_mode():
        attention._check_is_mem(mask, 32)


def test_irregular_landmark_positions_become_a_table_of_blocks():
    import torch
    from landmark_hip import attention
    attention._VALIDATED_MASKS.clear()
    mask = torch.zeros(20, dtype=torch.bool)
    mask[[3, 9, 11, 16]] = True
    seg = attention._check_is_mem(mask, 5, irregular_ok=True)
    assert seg.seg == [0, 4, 10, 12, 17, 20] and seg.n_blocks == 5 and seg.last_is_partial and seg.max_len == 6
    assert list(seg.seg_host) == seg.seg and seg.seg_dev.tolist() == seg.seg
    assert attention._check_is_mem(mask, 5, irregular_ok=True) is seg            # remembered with the mask
    assert seg.history_blocks(10) == 2 and seg.history_blocks(0) == 0
    with pytest.raises(AssertionError, match="whole blocks"):
        seg.history_blocks(5)
    with pytest.raises(AssertionError, match="last token of every block"):
        attention._check_is_mem(mask, 5)                                         # the same mask where it is not wanted
    two_in_a_row = mask.clone()
    two_in_a_row[4] = True
    with pytest.raises(AssertionError, match="two landmarks in a row"):
        attention._check_is_mem(two_in_a_row, 5, irregular_ok=True)
    wide = torch.zeros(300, dtype=torch.bool)
    wide[[200, 299]] = True
    with pytest.raises(AssertionError, match="more than 128"):
        attention._check_is_mem(wide, 5, irregular_ok=True)
    per_sequence = torch.stack((mask, mask.roll(1)))
    with pytest.raises(AssertionError, match="same for every sequence"):
        attention._check_is_mem(per_sequence, 5, irregular_ok=True)
    assert attention._check_is_mem(torch.arange(20) % 5 == 4, 5, irregular_ok=True) is None   # a regular mask stays one


def test_block_table_is_checked_on_the_host(lib):
    import ctypes
    t = _t4()

    def fwd(seg=(0, 4, 10, 12), n_blocks=3, max_len=6, partial=0, Lq=12, Lk=12, n_prefix=0, dev=0x9000, host=True):
        arr = (ctypes.c_int32 * len(seg))(*seg)
        return lib.lmk_attn_fwd_segments(t, t, t, t, 0x2000, 0x3000, arr if host else None, dev, n_blocks, max_len,
                                         partial, 1, 1, Lq, Lk, 128, 0.1, n_prefix, 0, None)

    assert fwd(host=False) == -1 and fwd(dev=0) == -1
    assert fwd(seg=(1, 4, 10, 12)) == -2                       # the first block starts at token 0
    assert fwd(seg=(0, 4, 10, 13)) == -2                       # the last one ends at Lk
    assert fwd(seg=(0, 4, 11, 12)) == -2                       # longer than max_block_tokens
    assert fwd(seg=(0, 4, 5, 12), max_len=8) == -2             # a landmark alone
    assert fwd(seg=(0, 4, 4, 12), max_len=8) == -2             # not increasing
    assert fwd(max_len=129) == -3 and fwd(max_len=1) == -3
    assert fwd(Lq=7, n_prefix=1) == -5                         # the history is not whole blocks
    assert fwd(n_prefix=3) == -2
    assert lib.lmk_attn_bwd_segments_workspace_bytes(1, 1, 3, 0, 6) == lib.lmk_attn_bwd_workspace_bytes(1, 1, 192, 192, 64)
    assert lib.lmk_attn_bwd_segments_workspace_bytes(1, 1, 3, 1, 100) == lib.lmk_attn_bwd_workspace_bytes(1, 1, 256, 384, 128)
    arr = (ctypes.c_int32 * 4)(0, 4, 10, 12)
    bwd = lib.lmk_attn_bwd_segments(t, t, t, t, t, 0x2000, 0x3000, t, t, t, 0x4000, 16, arr, 0x9000, 3, 6, 1, 1, 12, 12, 128,
                                    0.1, 0, 0, None)
    assert bwd == -8                                           # workspace too small: nothing is launched
