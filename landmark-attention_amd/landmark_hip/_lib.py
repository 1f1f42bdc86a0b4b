"""ctypes binding of liblandmark_hip.so (C ABI declared in include/lmk.h).

The library is the only compute path: if it is missing or a call fails the
caller gets an exception, never a fallback.
"""
from __future__ import annotations

import contextlib
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblandmark_hip.so")

DTYPE_CODES = {torch.bfloat16: 0, torch.float16: 1}


class LmkError(RuntimeError):
    def __init__(self, code: int, text: str):
        super().__init__(f"liblandmark_hip: {text} (code {code})")
        self.code = code


class Tensor4(ctypes.Structure):
    """``lmk_tensor4`` of include/lmk.h."""

    _fields_ = [("ptr", ctypes.c_void_p), ("stride_b", ctypes.c_int64), ("stride_h", ctypes.c_int64),
                ("stride_row", ctypes.c_int64)]


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: build it with `python landmark-attention_amd/build.py` "
                "(hipcc --offload-arch=gfx950); there is no fallback path")
        L = ctypes.CDLL(LIB_PATH)
        L.lmk_strerror.restype = ctypes.c_char_p
        L.lmk_strerror.argtypes = [ctypes.c_int]
        L.lmk_version.restype = ctypes.c_char_p
        T4 = ctypes.POINTER(Tensor4)
        i, f, vp = ctypes.c_int, ctypes.c_float, ctypes.c_void_p
        L.lmk_attn_fwd.restype = i
        L.lmk_attn_fwd.argtypes = [T4, T4, T4, T4, vp, vp, i, i, i, i, i, f, i, i, i, vp]
        L.lmk_attn_bwd_workspace_bytes.restype = ctypes.c_size_t
        L.lmk_attn_bwd_workspace_bytes.argtypes = [i, i, i, i, i]
        L.lmk_attn_bwd_handover_workspace_bytes.restype = ctypes.c_size_t
        L.lmk_attn_bwd_handover_workspace_bytes.argtypes = [i, i, i, i, i]
        L.lmk_attn_bwd.restype = i
        L.lmk_attn_bwd.argtypes = [T4, T4, T4, T4, T4, vp, vp, T4, T4, T4, vp, ctypes.c_size_t,
                                   i, i, i, i, i, f, i, i, i, vp]
        L.lmk_attn_bwd_phases.restype = i
        L.lmk_attn_bwd_phases.argtypes = [T4, T4, T4, T4, T4, vp, vp, T4, T4, T4, vp, ctypes.c_size_t,
                                          i, i, i, i, i, f, i, i, i, i, vp]
        i64, sz = ctypes.c_int64, ctypes.c_size_t
        L.lmk_padded_rows.restype = i64
        L.lmk_padded_rows.argtypes = [i64, i, i]
        L.lmk_pad_blocks.restype = i
        L.lmk_pad_blocks.argtypes = [T4, T4, i, i, i64, i, i, i, vp]
        L.lmk_unpad_blocks.restype = i
        L.lmk_unpad_blocks.argtypes = L.lmk_pad_blocks.argtypes
        L.lmk_attn_fwd_padded.restype = i
        L.lmk_attn_fwd_padded.argtypes = [T4, T4, T4, T4, vp, vp, i, i, i, i, i, f, i, i, i, i, vp]
        L.lmk_attn_bwd_padded.restype = i
        L.lmk_attn_bwd_padded.argtypes = [T4, T4, T4, T4, T4, vp, vp, T4, T4, T4, vp, ctypes.c_size_t,
                                          i, i, i, i, i, f, i, i, i, i, vp]
        L.lmk_attn_fwd_blocks.restype = i
        L.lmk_attn_fwd_blocks.argtypes = [T4, T4, T4, T4, vp, vp, i, i, i, i, i, f, i, i, i, vp]
        L.lmk_attn_bwd_blocks_workspace_bytes.restype = sz
        L.lmk_attn_bwd_blocks_workspace_bytes.argtypes = [i, i, i, i, i]
        L.lmk_attn_bwd_blocks.restype = i
        L.lmk_attn_bwd_blocks.argtypes = [T4, T4, T4, T4, T4, vp, vp, T4, T4, T4, vp, sz, i, i, i, i, i, f, i, i, i, vp]
        L.lmk_attn_fwd_group_scale.restype = i
        L.lmk_attn_fwd_group_scale.argtypes = [T4, T4, T4, T4, vp, vp, vp, i, i, i, i, i, f, i, i, i, vp]
        L.lmk_attn_bwd_group_scale_workspace_bytes.restype = sz
        L.lmk_attn_bwd_group_scale_workspace_bytes.argtypes = [i, i, i, i, i]
        L.lmk_attn_bwd_group_scale.restype = i
        L.lmk_attn_bwd_group_scale.argtypes = [T4, T4, T4, T4, T4, vp, vp, vp, T4, T4, T4, vp, sz, i, i, i, i, i, f, i, i, i, vp]
        L.lmk_retrieve_workspace_bytes.restype = sz
        L.lmk_retrieve_workspace_bytes.argtypes = [i, i, i, i, i, i]
        L.lmk_retrieve_topk.restype = i
        L.lmk_retrieve_topk.argtypes = [T4, T4, vp, vp, i64, i64, vp, vp, sz, i, i, i, i, i, i, i, i, vp]
        L.lmk_retrieve_topk_reuse.restype = i
        L.lmk_retrieve_topk_reuse.argtypes = L.lmk_retrieve_topk.argtypes
        L.lmk_retrieve_static_max_bytes.restype = sz
        L.lmk_retrieve_static_max_bytes.argtypes = []
        L.lmk_retrieve_static_init.restype = i
        L.lmk_retrieve_static_init.argtypes = []
        L.lmk_retrieve_topk_static.restype = i
        L.lmk_retrieve_topk_static.argtypes = [T4, T4, vp, vp, i64, i64, vp, i, i, i, i, i, i, i, i, vp]
        L.lmk_gather_attend.restype = i
        L.lmk_gather_attend.argtypes = [T4, T4, T4, vp, vp, vp, i64, i64, T4, vp, vp, i64, T4,
                                        i, i, i, i, i, f, i, i, i, vp]
        L.lmk_attend_workspace_bytes.restype = sz
        L.lmk_attend_workspace_bytes.argtypes = [i, i, i, i, i, i]
        L.lmk_attend.restype = i
        L.lmk_attend.argtypes = [T4, T4, T4, vp, T4, T4, vp, vp, i64, i64, T4, vp, sz,
                                 i, i, i, i, i, f, i, i, i, vp]
        L.lmk_retrieve_and_attend.restype = i
        L.lmk_retrieve_and_attend.argtypes = [T4, T4, T4, T4, T4, vp, vp, i64, i64, vp, T4, vp, sz, i, vp, sz,
                                              i, i, i, i, i, f, i, i, i, vp]
        L.lmk_local_window.restype = i
        L.lmk_local_window.argtypes = [T4, T4, T4, T4, T4, vp, vp, i64, i64, T4, T4, T4, i, i, i, i, i, i, i, vp]
        L.lmk_attn_fwd_segments.restype = i
        L.lmk_attn_fwd_segments.argtypes = [T4, T4, T4, T4, vp, vp, vp, vp, i, i, i, i, i, i, i, i, f, i, i, vp]
        L.lmk_attn_bwd_segments_workspace_bytes.restype = sz
        L.lmk_attn_bwd_segments_workspace_bytes.argtypes = [i, i, i, i, i]
        L.lmk_attn_bwd_segments.restype = i
        L.lmk_attn_bwd_segments.argtypes = [T4, T4, T4, T4, T4, vp, vp, T4, T4, T4, vp, sz, vp, vp, i, i, i, i, i, i, i, f,
                                            i, i, vp]
        L.lmk_ring_local_window.restype = i
        L.lmk_ring_local_window.argtypes = [T4, T4, T4, T4, T4, vp, vp, i64, i64, T4, T4, T4, i, i, i, i, i64, i, i, vp]
        L.lmk_retrieve_topk_shared.restype = i
        L.lmk_retrieve_topk_shared.argtypes = [T4, T4, vp, vp, i64, i64, vp, vp, vp, sz, i, i, i, i, i, i, i, i, vp]
        L.lmk_retrieve_topk_shared_landmarks.restype = i
        L.lmk_retrieve_topk_shared_landmarks.argtypes = L.lmk_retrieve_topk_shared.argtypes
        L.lmk_ring_retrieve_topk.restype = i
        L.lmk_ring_retrieve_topk.argtypes = [T4, T4, vp, vp, i64, i64, vp, vp, sz, i, i, i, i, i, i, i, i, i, i, vp]
        L.lmk_ring_gather_attend.restype = i
        L.lmk_ring_gather_attend.argtypes = [T4, T4, T4, vp, vp, vp, i64, i64, T4, vp, vp, i64, T4,
                                             i, i, i, i, i, f, i, i, i, i, i, vp]
        L.lmk_gather_window.restype = i
        L.lmk_gather_window.argtypes = [T4, T4, T4, vp, T4, T4, vp, vp, i64, i64, T4, T4, T4,
                                        i, i, i, i, i, i, i, i, vp]
        L.lmk_apply_rotary.restype = i
        L.lmk_apply_rotary.argtypes = [T4, T4, vp, vp, i64, i64, vp, i64, i, i, i, i, i, vp]
        L.lmk_attn_fwd_rotary_q.restype = i
        L.lmk_attn_fwd_rotary_q.argtypes = [T4, T4, T4, T4, vp, vp, vp, vp, i64, i64, vp, i64, i, i, i, i, i, f, i, i, i, vp]
        L.lmk_apply_rotary_qk.restype = i
        L.lmk_apply_rotary_qk.argtypes = [T4, T4, T4, T4, vp, vp, i64, i64, vp, i64, i, i, i, i, i, vp]
        _lib = L
    return _lib


def check(code: int) -> None:
    if code != 0:
        raise LmkError(code, lib().lmk_strerror(code).decode())


def tensor4(t: torch.Tensor) -> Tensor4:
    """Describe a (B, H, L, D) tensor with unit stride along D."""
    s = t.stride()
    assert len(s) == 4 and s[3] == 1
    return Tensor4(t.data_ptr(), s[0], s[1], s[2])


def kernel_ready(t: torch.Tensor) -> torch.Tensor:
    """Return ``t`` itself when the kernels can read it in place (unit stride along D, rows walked
    forwards, 16-byte aligned base and strides), otherwise a contiguous copy."""
    s = t.stride()
    if s[3] == 1 and s[2] > 0 and s[0] % 8 == 0 and s[1] % 8 == 0 and s[2] % 8 == 0 and t.data_ptr() % 16 == 0:
        return t
    return t.contiguous()


_SAME_DEVICE = contextlib.nullcontext()


def on_device(device):
    """Context that makes ``device`` current for the launches inside; free when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device(device)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # the handle without a Stream object around it


def current_stream(device) -> int:
    """hipStream_t of torch's current stream on ``device`` (a decode step asks several times per token)."""
    if _raw_stream is not None:
        index = device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream
