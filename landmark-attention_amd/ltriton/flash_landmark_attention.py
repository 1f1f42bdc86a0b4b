"""Drop-in for ``llama/ltriton/flash_landmark_attention.py``: same module path and the two
names its callers import (``llama/llama_mem.py:34``,
``llama/ltriton/test_flash_landmark_attention.py:4``), served by the HIP kernels."""
from landmark_hip.attention import FusedLandmarkAttention, fused_landmark_attention  # noqa: F401

__all__ = ["FusedLandmarkAttention", "fused_landmark_attention"]
