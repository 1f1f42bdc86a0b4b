"""MI355X-native landmark attention: Python host side over liblandmark_hip.so."""
from .attention import FusedLandmarkAttention, fused_landmark_attention  # noqa: F401
