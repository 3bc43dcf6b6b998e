"""Alias module: the reference keeps these types in ``hip_attn.v1_2.hip_config``."""
from ..config import HiPAttentionConfig, HiPAttentionPerLayerConfig  # noqa: F401
