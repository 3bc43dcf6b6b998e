"""Alias module: the reference keeps these types in ``hip_attn.v1_2.attention_metadata``."""
from ..metadata import *  # noqa: F401,F403
from ..metadata import HiPAttentionArgs, HiPAttentionOutputMetadata, ScanStage  # noqa: F401
