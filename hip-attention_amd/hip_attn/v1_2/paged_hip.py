"""Alias module: the reference keeps this entry point in ``hip_attn.v1_2.paged_hip``."""
from ..paged import forward_paged_hip  # noqa: F401
