"""Alias module: the reference keeps this class in ``hip_attn.v1_2.mask_refresh_interval``."""
from ..refresh import HiPMaskRefreshState  # noqa: F401
