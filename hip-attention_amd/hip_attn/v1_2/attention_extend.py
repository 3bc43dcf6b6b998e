"""Alias module: the reference keeps the operator in ``hip_attn.v1_2.attention_extend``."""
from ..operator import dual_stage_quadratic_hip_attention  # noqa: F401
