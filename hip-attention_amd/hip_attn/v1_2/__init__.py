"""Import paths of the reference's ``hip_attn.v1_2`` package (``src/hip_attn/v1_2/__init__.py:1-9``)."""
from ..operator import dual_stage_quadratic_hip_attention as hip_attention
