"""Import path of the reference's ``hip_attn.v1_2.model_offload_cache`` (``src/hip_attn/v1_2/model_offload_cache.py``)."""
from ..model_offload import HiPModelOffloadCache  # noqa: F401
