"""Import path of the reference's ``hip_attn.v1_2.hip_memory_pool`` (``src/hip_attn/v1_2/hip_memory_pool.py``)."""
from ..memory_pool import CachedBuffer, HiPMetadataCachePool  # noqa: F401
