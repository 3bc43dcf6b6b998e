"""Import paths of the reference's ``hip_attn.v1_2`` package (``src/hip_attn/v1_2/__init__.py:1-9``)."""
from ..operator import dual_stage_quadratic_hip_attention as hip_attention
from ..config import HiPAttentionConfig  # noqa: F401,E402
from ..refresh import HiPMaskRefreshState  # noqa: F401,E402
from ..paged import forward_paged_hip  # noqa: F401,E402
from ..memory_pool import HiPMetadataCachePool, cuda_graph_capture_configs  # noqa: F401,E402
