"""HiP / InfiniteHiP attention for AMD Instinct MI355X (gfx950).

Import surface of the reference package for the v1.2 operator (``src/hip_attn/__init__.py:30-45``):
``hip_attention_12(q, k, v, args=HiPAttentionArgs12()) -> (context, metadata)`` plus the paged entry
points.  Everything executes in hand-written HIP kernels behind ``libhipattn.so``.
"""
from .metadata import HiPAttentionArgs as HiPAttentionArgs12
from .metadata import HiPAttentionCacheAccessStatistics as HiPAttentionCacheAccessStatistics12
from .metadata import HiPAttentionOutputMetadata as HiPAttentionOutputMetadata12
from .metadata import ScanStage as ScanStage12
from .operator import dual_stage_quadratic_hip_attention as hip_attention_12
from .config import HiPAttentionConfig, HiPAttentionPerLayerConfig
from .refresh import HiPMaskRefreshState
from .paged import forward_paged_hip
from .offload import HiPOffloadCache
from .memory_pool import HiPMetadataCachePool, cuda_graph_capture_configs
from .model_offload import HiPModelOffloadCache



def prescale_keys(k, head_major: bool = True, rows=None):
    """``bf16(k * c_k)`` for a whole bf16 key tensor (dense ``[B, T, HKV, D]`` or a paged cache
    ``[pages, page, HKV, D]``): the copy ``HiPAttentionArgs.k_prescaled`` takes.  ``head_major`` lays the copy out
    with the kv head outermost in memory (same logical shape), which keeps the rows a search samples close together.
    No counterpart in the reference (an extension; see ``HiPAttentionArgs.k_prescaled``)."""
    from . import _native

    return _native.prescale_k(k, k.device, head_major=head_major)


hip_attention = hip_attention_12
HiPAttentionArgs = HiPAttentionArgs12
HiPAttentionOutputMetadata = HiPAttentionOutputMetadata12

__version__ = "1.2.0+mi355x"

__all__ = [
    "hip_attention_12",
    "HiPAttentionArgs12",
    "HiPAttentionOutputMetadata12",
    "HiPAttentionCacheAccessStatistics12",
    "ScanStage12",
    "hip_attention",
    "HiPAttentionArgs",
    "HiPAttentionOutputMetadata",
    "HiPAttentionConfig",
    "HiPAttentionPerLayerConfig",
    "HiPMaskRefreshState",
    "forward_paged_hip",
    "HiPOffloadCache",
    "HiPMetadataCachePool",
    "HiPModelOffloadCache",
    "cuda_graph_capture_configs",
    "prescale_keys",
]
