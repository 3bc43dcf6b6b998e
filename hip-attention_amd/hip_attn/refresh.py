"""Decode-time mask refresh schedule (``src/hip_attn/v1_2/mask_refresh_interval.py:4-30``)."""
from __future__ import annotations

from typing import Optional

from .config import HiPAttentionConfig


class HiPMaskRefreshState:
    """Tells the serving loop which stage of the hierarchy to recompute on each decode step.

    ``update()`` returns ``-1`` on the first step (recompute everything), otherwise the first stage
    ``i`` whose interval divides the step index (recompute stages ``i..last`` from cached inputs), or
    ``None`` (reuse the cached mask).
    """

    def __init__(self, hip_config: HiPAttentionConfig):
        self.hip_config = hip_config
        self.decode_index = 0

    def update(self) -> Optional[int]:
        stage: Optional[int] = None
        intervals = self.hip_config.mask_refresh_interval
        if intervals is not None:
            for i_stage, every in enumerate(intervals):
                if self.decode_index % every == 0:
                    stage = i_stage
                    break
        if self.decode_index == 0:
            stage = -1
        self.decode_index += 1
        return stage
