"""Static per-layer buffers for mask metadata, so that decode steps replayed from a HIP graph can hand the
mask of one step to the next.

Stands in for ``HiPMetadataCachePool`` (``src/hip_attn/v1_2/hip_memory_pool.py:55-433``): same constructor, same
buffer names, same storage formats (block indices and stage edges as uint32, stage scores as bf16, counters as
int64), same getters and setters.  A graph captures ``set_hip_metadata_cache`` after a refresh step and
``get_hip_metadata_cache`` before a cached step; both are plain copies between fixed addresses.

The reference's debugging switches that enlarge the buffers (``HIP_DEBUG_UNION_HEAD``, ``HIP_DIAG_INFO``,
``HIP_DEBUG_ADD_DELAY_WINDOW``) and its delayed-first-stage research mode (``HIP_DEBUG_DELAYED_STAGE0``) are not built.
"""
from __future__ import annotations

import logging
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .metadata import (
    HiPAttentionCacheAccessStatistics,
    HiPAttentionOutputMetadata,
    HiPAttentionStageInputCache,
)

logger = logging.getLogger(__name__)

_COUNTERS = ("access_count", "unique_access_count", "cache_miss_count")

_TOO_SMALL = ('Try lowering --cuda-graph-max-bs or raising --hip-attention-config {"metadata_cache_max_batch_size"}.')


def cuda_graph_capture_configs(hip_config) -> List[Tuple[Optional[int]]]:
    """One graph per "how many stages are cached": none, or stage 0 .. last (``paged_hip.py:27-32``)."""
    return [(None,)] + [(i,) for i in range(len(hip_config.layers[0].stages))]


@dataclass
class CachedBuffer:
    """One static tensor: rows are ``batch * heads`` (``"BH"``) or the tensor is ``[batch, 1, heads, ...]``
    (``"B,1,H"``); ``dtype`` is what callers see, the tensor itself may be narrower."""
    buffer: torch.Tensor
    batch_format: str
    dtype: torch.dtype

    def _check(self, batch: int):
        if self.buffer.shape[0] < batch:
            raise ValueError(f"Buffer batch size {self.buffer.shape[0]} is smaller than the requested batch size "
                             f"{batch}.\n{_TOO_SMALL}")

    def get(self, batch_size: int, head_size: int) -> torch.Tensor:
        if self.batch_format == "BH":
            self._check(batch_size)
            return self.buffer[: batch_size * head_size].to(self.dtype, copy=True)
        self._check(batch_size)
        return self.buffer[:batch_size, :, :head_size].to(self.dtype, copy=True)

    def set(self, value: torch.Tensor):
        self._check(value.shape[0])
        if self.batch_format == "BH":
            self.buffer[: value.shape[0]].copy_(value.to(self.buffer.dtype))
        else:
            self.buffer[: value.shape[0], :, : value.shape[2]].copy_(value.to(self.buffer.dtype))


class HiPMetadataCachePool:
    def __init__(self, max_total_num_tokens: int, query_head_num: int, layer_num: int, context_length: int,
                 device: str, hip_config):
        self.hip_config = hip_config
        self.layer_num = layer_num
        self.head_num = query_head_num
        self.max_batch_size = hip_config.metadata_cache_max_batch_size
        self.device = device
        self.cache: List[Dict[str, CachedBuffer]] = [{} for _ in range(layer_num)]
        self.layer_configs = {}

        for layer_idx in range(layer_num):
            dense = layer_idx in hip_config.dense_layers
            presets = hip_config.layers
            cfg = presets[0 if dense else 1] if len(presets) == 2 else presets[layer_idx]
            self.layer_configs[layer_idx] = cfg
            last_chunk = cfg.stages[-1].stage_chunk_size
            n_blocks = -(-cfg.second_stage_k // last_chunk)
            # decode only: one query block per sequence
            self.init_buffer(layer_idx, "indices", [1, n_blocks], torch.int64, store_dtype=torch.uint32)
            self.init_buffer(layer_idx, "ks", [1], torch.int64)
            self.init_buffer(layer_idx, "ks_count", [1, 1], torch.int64)
            self.init_buffer(layer_idx, "ks_start_end", [1, 2], torch.int64)
            for prefix in ("mask", "sa"):
                for name in _COUNTERS:
                    self.init_buffer(layer_idx, f"{prefix}_{name}", [1], torch.int64)
            room = context_length - cfg.sliding_window_size - cfg.sink_token_size
            for i_stage, stage in enumerate(cfg.stages):
                if i_stage == 0:
                    continue
                chunks = min(stage.stage_k, room) // stage.stage_chunk_size
                self.init_buffer(layer_idx, f"stage_{i_stage}_indices_left", [chunks], torch.int64, "B,1,H", torch.uint32)
                self.init_buffer(layer_idx, f"stage_{i_stage}_indices_right", [chunks], torch.int64, "B,1,H", torch.uint32)
                self.init_buffer(layer_idx, f"stage_{i_stage}_out_scores", [chunks], torch.float32, "B,1,H", torch.bfloat16)

        self.allocated_gpu_bytes = self.compute_allocated_bytes()
        logger.info("Allocated HiP metadata cache pool size: %.2f MB", self.allocated_gpu_bytes / 1024 / 1024)

    # ------------------------------------------------------------------ buffers
    def reset_decode_phase(self):
        """Kept for callers of the reference's pool; there is no delayed state to drop here."""

    def compute_allocated_bytes(self) -> int:
        return sum(b.buffer.numel() * b.buffer.element_size() for layer in self.cache for b in layer.values())

    def init_buffer(self, layer_idx: int, name: str, shape: Sequence[int], dtype: torch.dtype,
                    batch_format: str = "BH", store_dtype: Optional[torch.dtype] = None):
        if batch_format == "BH":
            full = (self.max_batch_size * self.head_num, *shape)
        elif batch_format == "B,1,H":
            full = (self.max_batch_size, 1, self.head_num, *shape)
        else:
            raise ValueError(f"unknown batch format {batch_format!r}")
        tensor = torch.zeros(full, device=self.device, dtype=store_dtype or dtype)
        self.cache[layer_idx][name] = CachedBuffer(tensor, batch_format, dtype)

    def _entry(self, layer_idx: int, name: str) -> CachedBuffer:
        if layer_idx not in range(len(self.cache)):
            raise KeyError(f"{layer_idx} is not in range({len(self.cache)})")
        if name not in self.cache[layer_idx]:
            raise KeyError(f"{name} is not in {list(self.cache[layer_idx].keys())}")
        return self.cache[layer_idx][name]

    def get_buffer(self, layer_idx: int, name: str, batch_size: int) -> torch.Tensor:
        return self._entry(layer_idx, name).get(batch_size, self.head_num)

    def set_buffer(self, layer_idx: int, name: str, value: torch.Tensor):
        self._entry(layer_idx, name).set(value)

    # ------------------------------------------------------------------ metadata in and out
    def get_hip_metadata_cache(self, layer_id: int, size: int, batch_size: int,
                               cached_stages: Optional[int]) -> Optional[HiPAttentionOutputMetadata]:
        """``cached_stages`` None (or the stage count): the finished mask; 0: nothing; k: stage inputs up to stage k."""
        assert size == batch_size
        n_stages = len(self.layer_configs[layer_id].stages)
        if cached_stages is None or cached_stages == n_stages:
            return HiPAttentionOutputMetadata(
                indices=self.get_buffer(layer_id, "indices", batch_size),
                ks=self.get_buffer(layer_id, "ks", batch_size),
                ks_count=self.get_buffer(layer_id, "ks_count", batch_size),
                ks_start_end=self.get_buffer(layer_id, "ks_start_end", batch_size),
                mask_cache_statistics=None, sa_cache_statistics=None, stage_caches=None)
        if cached_stages == 0:
            return None
        stage_caches = [HiPAttentionStageInputCache(None, None, None)]
        for i_stage in range(1, cached_stages + 1):
            stage_caches.append(HiPAttentionStageInputCache(
                indices_left=self.get_buffer(layer_id, f"stage_{i_stage}_indices_left", batch_size),
                indices_right=self.get_buffer(layer_id, f"stage_{i_stage}_indices_right", batch_size),
                out_scores=self.get_buffer(layer_id, f"stage_{i_stage}_out_scores", batch_size)))
        return HiPAttentionOutputMetadata(indices=None, ks=None, ks_count=None, ks_start_end=None,
                                          mask_cache_statistics=None, sa_cache_statistics=None,
                                          stage_caches=stage_caches)

    def set_hip_metadata_cache(self, layer_id: int, size: int, batch_size: int, metadata: HiPAttentionOutputMetadata):
        assert size == batch_size
        for name in ("indices", "ks", "ks_count", "ks_start_end"):
            self.set_buffer(layer_id, name, getattr(metadata, name))
        self._set_counters(layer_id, "sa", metadata.sa_cache_statistics)
        self._set_counters(layer_id, "mask", metadata.mask_cache_statistics)
        for i_stage, cache in enumerate(metadata.stage_caches or ()):
            if i_stage == 0:
                continue
            self.set_buffer(layer_id, f"stage_{i_stage}_indices_left", cache.indices_left)
            self.set_buffer(layer_id, f"stage_{i_stage}_indices_right", cache.indices_right)
            self.set_buffer(layer_id, f"stage_{i_stage}_out_scores", cache.out_scores)

    def _set_counters(self, layer_id: int, prefix: str, stats: Optional[HiPAttentionCacheAccessStatistics]):
        if stats is None:
            values = {name: torch.zeros((1,), dtype=torch.int64, device=self.device) for name in _COUNTERS}
        else:
            values = stats.compute_statistics()
        if values["access_count"] is None:
            return  # statistics are computed only when HIP_DISABLE_COMPUTE_STATISTICS=0
        for name in _COUNTERS:
            self.set_buffer(layer_id, f"{prefix}_{name}",
                            values[name].to(torch.int64).view(1, 1).expand(self.max_batch_size, 1))

    def compute_cache_statistics(self, batch_size: int):
        result = {}
        for prefix in ("sa", "mask"):
            access = sum(self.get_buffer(i, f"{prefix}_access_count", batch_size).sum() for i in range(self.layer_num))
            miss = sum(self.get_buffer(i, f"{prefix}_cache_miss_count", batch_size).sum() for i in range(self.layer_num))
            result.update({f"{prefix}_access": access, f"{prefix}_miss": miss,
                           f"{prefix}_hit_ratio": 1 - (miss / access)})
        return result
