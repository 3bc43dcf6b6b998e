"""Serving-side configuration: per-layer HiP presets parsed from a JSON string or file.

Same keys, defaults and unknown-key rejection as the reference
(``src/hip_attn/v1_2/hip_config.py:32-180``).
"""
from __future__ import annotations

import json
from dataclasses import InitVar, dataclass, field
from typing import List, Optional, Union

from .metadata import ScanStage


def _default_stages() -> List[ScanStage]:
    return [
        ScanStage(stage_block_size_q=64, stage_block_stride_q=4, stage_chunk_size=256, stage_k=None, stage_stride=1),
        ScanStage(stage_block_size_q=64, stage_block_stride_q=4, stage_chunk_size=32, stage_k=32768, stage_stride=1),
        ScanStage(stage_block_size_q=64, stage_block_stride_q=1, stage_chunk_size=8, stage_k=8192, stage_stride=1),
    ]


def _take(parsed: dict, obj, names, convert=None):
    """Move the listed keys from ``parsed`` onto ``obj`` (optionally through a converter)."""
    for name in names:
        if name in parsed:
            val = parsed.pop(name)
            setattr(obj, name, convert[name](val) if convert and name in convert else val)


@dataclass
class HiPAttentionPerLayerConfig:
    second_stage_k: int = 2048
    sliding_window_size: int = 1024
    sink_token_size: int = 256
    sa_extend_backend: str = "streaming"
    scan_extend_backend: Optional[str] = None
    stages: List[ScanStage] = field(default_factory=_default_stages)

    parsed_json: InitVar[Optional[dict]] = None

    def __post_init__(self, parsed_json: Optional[dict]):
        if parsed_json is None:
            return
        parsed_json = dict(parsed_json)
        _take(parsed_json, self,
              ("second_stage_k", "sliding_window_size", "sink_token_size", "sa_extend_backend",
               "scan_extend_backend", "stages"),
              convert={"stages": lambda lst: [ScanStage(**st) for st in lst]})
        if parsed_json:
            raise ValueError(f"Unknown keys in json: {parsed_json.keys()}")


def _default_layers() -> List[HiPAttentionPerLayerConfig]:
    # first preset serves the layers listed in dense_layers, second all others (hip_config.py:68-81)
    return [
        HiPAttentionPerLayerConfig(second_stage_k=4096, sa_extend_backend="streaming", scan_extend_backend="streaming"),
        HiPAttentionPerLayerConfig(second_stage_k=2048, sa_extend_backend="streaming", scan_extend_backend="relative"),
    ]


@dataclass
class HiPAttentionConfig:
    dense_layers: List[int] = field(default_factory=lambda: [0, 1, 2, 3, 31])
    block_sparse_block_size_q: int = 64
    metadata_cache_max_batch_size: int = 32
    mask_refresh_interval: Union[int, List[int]] = field(default_factory=lambda: [32, 16, 8])
    using_extend: bool = True
    layers: List[HiPAttentionPerLayerConfig] = field(default_factory=_default_layers)
    prefill_layers: List[HiPAttentionPerLayerConfig] = field(default_factory=_default_layers)

    # deprecated switches, still accepted
    apply_v_dot: bool = False
    prefill_always_dense: bool = False
    decode_always_dense: bool = False
    force_dense: bool = False
    prefill_dense_threshold: int = 8192

    json_or_path: InitVar[Optional[str]] = None

    def __post_init__(self, json_or_path: Optional[str]):
        if json_or_path is None:
            parsed = {}
        elif json_or_path.lstrip().startswith("{"):
            parsed = json.loads(json_or_path)
        else:
            with open(json_or_path, "r") as f:
                parsed = json.load(f)
        parsed = dict(parsed)
        if "mask_refresh_interval" in parsed:
            assert isinstance(parsed["mask_refresh_interval"], (int, list))
        layer_list = lambda lst: [HiPAttentionPerLayerConfig(parsed_json=layer) for layer in lst]
        _take(parsed, self,
              ("apply_v_dot", "dense_layers", "prefill_always_dense", "decode_always_dense", "force_dense",
               "prefill_dense_threshold", "block_sparse_block_size_q", "metadata_cache_max_batch_size",
               "mask_refresh_interval", "using_extend", "layers"),
              convert={"layers": layer_list})
        if self.prefill_layers is None:
            self.prefill_layers = self.layers
        _take(parsed, self, ("prefill_layers",), convert={"prefill_layers": layer_list})
        if parsed:
            raise ValueError(f"Unknown keys in json: {parsed.keys()}")

        num_stages = len(self.layers[0].stages)
        for layer in self.layers:
            assert num_stages == len(layer.stages)
        if isinstance(self.mask_refresh_interval, int):
            self.mask_refresh_interval = [self.mask_refresh_interval] * num_stages
