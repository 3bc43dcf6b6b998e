"""All layers' offloaded KV behind one object, with the next layer's prefix fetched while the current layer runs.

Stands in for ``HiPModelOffloadCache`` (``src/hip_attn/v1_2/model_offload_cache.py:19-466``): same constructor and the
same hooks a model runner calls (``on_model_start / on_layer_start / on_layer_end / on_model_end``,
``get_kv_buffer``, ``set_kv_buffer``, ``get_fetched_prefix_kv_buffer``).

The reference overlaps host work with Python threads: a thread per prefetch gathers pool rows on the CPU and uploads
them with blocking copies, another thread per asynchronous ``set_kv_buffer`` downloads the new rows, and the hooks
poll and sleep.  Here the device reads and writes the pinned pools itself, so both directions are kernels on one side
stream ordered with events; no thread, no host wait, and ``on_layer_end`` has nothing to synchronise.

fp8 (e5m2) pools hold bytes, as the reference's do (``model_offload_cache.py:39-41``); the prefetched prefix comes back
as ``float8_e5m2`` tensors.  ``HIP_OFFLOAD_CACHE_VALIDATION=1`` keeps a resident copy of every layer's rows
(``:117-128``): stores go to both, the prefetched prefix is compared with the copy, and ``get_kv_buffer`` /
``get_fetched_prefix_kv_buffer`` hand the copy out as the third value for ``forward_paged_hip(offloading_metadata=...)``.
Not built: in-kernel cache updates (``DEBUG_ONLINE``).
"""
from __future__ import annotations

import logging
import os
from typing import Any, Dict, Optional, Tuple

import torch
from torch import Tensor

from .offload import HiPOffloadCache

logger = logging.getLogger(__name__)


def format_size_bytes(n: int) -> str:
    for unit in ("B", "KB", "MB", "GB"):
        if n < 1024:
            return f"{n:.2f} {unit}"
        n /= 1024
    return f"{n:.2f} TB"


class HiPModelOffloadCache:
    def __init__(self, max_token_size: int, max_mask_cache_token_size: int, max_sa_cache_token_size: int,
                 dtype: torch.dtype, head_num: int, head_dim: int, layer_num: int, device: torch.device, hip_config):
        assert isinstance(device, torch.device) and device.index is not None
        if dtype not in (torch.bfloat16, torch.float32, torch.float8_e5m2):
            raise NotImplementedError(f"offload pools of dtype {dtype} are not built (bf16, f32 and float8_e5m2 are)")
        self.size = max_token_size
        self.dtype = dtype
        self.store_dtype = torch.uint8 if dtype == torch.float8_e5m2 else dtype
        self.device = device
        self.head_num, self.head_dim, self.layer_num = head_num, head_dim, layer_num
        self.max_mask_cache_token_size = max_mask_cache_token_size * head_num
        self.max_sa_cache_token_size = max_sa_cache_token_size * head_num
        self.online_update_cache = False
        self.layer_buffer = []
        for layer_id in range(layer_num):
            scale = 2 if layer_id in hip_config.dense_layers else 1  # dense layers attend to twice as many blocks
            self.layer_buffer.append(HiPOffloadCache(
                layer_id=layer_id, max_token_size=max_token_size + 1,
                max_mask_cache_token_size=min(max_token_size * head_num, self.max_mask_cache_token_size * scale),
                max_sa_cache_token_size=min(max_token_size * head_num, self.max_sa_cache_token_size * scale),
                head_num=head_num, head_dim=head_dim, dtype=dtype, device=device, online_cache_update=False))
            host, dev = self._calc_allocated_bytes()
            logger.info("[%d/%d] host: %s and GPU: %s are allocated. (%s on %s)", layer_id + 1, layer_num,
                        format_size_bytes(host), format_size_bytes(dev), dtype, device)
        self.copy_stream = torch.cuda.Stream(device=device)
        # (layer, batch item) -> (k, v, prefix length, table, event recorded after the gather)
        self.prefetched_kv: Dict[Tuple[int, int], Tuple[Tensor, Tensor, int, Tensor, torch.cuda.Event]] = {}
        # the reference's switch, spelled as it spells it (model_offload_cache.py:108)
        self.enable_async = os.getenv("HIP_DISABLE_AYSNC", "0") == "0"
        self.require_validation = os.getenv("HIP_OFFLOAD_CACHE_VALIDATION", "0") == "1"
        self.validation_cache = None
        if self.require_validation:  # resident copies [tokens + 1, heads, dim] per layer, K and V
            shape = (max_token_size + 1, head_num, head_dim)
            self.validation_cache = [(torch.zeros(shape, dtype=self.store_dtype, device=device),
                                      torch.zeros(shape, dtype=self.store_dtype, device=device))
                                     for _ in range(layer_num)]

    def is_online_cache_update_enabled(self) -> bool:
        return self.online_update_cache

    def get_kv_buffer(self, layer_id: int) -> Tuple[HiPOffloadCache, Any]:
        if self.require_validation:
            return self.layer_buffer[layer_id], self.validation_cache[layer_id]
        return self.layer_buffer[layer_id], None

    # ------------------------------------------------------------------ writes
    def set_kv_buffer(self, layer_id: int, table: Tensor, cache_k: Tensor, cache_v: Tensor, async_copy: bool = False,
                      push_to_gpu_cache: bool = False):
        """Store new rows of a layer.  ``async_copy`` moves the store to the side stream; readers of this layer are
        ordered after it (``HiPOffloadCache.kv_struct`` waits on the recorded event)."""
        layer = self.layer_buffer[layer_id]
        if cache_k.dtype != self.dtype:
            cache_k, cache_v = cache_k.to(self.dtype), cache_v.to(self.dtype)
        if self.require_validation:
            rows = table.reshape(-1).to(self.device, dtype=torch.int64)
            k_valid, v_valid = self.validation_cache[layer_id]
            k_valid[rows] = cache_k.to(self.device).reshape(-1, self.head_num, self.head_dim).view(self.store_dtype)
            v_valid[rows] = cache_v.to(self.device).reshape(-1, self.head_num, self.head_dim).view(self.store_dtype)
        if not (async_copy and self.enable_async and cache_k.is_cuda):
            layer.set_kv_buffer(table=table, table_gpu=table, cache_k=cache_k, cache_v=cache_v)
            return
        assert not torch.cuda.is_current_stream_capturing(), "asynchronous stores cannot be captured"
        current = torch.cuda.current_stream(self.device)
        self.copy_stream.wait_stream(current)
        with torch.cuda.stream(self.copy_stream):
            layer.set_kv_buffer(table=table, table_gpu=table, cache_k=cache_k, cache_v=cache_v)
            done = torch.cuda.Event()
            done.record(self.copy_stream)
        for t in (table, cache_k, cache_v):
            t.record_stream(self.copy_stream)
        layer.pending_write = done

    # ------------------------------------------------------------------ prefix prefetch around a prefill pass
    def on_model_start(self, is_prefill, batch_size: int, req_to_token: Tensor, req_pool_indices: Tensor,
                       extend_prefix_lens_cpu, extend_seq_lens_cpu):
        if is_prefill:
            self._prefetch_layer(0, batch_size, req_to_token, req_pool_indices, extend_prefix_lens_cpu,
                                 extend_seq_lens_cpu)

    def on_layer_start(self, layer_id: int, is_prefill: bool, batch_size: int, req_to_token: Tensor,
                       req_pool_indices: Tensor, extend_prefix_lens_cpu, extend_seq_lens_cpu):
        if is_prefill and layer_id < self.layer_num - 1:
            self._prefetch_layer(layer_id + 1, batch_size, req_to_token, req_pool_indices, extend_prefix_lens_cpu,
                                 extend_seq_lens_cpu)

    def on_layer_end(self, layer_id: int, is_prefill: bool):
        """Nothing to do: prefetches and stores are ordered by stream events, not by host waits."""

    def on_model_end(self, is_prefill: bool):
        if is_prefill:
            self._synchronize()

    def _prefetch_layer(self, layer_id: int, batch_size: int, req_to_token: Tensor, req_pool_indices: Tensor,
                        extend_prefix_lens_cpu, extend_seq_lens_cpu):
        for ibatch in range(batch_size):
            prefix, fresh = int(extend_prefix_lens_cpu[ibatch]), int(extend_seq_lens_cpu[ibatch])
            table = req_to_token.index_select(dim=0, index=req_pool_indices[ibatch:ibatch + 1])[0, : prefix + fresh]
            self._prefetch_prefix_kv_buffer(layer_id, ibatch, table, prefix)

    def _prefetch_prefix_kv_buffer(self, layer_id: int, batch_id: int, table: Tensor, prefix_seq_len: int):
        assert table.ndim == 1
        handle = (layer_id, batch_id)
        assert handle not in self.prefetched_kv, handle
        layer = self.layer_buffer[layer_id]
        fresh = table.numel() - prefix_seq_len
        stream = self.copy_stream if self.enable_async else torch.cuda.current_stream(self.device)
        stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(stream):
            if layer.pending_write is not None:
                stream.wait_event(layer.pending_write)
            k, v = layer.gather_rows(table[:prefix_seq_len], extra_rows=fresh)
            if self.store_dtype != self.dtype:
                k, v = k.view(self.dtype), v.view(self.dtype)
            done = torch.cuda.Event()
            done.record(stream)
        self.prefetched_kv[handle] = (k.unsqueeze(0), v.unsqueeze(0), prefix_seq_len, table, done)

    def get_fetched_prefix_kv_buffer(self, layer_id: int, batch_id: int, cache_k: Tensor, cache_v: Tensor):
        """``(k, v, None)``: dense ``[1, prefix + new, heads, dim]`` tensors holding the prefetched prefix of this
        layer followed by the rows of the chunk being prefilled (``cache_k / cache_v [1, new, heads, dim]``)."""
        handle = (layer_id, batch_id)
        assert handle in self.prefetched_kv, "the prefix of this layer was never prefetched"
        k, v, prefix_seq_len, table, done = self.prefetched_kv.pop(handle)
        assert cache_k.ndim == 4 and cache_k.shape[0] == 1 and cache_k.shape[2:] == (self.head_num, self.head_dim)
        assert k.shape[1] == prefix_seq_len + cache_k.shape[1], (k.shape, prefix_seq_len, cache_k.shape)
        current = torch.cuda.current_stream(self.device)
        current.wait_event(done)
        k.record_stream(current)
        v.record_stream(current)
        k[:, prefix_seq_len:] = cache_k.to(self.dtype)
        v[:, prefix_seq_len:] = cache_v.to(self.dtype)
        if self.require_validation:  # the gathered prefix must be what the resident copy holds (:211-226)
            k_valid, v_valid = self.validation_cache[layer_id]
            rows = table[:prefix_seq_len].to(self.device, dtype=torch.int64)
            for got, want, name in ((k, k_valid, "K"), (v, v_valid, "V")):
                err = float(((got[0, :prefix_seq_len].float() - want[rows].view(self.dtype).float()) ** 2).sum())
                assert err < 1e-5, f"prefetched {name} prefix of layer {layer_id} differs from the validation pool: {err}"
            return k, v, (k_valid, v_valid)
        return k, v, None

    def _synchronize(self):
        torch.cuda.synchronize(device=self.device)
        assert len(self.prefetched_kv) == 0, "prefetched prefixes were left unused"

    def _calc_allocated_bytes(self) -> Tuple[int, int]:
        host = dev = 0
        for cache in self.layer_buffer:
            for pool in (cache.k_uvm, cache.v_uvm):
                host += pool.allocated_cpu_bytes
                dev += pool.allocated_gpu_bytes
            dev += cache.mask_k_cache.allocated_gpu_bytes + cache.sa_kv_cache.allocated_gpu_bytes
        return host, dev
