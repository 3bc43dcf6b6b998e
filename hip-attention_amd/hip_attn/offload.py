"""KV offloading: keys and values live in pinned host memory, a block cache in HBM serves the kernels.

Takes the place of ``UVMCache`` / ``GPUCache`` / ``HiPOffloadCache`` of the reference
(``src/hip_attn/v1_2/uvm_gpu_cache.py:72-117,204-566,569-700``) with the same constructor arguments and
methods, re-designed for this hardware:

* the host pool is ordinary pinned memory that the GPU reads in place over the host link (the reference
  uses managed memory advised to stay on the CPU);
* the cache is block granular (``block_tokens`` consecutive pool rows of one kv head per slot) instead
  of token granular, so one table lookup covers a whole 16-token attention block;
* there are two caches as in the reference -- a large key-only one for mask estimation and a key+value
  one for sparse attention -- and replacement is exact LRU by the step of the last read;
* misses do not stall anything: the reading kernel takes the row from the host pool and flags the block;
  ``handle_cache_miss`` brings the flagged blocks in afterwards with device-side kernels (no host round
  trip), optionally on a side stream so that the copy overlaps whatever runs next.
"""
from __future__ import annotations

import os
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _native as N


def _as_stored(rows: Tensor, pool_dtype: torch.dtype) -> Tensor:
    """Rows in a pool's storage format; a byte pool takes float8_e5m2 values (rounded from wider inputs)."""
    if pool_dtype == torch.uint8:
        if rows.dtype not in (torch.uint8, torch.float8_e5m2):
            rows = rows.to(torch.float8_e5m2)
        return rows.contiguous().view(torch.uint8)
    return rows.to(pool_dtype).contiguous()


def concurrent_stream(device, tries: int = 6):
    """A side stream whose work really runs beside the current stream's, and whether the probe saw it do so.

    A process has few hardware queues (four by default) and the runtime spreads its streams over them, so a new stream
    may share the current stream's queue; work on it then waits for everything enqueued there before it, and a fetch
    on such a stream overlaps nothing.  The probe puts about a millisecond of small launches on the current stream
    and a small fill on the candidate: a candidate on a queue of its own finishes first.  Streams tried and rejected
    are kept alive, so that later streams do not take their place on the queues; the process keeps at most
    ``_MAX_REJECTED`` of them and probes those again once that many exist.  Called once per cache, at set-up."""
    device = torch.device(device)
    main = torch.cuda.current_stream(device)
    big = torch.empty(4 << 20, dtype=torch.float32, device=device)   # 16 MB: 128 passes take about a millisecond
    small = torch.empty(1024, dtype=torch.float32, device=device)
    cand = None
    for attempt in range(tries):
        fresh = len(_REJECTED_STREAMS) < _MAX_REJECTED
        if fresh:
            cand = torch.cuda.Stream(device=device)
            _REJECTED_STREAMS.append(cand)
        else:
            cand = _REJECTED_STREAMS[attempt % len(_REJECTED_STREAMS)]
        # the first launch on a stream sets its queue up and takes longer than the whole probe: a stream that has
        # never run anything always looks as if it waited for the main stream
        with torch.cuda.stream(cand):
            small.zero_()
        torch.cuda.synchronize(device)
        done_main, done_side = torch.cuda.Event(), torch.cuda.Event()
        for _ in range(128):
            big.add_(1.0)
        done_main.record(main)
        with torch.cuda.stream(cand):
            small.zero_()
            done_side.record(cand)
        done_side.synchronize()
        beside = not done_main.query()
        torch.cuda.synchronize(device)
        if beside:
            _REJECTED_STREAMS.remove(cand)
            return cand, True
    return cand, False


_MAX_REJECTED = 8
_REJECTED_STREAMS = []


class UVMCache:
    """Host pool ``[max_token_size, head_num, head_dim]`` in pinned memory (``uvm_gpu_cache.py:72-117``)."""

    def __init__(self, layer_id: int, max_token_size: int, head_num: int, head_dim: int, dtype: torch.dtype,
                 device: torch.device):
        if dtype not in (torch.bfloat16, torch.float32, torch.float8_e5m2, torch.uint8):
            raise NotImplementedError(f"offload pool dtype {dtype}: bfloat16, float32 and float8_e5m2 are built")
        if dtype == torch.float8_e5m2:
            dtype = torch.uint8  # fp8 (e5m2) rows are held as bytes, as the reference does (model_offload_cache.py:39-41)
        self.layer_id = layer_id
        self.max_token_size = max_token_size
        self.head_num = head_num
        self.head_dim = head_dim
        self.dtype = dtype
        self.device = torch.device(device)
        self.bank_cpu = torch.zeros((max_token_size, head_num, head_dim), dtype=dtype, pin_memory=True)
        self.device_ptr = N.host_device_pointer(self.bank_cpu)
        # per-token generation, bumped on every overwrite (uvm_gpu_cache.py:109-114,681-688)
        self.metadata = torch.zeros((max_token_size, 1), dtype=torch.int32, device=self.device)
        self.allocated_cpu_bytes = self.bank_cpu.numel() * self.bank_cpu.element_size()
        self.allocated_gpu_bytes = self.metadata.numel() * self.metadata.element_size()

    def gather_cpu(self, table: Tensor, pin_memory: bool = False) -> Tensor:
        out = torch.empty((table.numel(), self.head_num, self.head_dim), dtype=self.dtype, pin_memory=pin_memory)
        torch.index_select(self.bank_cpu, 0, table.reshape(-1).to(torch.int64), out=out)
        return out


class GPUCache:
    """Block cache in device memory over one or two host pools (``uvm_gpu_cache.py:204-566``)."""

    def __init__(self, k_uvm: UVMCache, v_uvm: Optional[UVMCache], max_cache_token_size: int,
                 online_cache_update: bool = False, block_tokens: int = 16, max_fetch: Optional[int] = None):
        if online_cache_update:
            raise NotImplementedError("online_cache_update (cache fill inside the attention kernel) is not built")
        self.k_uvm = k_uvm
        self.v_uvm = v_uvm
        self.kv_packed = v_uvm is not None
        self.device = k_uvm.device
        self.block_tokens = block_tokens
        self.max_cache_token_size = max_cache_token_size
        self.slots = max(1, max_cache_token_size // block_tokens)
        self.max_fetch = int(max_fetch if max_fetch is not None else min(self.slots, 65536))

        d = N.CacheDesc()
        d.dtype = N.storage_code(k_uvm.bank_cpu)
        d.HKV, d.HID = k_uvm.head_num, k_uvm.head_dim
        d.block_tokens = block_tokens
        d.with_v = int(self.kv_packed)
        d.pool_rows = k_uvm.max_token_size
        d.slots = self.slots
        d.host_k = k_uvm.device_ptr
        d.host_v = v_uvm.device_ptr if v_uvm is not None else 0
        d.host_stride_row, d.host_stride_h = k_uvm.bank_cpu.stride(0), k_uvm.bank_cpu.stride(1)
        if v_uvm is not None:
            assert v_uvm.bank_cpu.shape == k_uvm.bank_cpu.shape and v_uvm.bank_cpu.stride() == k_uvm.bank_cpu.stride()
        sz = N.cache_sizes(d, self.max_fetch)
        self.n_blocks = sz.n_blocks
        dev = self.device
        esz = k_uvm.bank_cpu.element_size()
        self.bank = torch.empty(sz.bank_bytes // esz, dtype=k_uvm.dtype, device=dev)
        self.table = torch.empty((k_uvm.head_num, sz.n_blocks), dtype=torch.int32, device=dev)
        self.last_use = torch.empty(self.slots, dtype=torch.int32, device=dev)
        self.backref = torch.empty(self.slots, dtype=torch.int32, device=dev)
        self.miss = torch.empty((k_uvm.head_num, sz.n_blocks), dtype=torch.uint8, device=dev)
        self.workspace = torch.empty(sz.workspace_bytes, dtype=torch.uint8, device=dev)
        d.bank, d.table, d.last_use = self.bank.data_ptr(), self.table.data_ptr(), self.last_use.data_ptr()
        d.backref, d.miss, d.workspace = self.backref.data_ptr(), self.miss.data_ptr(), self.workspace.data_ptr()
        self._desc = d
        self.handle = N.cache_create(d, self.max_fetch, dev)
        self._ready: Optional[torch.cuda.Event] = None
        # schedule + commit are about twenty small launches whose enqueueing costs more host time than the kernels
        # take when there is little to fetch: after a first eager run they are replayed from one HIP graph
        self._miss_graph: Optional[torch.cuda.CUDAGraph] = None
        self._miss_graph_failed = False
        self._miss_calls = 0
        self.allocated_gpu_bytes = sum(t.numel() * t.element_size() for t in (
            self.bank, self.table, self.last_use, self.backref, self.miss, self.workspace))

    def __del__(self):
        h, self.handle = getattr(self, "handle", 0), 0
        try:
            if h:
                N.cache_destroy(h)
        except Exception:  # interpreter shutdown: the module may already be torn down
            pass

    def flush(self):
        self.wait()
        N.cache_flush(self.handle, self.device)

    def wait(self):
        """Order the current stream after the last ``handle_cache_miss`` issued on another stream."""
        if self._ready is not None:
            torch.cuda.current_stream(self.device).wait_event(self._ready)
            self._ready = None

    def handle_cache_miss(self, metadata=None, stats=None, stream: Optional[torch.cuda.Stream] = None,
                          after: Optional[torch.cuda.Event] = None):
        """Bring the blocks flagged during the last step into the cache (``uvm_gpu_cache.py:305-398``).

        ``metadata`` / ``stats`` are accepted for signature compatibility: the readers already recorded
        what missed.  With ``stream`` the work runs there, after everything enqueued so far on the current
        stream, or, with ``after``, after that event only (recorded behind the step whose misses are fetched:
        work enqueued on the current stream since then runs beside the fetch); the next attention call waits for it.
        """
        if stream is None:
            self.wait()
            self._schedule_and_commit()
            return
        if after is not None:
            stream.wait_event(after)
        else:
            stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(stream):
            self._schedule_and_commit()
            self._ready = torch.cuda.Event()
            self._ready.record(stream)

    def prepare_miss_graph(self, run_first: bool = True) -> bool:
        """Record the lookup and the fetch into a HIP graph now (set-up time: a capture collects garbage and
        synchronises the device).  Captured in thread-local mode, so that allocations or synchronisations of other host
        threads do not break it; if the capture fails all the same, later calls launch eagerly.  ``run_first``: launch
        the two calls once eagerly before recording them (an empty step when nothing has been read yet; it loads the
        kernels outside the capture).  Returns whether a graph is in place."""
        if self._miss_graph is not None:
            return True
        if self._miss_graph_failed or os.getenv("HIP_ATTN_CACHE_MISS_GRAPH", "1") != "1":
            return False
        if torch.cuda.is_current_stream_capturing():
            return False
        current = torch.cuda.current_stream(self.device)
        try:
            if run_first and self._miss_calls == 0:
                N.cache_schedule(self.handle, self.device)
                N.cache_commit(self.handle, self.device)
            graph = torch.cuda.CUDAGraph()
            cap = torch.cuda.Stream(device=self.device)
            cap.wait_stream(current)
            with torch.cuda.graph(graph, stream=cap, capture_error_mode="thread_local"):
                N.cache_schedule(self.handle, self.device)
                N.cache_commit(self.handle, self.device)
            current.wait_stream(cap)
            self._miss_graph = graph
        except Exception:  # a failed capture must not take the serving path down with it
            self._miss_graph_failed = True
            torch.cuda.synchronize(self.device)
            return False
        return True

    def _schedule_and_commit(self):
        """Enqueue the lookup and the fetch on the current stream: as one replay of the graph ``prepare_miss_graph``
        recorded (the kernels take the cache's arrays by address and read every count on the device, so one recording
        serves every call), eagerly inside a caller's own graph capture or when there is no graph.  A cache whose
        owner never called ``prepare_miss_graph`` records it on its second call."""
        capturing = torch.cuda.is_current_stream_capturing()
        use_graph = os.getenv("HIP_ATTN_CACHE_MISS_GRAPH", "1") == "1" and not capturing
        self._miss_calls += 1
        if use_graph and self._miss_graph is None and not self._miss_graph_failed and self._miss_calls >= 2:
            self.prepare_miss_graph(run_first=False)
        if use_graph and self._miss_graph is not None:
            self._miss_graph.replay()
        else:
            N.cache_schedule(self.handle, self.device)
            N.cache_commit(self.handle, self.device)

    def on_set_kv_buffer(self, table: Tensor, cache_k: Tensor, cache_v: Optional[Tensor]):
        """Resident blocks receive freshly written rows (``uvm_gpu_cache.py:548-563``)."""
        self.wait()
        rows = table.reshape(-1).to(device=self.device, dtype=torch.int64).contiguous()
        k_rows = _as_stored(cache_k.to(self.device), self.k_uvm.dtype)
        v_rows = _as_stored(cache_v.to(self.device), self.k_uvm.dtype) if (self.kv_packed and cache_v is not None) else None
        N.cache_write_rows(self.handle, rows, k_rows, v_rows, self.device)

    def statistics(self) -> dict:
        s = N.cache_stats(self.handle, self.device)
        keys = ("steps", "blocks_hit", "blocks_missed", "blocks_fetched", "blocks_evicted", "last_hit", "last_missed",
                "last_fetched")
        return dict(zip(keys, s))


class HiPOffloadCache:
    """Host-resident K/V of one layer with its two device caches (``uvm_gpu_cache.py:569-700``)."""

    def __init__(self, layer_id: int, max_token_size: int, max_mask_cache_token_size: int,
                 max_sa_cache_token_size: int, head_num: int, head_dim: int, dtype: torch.dtype,
                 device: torch.device, online_cache_update: bool = False, block_tokens: int = 16,
                 max_fetch: Optional[int] = None):
        self.layer_id = layer_id
        self.device = torch.device(device)
        self.head_kv = head_num
        self.head_dim = head_dim
        self.page_size = 1
        self.k_uvm = UVMCache(layer_id, max_token_size, head_num, head_dim, dtype, device)
        self.v_uvm = UVMCache(layer_id, max_token_size, head_num, head_dim, dtype, device)
        self.mask_k_cache = GPUCache(self.k_uvm, None, max_mask_cache_token_size, online_cache_update,
                                     block_tokens=block_tokens, max_fetch=max_fetch)
        self.sa_kv_cache = GPUCache(self.k_uvm, self.v_uvm, max_sa_cache_token_size, online_cache_update,
                                    block_tokens=block_tokens, max_fetch=max_fetch)
        self.miss_stream: Optional[torch.cuda.Stream] = None
        # event of a store into the pools that was issued on another stream; readers wait for it
        self.pending_write: Optional[torch.cuda.Event] = None

    def get_page_count(self) -> int:
        assert self.k_uvm.bank_cpu.shape == self.v_uvm.bank_cpu.shape
        return self.k_uvm.bank_cpu.shape[0]

    # ------------------------------------------------------------------ what the operator needs
    def kv_struct(self, block_table: Tensor, cache_seq_lens: Tensor, max_tsrc: int, masking: bool):
        """Paged (page size 1) description of the host pools with the cache that serves this phase."""
        cache = self.mask_k_cache if masking else self.sa_kv_cache
        cache.wait()
        self._wait_pending_write()
        kb, vb = self.k_uvm.bank_cpu, self.v_uvm.bank_cpu
        s = N.KVStruct()
        s.k, s.v = self.k_uvm.device_ptr, self.v_uvm.device_ptr
        s.k_stride_b, s.k_stride_t, s.k_stride_h = kb.stride(0), kb.stride(0), kb.stride(1)
        s.v_stride_b, s.v_stride_t, s.v_stride_h = vb.stride(0), vb.stride(0), vb.stride(1)
        s.tsrc = 0
        s.max_tsrc = max_tsrc
        s.block_table = block_table.data_ptr()
        s.cache_seq_lens = cache_seq_lens.data_ptr()
        s.bt_stride_b = block_table.stride(0)
        s.bt_is64 = int(block_table.dtype == torch.int64)
        s.sl_is64 = int(cache_seq_lens.dtype == torch.int64)
        s.paged = 1
        s.page_size = 1
        s.HKV = self.head_kv
        s.cache = cache.handle
        s.fp8 = int(kb.dtype == torch.uint8)
        return s

    # ------------------------------------------------------------------ reference methods
    def prefetch_prefix_kv_buffer(self, table: Tensor, device: torch.device) -> Tuple[Tensor, Tensor]:
        """Dense device copies ``[1, n, head, dim]`` of the pool rows listed in ``table``."""
        k, v = self.gather_rows(table, extra_rows=0)
        return k.unsqueeze(0), v.unsqueeze(0)

    def gather_rows(self, table: Tensor, extra_rows: int = 0) -> Tuple[Tensor, Tensor]:
        """Device tensors ``[n + extra_rows, head, dim]`` whose first ``n`` rows are the pool rows listed in ``table``;
        the device reads the pinned pools in place on the current stream (nothing blocks the host)."""
        rows = table.reshape(-1).to(self.device, dtype=torch.int64).contiguous()
        n = rows.numel()
        out = []
        for pool in (self.k_uvm, self.v_uvm):
            dst = torch.empty((n + extra_rows, self.head_kv, self.head_dim), dtype=pool.bank_cpu.dtype, device=self.device)
            N.pool_read_rows(pool.device_ptr, pool.bank_cpu.stride(0), pool.bank_cpu.stride(1), self.head_kv,
                             self.head_dim, N.storage_code(pool.bank_cpu), rows, dst, self.device)
            out.append(dst)
        return out[0], out[1]

    def set_kv_buffer(self, table: Tensor, table_gpu: Tensor, cache_k: Tensor, cache_v: Tensor):
        """Store rows into the host pools and keep resident cache blocks current."""
        assert table.device == cache_k.device and cache_v.device == cache_k.device
        if cache_k.device.type == "cpu":
            idx = table.reshape(-1).to(torch.int64)
            self.k_uvm.bank_cpu.index_copy_(0, idx, _as_stored(cache_k.reshape(-1, self.head_kv, self.head_dim), self.k_uvm.dtype))
            self.v_uvm.bank_cpu.index_copy_(0, idx, _as_stored(cache_v.reshape(-1, self.head_kv, self.head_dim), self.v_uvm.dtype))
        else:
            rows = table.reshape(-1).to(torch.int64).contiguous()
            for pool, src in ((self.k_uvm, cache_k), (self.v_uvm, cache_v)):
                src = _as_stored(src.reshape(-1, self.head_kv, self.head_dim), pool.dtype)
                N.pool_write_rows(pool.device_ptr, pool.bank_cpu.stride(0), pool.bank_cpu.stride(1), self.head_kv,
                                  self.head_dim, N.storage_code(pool.bank_cpu), rows, src, self.device)
        self.mask_k_cache.on_set_kv_buffer(table_gpu, cache_k, None)
        self.sa_kv_cache.on_set_kv_buffer(table_gpu, cache_k, cache_v)
        idx_gpu = table_gpu.reshape(-1).to(torch.int64)
        for pool in (self.k_uvm, self.v_uvm):
            pool.metadata.index_put_((idx_gpu,), torch.index_select(pool.metadata, 0, idx_gpu) + 1)

    def enable_miss_stream(self) -> bool:
        """Fetch missed blocks on a side stream from now on (``miss_stream``); returns whether that stream was seen to
        run beside the current one (see ``concurrent_stream``)."""
        self.miss_stream, beside = concurrent_stream(self.device)
        # set-up is also the time to record the fetch graphs (a capture synchronises the device)
        self.mask_k_cache.prepare_miss_graph()
        self.sa_kv_cache.prepare_miss_graph()
        return beside

    def _wait_pending_write(self, stream: Optional[torch.cuda.Stream] = None):
        """Order ``stream`` (default: the current one) after a store into the pools issued on another stream: a fetch
        that ran beside the store could copy a pool row's old bytes into a block that the store's write-through
        had just found absent."""
        if self.pending_write is not None:
            (stream or torch.cuda.current_stream(self.device)).wait_event(self.pending_write)

    def handle_cache_miss(self, metadata=None, after: Optional[torch.cuda.Event] = None):
        """``after``: with ``miss_stream`` set, an event recorded behind the step whose misses are to be fetched; what
        the caller has enqueued on the current stream since then (the next layers) runs beside the fetch."""
        stats_m = getattr(metadata, "mask_cache_statistics", None)
        stats_s = getattr(metadata, "sa_cache_statistics", None)
        self._wait_pending_write(self.miss_stream)
        self.mask_k_cache.handle_cache_miss(metadata=metadata, stats=stats_m, stream=self.miss_stream, after=after)
        self.sa_kv_cache.handle_cache_miss(metadata=metadata, stats=stats_s, stream=self.miss_stream, after=after)

    def flush(self):
        self._wait_pending_write()
        self.mask_k_cache.flush()
        self.sa_kv_cache.flush()
