"""ctypes binding of ``libhipattn.so`` (the C ABI declared in ``include/hipattn.h``).

PyTorch is used only for device memory and the current HIP stream; every kernel is entered
through the plain-C entry points.  Loading fails loudly when the library is missing: there is
no CPU or eager fallback behind this module.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.environ.get("HIPATTN_LIBRARY", os.path.join(_HERE, "libhipattn.so"))
_lib = None

F32, BF16 = 0, 1


class HipAttnError(RuntimeError):
    pass


class QStruct(ctypes.Structure):
    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("stride_b", ctypes.c_int64), ("stride_t", ctypes.c_int64), ("stride_h", ctypes.c_int64),
        ("pos", ctypes.c_void_p),
        ("pos_stride_b", ctypes.c_int64), ("pos_stride_t", ctypes.c_int64),
        ("B", ctypes.c_int32), ("TDST", ctypes.c_int32), ("HEAD", ctypes.c_int32), ("HID", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("rope", ctypes.c_void_p),
        ("logit_softcap", ctypes.c_float),
        ("non_causal", ctypes.c_int32),
    ]


class RopeStruct(ctypes.Structure):
    _fields_ = [
        ("cos", ctypes.c_void_p), ("sin", ctypes.c_void_p),
        ("stride_t", ctypes.c_int64), ("len", ctypes.c_int64),
        ("backend", ctypes.c_int32),
        ("k_side_delta", ctypes.c_int64),
        ("model_context_length", ctypes.c_int64),
    ]


EXTEND_BACKENDS = {"relative": 1, "streaming": 2, "infllm": 3, "dynamic_extend": 4, "self_extend": 5}


class KVStruct(ctypes.Structure):
    _fields_ = [
        ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("k_stride_b", ctypes.c_int64), ("k_stride_t", ctypes.c_int64), ("k_stride_h", ctypes.c_int64),
        ("v_stride_b", ctypes.c_int64), ("v_stride_t", ctypes.c_int64), ("v_stride_h", ctypes.c_int64),
        ("tsrc", ctypes.c_int64), ("max_tsrc", ctypes.c_int64),
        ("block_table", ctypes.c_void_p), ("cache_seq_lens", ctypes.c_void_p),
        ("bt_stride_b", ctypes.c_int64),
        ("bt_is64", ctypes.c_int32), ("sl_is64", ctypes.c_int32),
        ("paged", ctypes.c_int32), ("page_size", ctypes.c_int32),
        ("HKV", ctypes.c_int32),
        ("cache", ctypes.c_void_p),
        ("access_flags", ctypes.c_void_p), ("miss_flags", ctypes.c_void_p),
        ("flags_stride_b", ctypes.c_int64), ("flags_stride_h", ctypes.c_int64),
        ("fp8", ctypes.c_int32),
    ]


_FP8_DTYPES = (torch.uint8, torch.float8_e5m2)  # a float8_e5m2 cache, or its uint8 view (paged_hip.py:409-418)


class CacheDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32), ("HKV", ctypes.c_int32), ("HID", ctypes.c_int32),
        ("block_tokens", ctypes.c_int32), ("with_v", ctypes.c_int32),
        ("pool_rows", ctypes.c_int64), ("slots", ctypes.c_int64),
        ("host_k", ctypes.c_void_p), ("host_v", ctypes.c_void_p),
        ("host_stride_row", ctypes.c_int64), ("host_stride_h", ctypes.c_int64),
        ("bank", ctypes.c_void_p), ("table", ctypes.c_void_p), ("last_use", ctypes.c_void_p),
        ("backref", ctypes.c_void_p), ("miss", ctypes.c_void_p), ("workspace", ctypes.c_void_p),
    ]


class CacheSizes(ctypes.Structure):
    _fields_ = [
        ("n_blocks", ctypes.c_int64), ("bank_bytes", ctypes.c_int64), ("table_bytes", ctypes.c_int64),
        ("last_use_bytes", ctypes.c_int64), ("backref_bytes", ctypes.c_int64), ("miss_bytes", ctypes.c_int64),
        ("workspace_bytes", ctypes.c_int64),
    ]


def lib_path() -> str:
    return _LIB_PATH


def lib():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise HipAttnError(
                f"{_LIB_PATH} is missing: build it with `make -C hip-attention_amd/csrc` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`). There is no fallback path.")
        L = ctypes.CDLL(_LIB_PATH)
        L.hipattn_version.restype = ctypes.c_char_p
        L.hipattn_last_error.restype = ctypes.c_char_p
        L.hipattn_bsa_decode_workspace_bytes.restype = ctypes.c_int64
        L.hipattn_mask_stage_workspace_bytes.restype = ctypes.c_int64
        L.hipattn_bsa_decode_default_splits.restype = ctypes.c_int32
        for name in ("hipattn_mask_stage", "hipattn_prescale_k", "hipattn_select_stage", "hipattn_finalize_indices",
                     "hipattn_bsa_prefill", "hipattn_bsa_decode_partial", "hipattn_bsa_decode_merge", "hipattn_bsa_decode",
                     "hipattn_bsa_decode_static",
                     "hipattn_cache_sizes", "hipattn_cache_create", "hipattn_cache_flush",
                     "hipattn_cache_lookup_and_schedule", "hipattn_cache_commit", "hipattn_cache_write_rows",
                     "hipattn_cache_stats", "hipattn_pool_write_rows", "hipattn_host_device_pointer",
                     "hipattn_host_alloc", "hipattn_host_free"):
            getattr(L, name).restype = ctypes.c_int
        L.hipattn_cache_destroy.restype = None
        L.hipattn_cache_destroy.argtypes = [ctypes.c_void_p]
        _lib = L
    return _lib


def check(rc: int, what: str):
    if rc != 0:
        msg = lib().hipattn_last_error().decode()
        kind = "argument error" if rc < 0 else "HIP error"
        raise HipAttnError(f"{what}: {kind} {rc}: {msg}")


FP8_E5M2 = 2  # storage only: offload pools and their caches


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return BF16
    if t.dtype == torch.float32:
        return F32
    raise HipAttnError(f"unsupported dtype {t.dtype}: the kernels take float32 or bfloat16")


def storage_code(t: torch.Tensor) -> int:
    """Code of a K/V storage tensor: float32, bfloat16, or fp8 (e5m2) bytes held as uint8 / float8_e5m2."""
    return FP8_E5M2 if t.dtype in _FP8_DTYPES else dtype_code(t)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device) -> ctypes.c_void_p:
    """The current stream of ``device`` as the pointer the C ABI takes (the raw-handle query where torch has it: a
    tenth of the cost of building a ``torch.cuda.Stream`` object, on a path that makes one per launch)."""
    if _raw_stream is not None:
        if not isinstance(device, torch.device):
            device = torch.device(device)
        idx = device.index
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device() if idx is None else idx))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def make_rope(cos: torch.Tensor, sin: torch.Tensor, backend: str, k_side_delta: int = 0,
              model_context_length: int = 0, attention: bool = False) -> RopeStruct:
    """Describe RoPE tables ``[len, >= HID/2]`` (q's dtype, unit inner stride) and the rotation rule of one call.
    ``attention`` marks a call of block sparse attention, which knows fewer rules than the mask stage."""
    # the reference's attention kernels know neither "relative" nor "self_extend" (attention_extend_bsa.py:62-63)
    built = [b for b in EXTEND_BACKENDS if not (attention and b in ("relative", "self_extend"))]
    if backend not in built:
        where = "block sparse attention" if attention else "the mask stage"
        raise NotImplementedError(f"extend backend {backend!r} is not built for {where} (built: {sorted(built)})")
    assert cos.ndim == 2 and sin.shape == cos.shape and cos.stride(1) == 1 and sin.stride(1) == 1
    assert cos.stride(0) == sin.stride(0) and cos.dtype == sin.dtype
    r = RopeStruct()
    r.cos, r.sin = cos.data_ptr(), sin.data_ptr()
    r.stride_t, r.len = cos.stride(0), cos.shape[0]
    r.backend = EXTEND_BACKENDS[backend]
    r.k_side_delta = k_side_delta
    r.model_context_length = int(model_context_length)
    return r


def make_q(q: torch.Tensor, pos: torch.Tensor, rope: Optional[RopeStruct] = None,
           logit_softcap: Optional[float] = None, non_causal: bool = False) -> QStruct:
    assert q.ndim == 4 and q.stride(3) == 1
    assert pos.dtype == torch.int64 and pos.ndim == 2
    s = QStruct()
    s.logit_softcap = float(logit_softcap or 0.0)
    s.non_causal = int(bool(non_causal))
    s._pos_keep = pos  # the struct holds a bare pointer to it
    if rope is not None:
        s._rope_keep = rope  # the struct holds a bare pointer to it
        s.rope = ctypes.addressof(rope)
    s.ptr = q.data_ptr()
    s.stride_b, s.stride_t, s.stride_h = q.stride(0), q.stride(1), q.stride(2)
    s.pos = pos.data_ptr()
    s.pos_stride_b, s.pos_stride_t = pos.stride(0), pos.stride(1)
    s.B, s.TDST, s.HEAD, s.HID = q.shape
    s.dtype = dtype_code(q)
    return s


def make_kv_dense(k: torch.Tensor, v: torch.Tensor) -> KVStruct:
    assert k.ndim == 4 and k.stride(3) == 1 and v.stride(3) == 1
    s = KVStruct()
    s.k, s.v = k.data_ptr(), v.data_ptr()
    s.k_stride_b, s.k_stride_t, s.k_stride_h = k.stride(0), k.stride(1), k.stride(2)
    s.v_stride_b, s.v_stride_t, s.v_stride_h = v.stride(0), v.stride(1), v.stride(2)
    s.tsrc = k.shape[1]
    s.max_tsrc = k.shape[1]
    s.paged = 0
    s.page_size = 1
    s.HKV = k.shape[2]
    return s


def set_flags(s: KVStruct, access: Optional[torch.Tensor], miss: Optional[torch.Tensor]) -> KVStruct:
    """Attach ``uint8 [B, HKV, pages]`` access / miss flag tensors to a KV description (returns a copy)."""
    out = KVStruct.from_buffer_copy(s)
    if access is not None:
        assert access.dtype == torch.uint8 and access.ndim == 3 and access.stride(2) == 1, \
            "statistics flags are bytes until a counter has been read; a call needs fresh ones"
        out.access_flags = access.data_ptr()
        out.flags_stride_b, out.flags_stride_h = access.stride(0), access.stride(1)
        if miss is not None:
            assert miss.shape == access.shape and miss.stride() == access.stride() and miss.dtype == torch.uint8
            out.miss_flags = miss.data_ptr()
    return out


def make_kv_paged(k_cache, v_cache, block_table, cache_seq_lens, max_tsrc: int) -> KVStruct:
    assert k_cache.ndim == 4 and k_cache.stride(3) == 1 and v_cache.stride(3) == 1
    assert block_table.ndim == 2 and block_table.stride(1) == 1
    assert cache_seq_lens.ndim == 1 and cache_seq_lens.stride(0) == 1
    assert block_table.dtype in (torch.int32, torch.int64)
    assert cache_seq_lens.dtype in (torch.int32, torch.int64)
    s = KVStruct()
    s.k, s.v = k_cache.data_ptr(), v_cache.data_ptr()
    s.k_stride_b, s.k_stride_t, s.k_stride_h = k_cache.stride(0), k_cache.stride(1), k_cache.stride(2)
    s.v_stride_b, s.v_stride_t, s.v_stride_h = v_cache.stride(0), v_cache.stride(1), v_cache.stride(2)
    s.tsrc = 0
    s.max_tsrc = max_tsrc
    s.block_table = block_table.data_ptr()
    s.cache_seq_lens = cache_seq_lens.data_ptr()
    s.bt_stride_b = block_table.stride(0)
    s.bt_is64 = int(block_table.dtype == torch.int64)
    s.sl_is64 = int(cache_seq_lens.dtype == torch.int64)
    s.paged = 1
    s.page_size = k_cache.shape[1]
    s.HKV = k_cache.shape[2]
    if k_cache.dtype in _FP8_DTYPES:
        if v_cache.dtype not in _FP8_DTYPES:
            raise HipAttnError("k_cache is fp8 but v_cache is not")
        s.fp8 = 1
    elif k_cache.dtype == torch.float8_e4m3fn:
        raise NotImplementedError("fp8 KV caches are read as e5m2 (as the reference does); e4m3 is not built")
    return s


# ------------------------------------------------------------------ optional per-launch timing
_profile = None


def profile_begin():
    """Start recording a (name, start_event, end_event) triple around every kernel entry point."""
    global _profile
    _profile = []


def profile_end():
    """Stop recording and return ``[(name, milliseconds), ...]`` in launch order (synchronises)."""
    global _profile
    rec, _profile = _profile, None
    torch.cuda.synchronize()
    return [(name, s.elapsed_time(e)) for name, s, e in (rec or [])]


class _timed:
    def __init__(self, name):
        self.name = name

    def __enter__(self):
        if _profile is not None:
            self.s = torch.cuda.Event(enable_timing=True)
            self.e = torch.cuda.Event(enable_timing=True)
            self.s.record()
        return self

    def __exit__(self, *exc):
        if _profile is not None and exc[0] is None:
            self.e.record()
            _profile.append((self.name, self.s, self.e))
        return False


# ------------------------------------------------------------------ thin wrappers, one per entry point

def prescale_k(k: torch.Tensor, device, head_major: bool = False) -> torch.Tensor:
    """``bf16(k * c_k)`` for a whole 4-D bf16 key tensor (dense ``[B,T,HKV,D]`` or a paged cache).

    ``head_major``: the copy is laid out ``[HKV, n0, n1, D]`` in memory (and returned as a view of the input's shape),
    so that consecutive tokens of a kv head -- of a page, for a paged cache -- are consecutive rows."""
    assert k.ndim == 4 and k.dtype == torch.bfloat16 and k.stride(3) == 1
    if head_major:
        return prescale_k(k.permute(2, 0, 1, 3), device).permute(1, 2, 0, 3)
    out = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    with _timed("prescale_k"):
      rc = lib().hipattn_prescale_k(
        _p(k), ctypes.c_int64(k.stride(0)), ctypes.c_int64(k.stride(1)), ctypes.c_int64(k.stride(2)),
        ctypes.c_int64(k.shape[0]), ctypes.c_int32(k.shape[1]), ctypes.c_int32(k.shape[2]),
        ctypes.c_int32(k.shape[3]), _p(out), stream_ptr(device))
    check(rc, "hipattn_prescale_k")
    return out


def prescale_k_rope(k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions, device) -> torch.Tensor:
    """``[len(positions), *k.shape]``: for each position p the copy ``bf16(rot(k, p) * c_k)`` of a 4-D bf16 key tensor."""
    assert k.ndim == 4 and k.dtype == torch.bfloat16 and k.stride(3) == 1
    assert cos.dtype == torch.bfloat16 and sin.dtype == torch.bfloat16 and cos.stride(1) == 1 and sin.stride(1) == 1
    out = torch.empty((len(positions),) + tuple(k.shape), dtype=k.dtype, device=k.device)
    esz = 2
    for i, p in enumerate(positions):
        with _timed("prescale_k"):
          rc = lib().hipattn_prescale_k_rope(
            _p(k), ctypes.c_int64(k.stride(0)), ctypes.c_int64(k.stride(1)), ctypes.c_int64(k.stride(2)),
            ctypes.c_int64(k.shape[0]), ctypes.c_int32(k.shape[1]), ctypes.c_int32(k.shape[2]),
            ctypes.c_int32(k.shape[3]), ctypes.c_void_p(cos.data_ptr() + p * cos.stride(0) * esz),
            ctypes.c_void_p(sin.data_ptr() + p * sin.stride(0) * esz), _p(out[i]), stream_ptr(device))
        check(rc, "hipattn_prescale_k_rope")
    return out


def prescale_k_rope_chunks(k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, first: int, chunk: int, device) -> torch.Tensor:
    """``bf16(rot(k[b, t, h], (t - first) // chunk) * c_k)`` for a dense ``[B, T, HKV, D]`` bf16 key tensor: every key
    rotated to the place of its chunk in a first stage's list (the streaming rule there) and scaled."""
    assert k.ndim == 4 and k.dtype == torch.bfloat16 and k.stride(3) == 1
    assert cos.dtype == torch.bfloat16 and sin.dtype == torch.bfloat16 and cos.stride(1) == 1 and sin.stride(1) == 1
    assert cos.stride(0) == sin.stride(0) and cos.shape[0] == sin.shape[0]
    out = torch.empty(tuple(k.shape), dtype=k.dtype, device=k.device)
    with _timed("prescale_k"):
        rc = lib().hipattn_prescale_k_rope_chunks(
            _p(k), ctypes.c_int64(k.stride(0)), ctypes.c_int64(k.stride(1)), ctypes.c_int64(k.stride(2)),
            ctypes.c_int64(k.shape[0]), ctypes.c_int32(k.shape[1]), ctypes.c_int32(k.shape[2]),
            ctypes.c_int32(k.shape[3]), _p(cos), _p(sin), ctypes.c_int64(cos.stride(0)), ctypes.c_int64(cos.shape[0]),
            ctypes.c_int32(first), ctypes.c_int32(chunk), _p(out), stream_ptr(device))
    check(rc, "hipattn_prescale_k_rope_chunks")
    return out


def mask_stage(qs, kvs, chunk_left, hg, n, chunk, right_clamp, bs, bq, stride_q, block_chunk, scan_stride,
               sw_eff, terminate, scores, left_out, device, k_prescaled=False, reduce_heads=False, workspace=None,
               near_pool=False):
    """``workspace``: the tensor an earlier call with the same query rows (same q, bs, bq, stride_q, scan_stride, no
    rotation) returned; the rows it holds are used as they are.  ``near_pool``: the keys are a paged pool that spans
    less than 32 GiB (a dense tensor's extent is worked out by the library).
    Returns the workspace (None for f32)."""
    q_ready = workspace is not None
    if workspace is None:
        need = lib().hipattn_mask_stage_workspace_bytes(
            ctypes.c_int32(qs.dtype), ctypes.c_int32(qs.B), ctypes.c_int32(bs), ctypes.c_int32(qs.HEAD),
            ctypes.c_int32(qs.HID), ctypes.c_int32(bq), ctypes.c_int32(stride_q))
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=scores.device) if need > 0 else None
    with _timed(f"mask_stage[n={n},chunk={chunk},rows={bq // stride_q}]"):
      rc = lib().hipattn_mask_stage(
        ctypes.byref(qs), ctypes.byref(kvs), _p(chunk_left), ctypes.c_int32(hg), ctypes.c_int32(n),
        ctypes.c_int32(chunk), ctypes.c_int64(right_clamp), ctypes.c_int32(bs), ctypes.c_int32(bq),
        ctypes.c_int32(stride_q), ctypes.c_int32(block_chunk), ctypes.c_int32(scan_stride),
        ctypes.c_int32(sw_eff), ctypes.c_int32(terminate), ctypes.c_int32(int(bool(k_prescaled)) | (2 if q_ready else 0) | (4 if near_pool else 0)),
        ctypes.c_int32(int(reduce_heads)), _p(workspace),
        _p(scores),
        _p(left_out), stream_ptr(device))
    check(rc, "hipattn_mask_stage")
    return workspace


def select_stage(scores, chunk_left, B, bs_in, bs_out, row_rep, HEAD, hg, n, k, chunk, splits, next_left, device,
                 left64=None, right64=None, next_scores=None):
    """``next_scores``: the next stage's head-reduced scores (shape of ``next_left`` with ``hg == 1``), set to -inf here
    so that ``mask_stage(..., reduce_heads=2)`` finds them initialised."""
    with _timed("select_stage"):
      rc = lib().hipattn_select_stage(
        _p(scores), _p(chunk_left), ctypes.c_int32(B), ctypes.c_int32(bs_in), ctypes.c_int32(bs_out),
        ctypes.c_int32(row_rep), ctypes.c_int32(HEAD), ctypes.c_int32(hg), ctypes.c_int32(n), ctypes.c_int32(k),
        ctypes.c_int32(chunk), ctypes.c_int32(splits), _p(next_left), _p(left64), _p(right64), _p(next_scores),
        stream_ptr(device))
    check(rc, "hipattn_select_stage")


def finalize_indices(scores, left_out, pos, B, bs, bdst, scan_stride, HEAD, score_heads, hg, n, K, chunk, bq,
                     indices, ks, ks_start_end, device):
    with _timed("finalize_indices"):
      rc = lib().hipattn_finalize_indices(
        _p(scores), _p(left_out), _p(pos), ctypes.c_int64(pos.stride(0)), ctypes.c_int64(pos.stride(1)),
        ctypes.c_int32(B), ctypes.c_int32(bs), ctypes.c_int32(bdst), ctypes.c_int32(scan_stride),
        ctypes.c_int32(HEAD), ctypes.c_int32(score_heads), ctypes.c_int32(hg), ctypes.c_int32(n), ctypes.c_int32(K),
        ctypes.c_int32(chunk),
        ctypes.c_int32(bq), _p(indices), _p(ks), _p(ks_start_end), stream_ptr(device))
    check(rc, "hipattn_finalize_indices")


def bsa_prefill(qs, kvs, indices, ks_start_end, BK, bq, bk, sw, sink, share_first_head, impl, out, device,
                k_prescaled=None):
    assert indices.dtype == torch.int64 and indices.is_contiguous()
    assert ks_start_end.dtype == torch.int32 and ks_start_end.is_contiguous()
    with _timed("bsa_prefill"):
      rc = lib().hipattn_bsa_prefill(
        ctypes.byref(qs), ctypes.byref(kvs), _p(indices), _p(ks_start_end), ctypes.c_int32(indices.shape[1]),
        ctypes.c_int32(BK), ctypes.c_int32(bq), ctypes.c_int32(bk), ctypes.c_int32(sw), ctypes.c_int32(sink),
        ctypes.c_int32(int(share_first_head)), ctypes.c_int32(impl), _p(k_prescaled), _p(out),
        ctypes.c_int64(out.stride(0)),
        ctypes.c_int64(out.stride(1)), ctypes.c_int64(out.stride(2)), stream_ptr(device))
    check(rc, "hipattn_bsa_prefill")


def bsa_decode(qs, kvs, indices, ks_start_end, BK, bk, sw, sink, out, device, nsplits=0, workspace=None,
               second_stage_k=0):
    assert indices.dtype == torch.int64 and indices.is_contiguous()
    assert ks_start_end.dtype == torch.int32 and ks_start_end.is_contiguous()
    L = lib()
    B, HEAD, HID = qs.B, qs.HEAD, qs.HID
    if nsplits <= 0:
        nsplits = L.hipattn_bsa_decode_default_splits(ctypes.c_int32(B), ctypes.c_int32(kvs.HKV),
                                                      ctypes.c_int32(BK * bk + sink + sw + 1))
    need = L.hipattn_bsa_decode_workspace_bytes(ctypes.c_int32(B), ctypes.c_int32(HEAD), ctypes.c_int32(HID),
                                                ctypes.c_int32(nsplits))
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty(need // 4, dtype=torch.float32, device=out.device)
    with _timed("bsa_decode"):
      rc = L.hipattn_bsa_decode(
        ctypes.byref(qs), ctypes.byref(kvs), _p(indices), _p(ks_start_end), ctypes.c_int32(indices.shape[1]),
        ctypes.c_int32(BK), ctypes.c_int32(bk), ctypes.c_int32(sw), ctypes.c_int32(sink),
        ctypes.c_int32(second_stage_k), ctypes.c_int32(nsplits), _p(workspace), _p(out),
        ctypes.c_int64(out.stride(0)), ctypes.c_int64(out.stride(2)), stream_ptr(device))
    check(rc, "hipattn_bsa_decode")
    return workspace


def bsa_decode_static(qs, kvs, indices, ks_start_end, BK, bk, sw, sink, out, device, nsplits=0, second_stage_k=0):
    """Decode attention through ``hipattn_bsa_decode_static``: the split partials live in a device array inside the
    library, so the call allocates nothing (for callers that cannot: graph capture, tight serving loops)."""
    assert indices.dtype == torch.int64 and indices.is_contiguous()
    assert ks_start_end.dtype == torch.int32 and ks_start_end.is_contiguous()
    with _timed("bsa_decode"):
      rc = lib().hipattn_bsa_decode_static(
        ctypes.byref(qs), ctypes.byref(kvs), _p(indices), _p(ks_start_end), ctypes.c_int32(indices.shape[1]),
        ctypes.c_int32(BK), ctypes.c_int32(bk), ctypes.c_int32(sw), ctypes.c_int32(sink),
        ctypes.c_int32(second_stage_k), ctypes.c_int32(nsplits), _p(out), ctypes.c_int64(out.stride(0)),
        ctypes.c_int64(out.stride(2)), stream_ptr(device))
    check(rc, "hipattn_bsa_decode_static")


# ------------------------------------------------------------------ offload cache

class HostPool:
    """Pinned host memory from ``hipattn_host_alloc`` exposed as a CPU tensor; freed with the object."""

    def __init__(self, shape, dtype: torch.dtype, coherent: bool = True):
        n = 1
        for d in shape:
            n *= int(d)
        self.nbytes = max(16, n * torch.empty((), dtype=dtype).element_size())
        out = ctypes.c_void_p(0)
        check(lib().hipattn_host_alloc(ctypes.c_int64(self.nbytes), ctypes.c_int32(int(coherent)), ctypes.byref(out)),
              "hipattn_host_alloc")
        self.ptr = int(out.value)
        buf = (ctypes.c_uint8 * self.nbytes).from_address(self.ptr)
        self.tensor = torch.frombuffer(buf, dtype=dtype, count=n).view(*shape)

    def __del__(self):
        p, self.ptr = getattr(self, "ptr", 0), 0
        try:
            if p and _lib is not None:
                self.tensor = None
                _lib.hipattn_host_free(ctypes.c_void_p(p))
        except Exception:  # interpreter shutdown
            pass


def host_device_pointer(t: torch.Tensor) -> int:
    """Device-visible address of a pinned host tensor."""
    assert not t.is_cuda, "the host pool must live in pinned host memory"
    out = ctypes.c_void_p(0)
    rc = lib().hipattn_host_device_pointer(ctypes.c_void_p(t.data_ptr()), ctypes.byref(out))
    check(rc, "hipattn_host_device_pointer")
    return int(out.value)


def cache_sizes(desc: CacheDesc, max_fetch: int) -> CacheSizes:
    out = CacheSizes()
    check(lib().hipattn_cache_sizes(ctypes.byref(desc), ctypes.c_int64(max_fetch), ctypes.byref(out)),
          "hipattn_cache_sizes")
    return out


def cache_create(desc: CacheDesc, max_fetch: int, device) -> int:
    handle = ctypes.c_void_p(0)
    check(lib().hipattn_cache_create(ctypes.byref(desc), ctypes.c_int64(max_fetch), ctypes.byref(handle),
                                     stream_ptr(device)), "hipattn_cache_create")
    return int(handle.value)


def cache_destroy(handle: int):
    if _lib is not None and handle and ctypes is not None:
        _lib.hipattn_cache_destroy(ctypes.c_void_p(handle))


def cache_flush(handle: int, device):
    check(lib().hipattn_cache_flush(ctypes.c_void_p(handle), stream_ptr(device)), "hipattn_cache_flush")


def cache_schedule(handle: int, device):
    with _timed("cache_lookup_and_schedule"):
        rc = lib().hipattn_cache_lookup_and_schedule(ctypes.c_void_p(handle), stream_ptr(device))
    check(rc, "hipattn_cache_lookup_and_schedule")


def cache_commit(handle: int, device):
    with _timed("cache_commit"):
        rc = lib().hipattn_cache_commit(ctypes.c_void_p(handle), stream_ptr(device))
    check(rc, "hipattn_cache_commit")


def cache_write_rows(handle: int, rows: torch.Tensor, k_rows: torch.Tensor, v_rows: Optional[torch.Tensor], device):
    assert rows.dtype == torch.int64 and rows.is_cuda and rows.is_contiguous()
    assert k_rows.is_cuda and k_rows.is_contiguous() and (v_rows is None or (v_rows.is_cuda and v_rows.is_contiguous()))
    check(lib().hipattn_cache_write_rows(ctypes.c_void_p(handle), _p(rows), ctypes.c_int64(rows.numel()), _p(k_rows),
                                         _p(v_rows), stream_ptr(device)), "hipattn_cache_write_rows")


def cache_stats(handle: int, device) -> list:
    out = (ctypes.c_int64 * 8)()
    check(lib().hipattn_cache_stats(ctypes.c_void_p(handle), out, stream_ptr(device)), "hipattn_cache_stats")
    return list(out)


def pool_read_rows(pool_ptr: int, stride_row: int, stride_h: int, HKV: int, HID: int, dtype: int,
                   rows: torch.Tensor, dst: torch.Tensor, device):
    """Gather rows of the pinned host pool into device ``dst [>= n, HKV, HID]`` (first ``n = rows.numel()`` rows)."""
    assert rows.dtype == torch.int64 and rows.is_cuda and rows.is_contiguous() and dst.is_cuda
    assert dst.ndim == 3 and dst.stride(2) == 1 and dst.stride(1) == HID and dst.shape[0] >= rows.numel()
    check(lib().hipattn_pool_read_rows(ctypes.c_void_p(pool_ptr), ctypes.c_int64(stride_row), ctypes.c_int64(stride_h),
                                       ctypes.c_int32(HKV), ctypes.c_int32(HID), ctypes.c_int32(dtype), _p(rows),
                                       ctypes.c_int64(rows.numel()), _p(dst), ctypes.c_int64(dst.stride(0)),
                                       stream_ptr(device)),
          "hipattn_pool_read_rows")


def pool_write_rows(pool_ptr: int, stride_row: int, stride_h: int, HKV: int, HID: int, dtype: int,
                    rows: torch.Tensor, src: torch.Tensor, device):
    """Scatter device rows ``src [n, HKV, HID]`` into the pinned host pool at ``rows``."""
    assert rows.dtype == torch.int64 and rows.is_cuda and rows.is_contiguous() and src.is_cuda and src.is_contiguous()
    check(lib().hipattn_pool_write_rows(ctypes.c_void_p(pool_ptr), ctypes.c_int64(stride_row), ctypes.c_int64(stride_h),
                                        ctypes.c_int32(HKV), ctypes.c_int32(HID), ctypes.c_int32(dtype), _p(rows),
                                        ctypes.c_int64(rows.numel()), _p(src), stream_ptr(device)),
          "hipattn_pool_write_rows")
