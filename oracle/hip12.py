"""CPU oracle driver for ``hip_attention_12`` -- TEST INFRASTRUCTURE ONLY.

Restates the host-side driver of the reference operator
(``src/hip_attn/v1_2/attention_extend.py:1918-3133``) in NumPy and calls the C restatement of
the device kernels in ``hip_oracle.c``.  The shipped package never imports this module; tests,
``__graft_entry__.smoke`` and the benchmark's ``cpu_baseline`` leg do.

Unlike the product, which keeps one chunk list per (batch, query block) when scores are
max-reduced over heads, this driver keeps the reference's full ``[B, BDST, HEAD, chunks]``
int64 tensors and performs every glue step (truncate, realign, sort, split, top-k, gather)
literally, so the product's shortcuts are checked against the long form.

Tie-break rule (the reference leaves ties to ``torch.topk`` / unstable ``sort``): candidates are
ordered by (score descending, current list position ascending).

bf16 tensors are carried as ``uint16`` bit patterns.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

INT64_MAX = np.iinfo(np.int64).max


class _Tensors(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int),
        ("B", ctypes.c_int),
        ("TDST", ctypes.c_int),
        ("HEAD", ctypes.c_int),
        ("HKV", ctypes.c_int),
        ("HID", ctypes.c_int),
        ("q", ctypes.c_void_p),
        ("pos", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("TSRC", ctypes.c_int64),
        ("k_cache", ctypes.c_void_p),
        ("v_cache", ctypes.c_void_p),
        ("page_size", ctypes.c_int),
        ("block_table", ctypes.c_void_p),
        ("bt_cols", ctypes.c_int64),
        ("cache_seq_lens", ctypes.c_void_p),
        ("MAX_TSRC", ctypes.c_int64),
        ("access", ctypes.c_void_p),
        ("access_pages", ctypes.c_int64),
        ("rope_cos", ctypes.c_void_p),
        ("rope_sin", ctypes.c_void_p),
        ("rope_len", ctypes.c_int64),
        ("scan_backend", ctypes.c_int),
        ("sa_backend", ctypes.c_int),
        ("logit_softcap", ctypes.c_float),
        ("model_context_length", ctypes.c_int64),
        ("non_causal", ctypes.c_int),
    ]


EXTEND_BACKENDS = {None: 0, "relative": 1, "streaming": 2, "infllm": 3, "dynamic_extend": 4, "self_extend": 5}


def build(force: bool = False) -> str:
    """Compile ``libhip_oracle.so`` next to this file and return its path."""
    so = os.path.join(_HERE, "libhip_oracle.so")
    src = os.path.join(_HERE, "hip_oracle.c")
    if force or (not os.path.exists(so)) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libhip_oracle.so"], stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        L = ctypes.CDLL(build())
        L.hipo_round_bf16.restype = ctypes.c_float
        L.hipo_round_bf16.argtypes = [ctypes.c_float]
        L.hipo_dot.restype = ctypes.c_float
        L.hipo_dot.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        L.hipo_dot_mfma.restype = ctypes.c_float
        L.hipo_dot_mfma.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        L.hipo_scale_constants.restype = None
        L.hipo_mask_stage.restype = ctypes.c_int
        L.hipo_bsa.restype = ctypes.c_int
        L.hipo_rope_row.restype = None
        L.hipo_num_threads.restype = ctypes.c_int
        _LIB = L
    return _LIB


# ------------------------------------------------------------------ bf16 helpers (uint16 bits)

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bf16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (r >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def scale_constants(hid: int, dtype: str):
    cq, ck = ctypes.c_float(), ctypes.c_float()
    lib().hipo_scale_constants(ctypes.c_int(hid), ctypes.c_int(1 if dtype == "bf16" else 0),
                               ctypes.byref(cq), ctypes.byref(ck))
    return cq.value, ck.value


# ------------------------------------------------------------------ argument containers

@dataclass
class OStage:
    """One ScanStage (attention_metadata.py:55-60)."""
    stage_block_size_q: int
    stage_block_stride_q: int
    stage_chunk_size: int
    stage_k: Optional[int]
    stage_stride: int = 1
    stage_extend_backend: Optional[str] = None


def default_stages() -> List[OStage]:
    return [OStage(64, 4, 256, None, 1), OStage(64, 4, 32, 32768, 1), OStage(64, 1, 8, 8192, 1)]


@dataclass
class OArgs:
    """The subset of HiPAttentionArgs the oracle models (attention_metadata.py:134-215)."""
    sink_token_size: int = 256
    sliding_window_size: int = 512
    block_size_k: int = 64  # BLOCK_CHUNK
    second_stage_k: int = 2048
    stages: List[OStage] = field(default_factory=default_stages)
    model_context_length: int = 131072
    extend_context_length: int = 512 * 1024
    block_sparse_block_size_q: Optional[int] = 64
    stage_early_terminate: int = 1
    disable_flashdecode: bool = False
    is_causal: bool = True  # attention_metadata.py:189; read by block sparse attention only
    head_reduce: bool = True  # env HIP_HEAD_REDUCE, default on (attention_extend.py:2566)
    mask_only: bool = False
    # RoPE applied on load (attention_metadata.py:191-198); only using_extend with need_apply_rope is modelled
    using_extend: bool = False
    need_apply_rope: bool = False
    scan_extend_backend: str = "relative"
    sa_extend_backend: str = "streaming"
    logit_softcap: Optional[float] = None  # attention logits only (attention_extend_bsa.py:507-508)


@dataclass
class OInputs:
    dtype: str  # "f32" | "bf16"
    q: np.ndarray  # [B,TDST,HEAD,HID] float32, or uint16 bits for bf16
    pos: np.ndarray  # [B,TDST] int64
    k: Optional[np.ndarray] = None  # [B,TSRC,HKV,HID]
    v: Optional[np.ndarray] = None
    k_cache: Optional[np.ndarray] = None  # [pages,page,HKV,HID]
    v_cache: Optional[np.ndarray] = None
    block_table: Optional[np.ndarray] = None  # [B,cols] int64
    cache_seq_lens: Optional[np.ndarray] = None  # [B] int64
    access: Optional[np.ndarray] = None  # int32 [B,HKV,pages]: flags set by every key row the kernels fetch
    rope_cos: Optional[np.ndarray] = None  # float32 [L,HID] (values of the tables' own dtype, widened)
    rope_sin: Optional[np.ndarray] = None
    model_context_length: int = 131072  # only the "dynamic_extend" rules read it
    scan_backend: Optional[str] = None  # rotation rule of the mask stage / of sparse attention; None = no RoPE
    sa_backend: Optional[str] = None
    logit_softcap: float = 0.0
    non_causal: int = 0  # block sparse attention only: 1 = query-block kernel's form, 2 = decode kernel's (hipo_bsa)

    def c_struct(self, max_tsrc: int):
        np_t = np.uint16 if self.dtype == "bf16" else np.float32
        keep = []

        def arr(a, t):
            if a is None:
                return None
            a = np.ascontiguousarray(a, dtype=t)
            keep.append(a)
            return a.ctypes.data

        B, TDST, HEAD, HID = self.q.shape
        S = _Tensors()
        S.dtype = 1 if self.dtype == "bf16" else 0
        S.B, S.TDST, S.HEAD, S.HID = B, TDST, HEAD, HID
        S.q = arr(self.q, np_t)
        S.pos = arr(self.pos, np.int64)
        if self.k is not None:
            S.HKV = self.k.shape[2]
            S.TSRC = self.k.shape[1]
            S.k = arr(self.k, np_t)
            S.v = arr(self.v if self.v is not None else self.k, np_t)
            S.page_size = 1
        else:
            S.HKV = self.k_cache.shape[2]
            S.TSRC = 0
            S.k = None
            S.v = None
            S.k_cache = arr(self.k_cache, np_t)
            S.v_cache = arr(self.v_cache if self.v_cache is not None else self.k_cache, np_t)
            S.page_size = self.k_cache.shape[1]
            S.block_table = arr(self.block_table, np.int64)
            S.bt_cols = self.block_table.shape[1]
            S.cache_seq_lens = arr(self.cache_seq_lens, np.int64)
        S.MAX_TSRC = max_tsrc
        S.logit_softcap = float(self.logit_softcap or 0.0)
        S.model_context_length = int(self.model_context_length)
        S.non_causal = int(self.non_causal)
        if self.access is not None:
            assert self.access.dtype == np.int32 and self.access.flags.c_contiguous and self.access.ndim == 3
            S.access = self.access.ctypes.data
            S.access_pages = self.access.shape[2]
        if self.scan_backend is not None or self.sa_backend is not None:
            assert self.rope_cos is not None and self.rope_cos.shape == self.rope_sin.shape
            assert self.rope_cos.ndim == 2 and self.rope_cos.shape[1] == HID
            S.rope_cos = arr(self.rope_cos, np.float32)
            S.rope_sin = arr(self.rope_sin, np.float32)
            S.rope_len = self.rope_cos.shape[0]
            S.scan_backend = EXTEND_BACKENDS[self.scan_backend]
            S.sa_backend = EXTEND_BACKENDS[self.sa_backend]
        return S, keep


def cdiv(a, b):
    return -(-a // b)


def npow2(x: int) -> int:
    return 1 if x <= 1 else 1 << (int(x) - 1).bit_length()


def topk_order(scores: np.ndarray, k: int) -> np.ndarray:
    """Positions of the k best entries along the last axis under (score desc, position asc)."""
    order = np.argsort(-scores.astype(np.float64), axis=-1, kind="stable")
    return order[..., :k]


# ------------------------------------------------------------------ kernels

def mask_stage(X: OInputs, max_tsrc, left, right, scores, BS, BQ, stride_q, block_chunk,
               scan_stride, sw_eff, terminate=1):
    """In-place scan of one stage; arrays as in the reference: int64 [B,BS,HEAD,n], f32 scores."""
    assert left.dtype == np.int64 and right.dtype == np.int64 and scores.dtype == np.float32
    assert left.flags.c_contiguous and right.flags.c_contiguous and scores.flags.c_contiguous
    S, keep = X.c_struct(max_tsrc)
    n = left.shape[-1]
    rc = lib().hipo_mask_stage(ctypes.byref(S), ctypes.c_void_p(left.ctypes.data),
                               ctypes.c_void_p(right.ctypes.data), ctypes.c_void_p(scores.ctypes.data),
                               ctypes.c_int(n), ctypes.c_int(scores.shape[-1]), ctypes.c_int(BS),
                               ctypes.c_int(BQ), ctypes.c_int(stride_q), ctypes.c_int(block_chunk),
                               ctypes.c_int(scan_stride), ctypes.c_int(sw_eff), ctypes.c_int(terminate))
    if rc != 0:
        raise RuntimeError(f"hipo_mask_stage failed: {rc}")
    del keep


def rope_row(X: OInputs, row: np.ndarray, pos: int) -> np.ndarray:
    """One row (float32 values of X's dtype) rotated to ``pos`` with X's tables."""
    S, keep = X.c_struct(0)
    if not S.rope_cos:
        raise ValueError("rope_row needs X's tables: give X a scan_backend or sa_backend")
    out = np.ascontiguousarray(row, dtype=np.float32).copy()
    lib().hipo_rope_row(ctypes.byref(S), ctypes.c_void_p(out.ctypes.data), ctypes.c_int64(pos))
    del keep
    return out


def decode_seams(second_stage_k: int, sink: int, sw: int, block_size_k: int, BK: int):
    """``(share, overhang)`` of the decode kernel's programs over an index row of ``BK`` entries: the launcher gives
    the selected blocks ``min(12, ceil(second_stage_k / ceil((second_stage_k + sink + sw) / 8)))`` programs
    (attention_decode_bsa.py:1070-1076) that walk their ``share`` of the row in tiles of ``16 // block_size_k`` entries
    (:1391-1393); ``overhang`` is how far a program's last tile reaches into the next share (:239-247)."""
    chunk = cdiv(second_stage_k + sink + sw, 8)
    programs = min(12, cdiv(second_stage_k, chunk)) if chunk > 0 else 0
    if programs <= 0 or BK <= 0:
        return 0, 0
    share = cdiv(BK, programs)
    tile = max(1, min(16, 16 // block_size_k))
    return share, cdiv(share, tile) * tile - share


def decode_sink_share(second_stage_k: int, sink: int, sw: int) -> int:
    """Sink tokens per program of the decode kernel: ``min(12, ceil(sink / ceil((second_stage_k + sink + sw) / 8)))``
    programs (attention_decode_bsa.py:1077) share the sink evenly (:514)."""
    chunk = cdiv(second_stage_k + sink + sw, 8)
    if sink <= 0 or chunk <= 0:
        return 0
    return cdiv(sink, min(12, cdiv(sink, chunk)))


def seam_multiplicity(j: int, share: int, overhang: int) -> int:
    return int(lib().hipo_seam_multiplicity(ctypes.c_int(j), ctypes.c_int(share), ctypes.c_int(overhang)))


def bsa(X: OInputs, max_tsrc, indices, ks_start_end, block_size_q, block_size_k, sw, sink,
        share_first_head=False, seams=(0, 0), sink_share=0):
    """Block-sparse attention given indices; returns context with q's shape and dtype.  ``seams``: see
    ``decode_seams`` (decode only; ``(0, 0)`` attends every selected block once); ``sink_share``: see
    ``decode_sink_share`` (decode with the streaming rotation rule only; 0 numbers sink tokens by themselves)."""
    S, keep = X.c_struct(max_tsrc)
    indices = np.ascontiguousarray(indices, dtype=np.int64)
    kse = np.ascontiguousarray(ks_start_end, dtype=np.int32)
    out = np.zeros(X.q.shape, dtype=np.uint16 if X.dtype == "bf16" else np.float32)
    rc = lib().hipo_bsa(ctypes.byref(S), ctypes.c_void_p(indices.ctypes.data), ctypes.c_void_p(kse.ctypes.data),
                        ctypes.c_int(indices.shape[1]), ctypes.c_int(indices.shape[2]),
                        ctypes.c_int(block_size_q), ctypes.c_int(block_size_k), ctypes.c_int(sw),
                        ctypes.c_int(sink), ctypes.c_int(1 if share_first_head else 0),
                        ctypes.c_int(seams[0]), ctypes.c_int(seams[1]), ctypes.c_int(sink_share),
                        ctypes.c_void_p(out.ctypes.data))
    if rc != 0:
        raise RuntimeError(f"hipo_bsa failed: {rc}")
    del keep
    return out


# ------------------------------------------------------------------ driver

@dataclass
class OStageCache:
    indices_left: Optional[np.ndarray]
    indices_right: Optional[np.ndarray]
    out_scores: Optional[np.ndarray]


@dataclass
class OMetadata:
    indices: Optional[np.ndarray]
    ks: Optional[np.ndarray]
    ks_count: Optional[np.ndarray]
    ks_start_end: Optional[np.ndarray]
    stage_caches: Optional[List[OStageCache]]
    mask_access: Optional[np.ndarray] = None  # int32 [B,HKV,pages] (None when the mask was reused)
    sa_access: Optional[np.ndarray] = None


def hip_attention_12(X: OInputs, A: OArgs, cached: Optional[OMetadata] = None):
    """Restatement of dual_stage_quadratic_hip_attention (attention_extend.py:1918-3133)."""
    B, TDST, HEAD, HID = X.q.shape
    if X.k is not None:
        TSRC = X.k.shape[1]
        MAX_TSRC = TSRC
    else:
        MAX_TSRC = A.extend_context_length
        TSRC = MAX_TSRC
    stages = A.stages
    assert len(stages) > 0
    STAGE_STRIDE = stages[0].stage_stride
    BQ = stages[0].stage_block_size_q
    BDST = cdiv(TDST, BQ)
    BS = cdiv(BDST, STAGE_STRIDE)
    BLOCK_CHUNK = A.block_size_k
    chunk = stages[0].stage_chunk_size
    n = cdiv(max(0, MAX_TSRC - A.sink_token_size - A.sliding_window_size), chunk)  # :1971-1973

    mask_k = stages[0].stage_chunk_size  # :1976
    sw_orig = A.sliding_window_size
    sw_eff = max(0, sw_orig - mask_k)  # :1978
    sink = A.sink_token_size
    pos = np.ascontiguousarray(X.pos, dtype=np.int64)
    assert pos.shape == (B, TDST)

    stage_caches = [] if (cached is None or cached.stage_caches is None) else cached.stage_caches

    user_backends = (X.scan_backend, X.sa_backend)
    if A.using_extend:
        assert A.need_apply_rope, "only keys stored without rotation are modelled"
        assert X.rope_cos is not None and X.rope_sin is not None
        X.scan_backend, X.sa_backend = A.scan_extend_backend, A.sa_extend_backend
        X.model_context_length = A.model_context_length
    else:
        X.scan_backend = X.sa_backend = None

    # access flags (attention_extend.py:1988-2006): one entry per token (dense) or pool page (paged)
    HKV = X.k.shape[2] if X.k is not None else X.k_cache.shape[2]
    pages = MAX_TSRC if X.k is not None else X.k_cache.shape[0]
    mask_access = None
    sa_access = np.zeros((B, HKV, pages), dtype=np.int32)
    user_access = X.access

    if cached is None or cached.indices is None:
        mask_access = np.zeros((B, HKV, pages), dtype=np.int32)
        X.access = mask_access
        fresh = cached is None or cached.stage_caches is None
        # A cache holding only the (empty) stage-0 entry carries no tensors: the reference would fail on
        # None.clone() (attention_extend.py:2052-2056) although its own replay test passes such a list
        # (tests/v1_2/test_gen3_stage_caching.py:170-181); treated here as a fresh start.
        if not fresh and stage_caches[-1].indices_left is None:
            assert len(stage_caches) == 1
            fresh = True
        if fresh:
            left = np.zeros((B, BS, HEAD, n), dtype=np.int64)
            left[...] = (np.floor(np.arange(n, dtype=np.float64) * chunk + sink)).astype(np.int64)
            right = np.minimum(left + chunk, MAX_TSRC - sw_eff)
            scores = np.full((B, BS, HEAD, npow2(n)), -32000.0, dtype=np.float32)
        else:
            assert len(stage_caches) <= len(stages)
            last = stage_caches[-1]
            left = last.indices_left.copy()
            right = last.indices_right.copy()
            scores = last.out_scores.copy()

        for i, st in enumerate(stages):
            if i < len(stage_caches) - 1:
                continue
            elif i == len(stage_caches) - 1:
                # The reference enters a restarted stage with the query block size and stage stride of stage 0
                # (:1960-1965; the code that switches them, :2092-2124, runs only for stages that are not restarted).
                # Its own restart test keeps them equal over all stages (tests/v1_2/test_gen3_stage_caching.py); a
                # restart at a stage where they differ is not modelled.
                if i > 0 and (st.stage_block_size_q, st.stage_stride) != (stages[0].stage_block_size_q, stages[0].stage_stride):
                    raise NotImplementedError("restart at a stage whose block size or stride differs from stage 0's")
            elif i > 0:
                assert st.stage_k % chunk == 0
                kk = st.stage_k // chunk
                left = left[..., :kk]
                left = (left - sink) // chunk * chunk + sink  # realign :2077-2080
                right = left + chunk
                scores = scores[..., :kk].copy()
                scores.fill(-32000.0)
                order = np.argsort(left, axis=-1, kind="stable")
                left = np.take_along_axis(left, order, -1)
                right = np.take_along_axis(right, order, -1)
                scores = np.take_along_axis(scores, order, -1)
                if BQ != st.stage_block_size_q:
                    assert BQ > st.stage_block_size_q and BQ % st.stage_block_size_q == 0
                    num_split = BQ // st.stage_block_size_q
                    BQ = st.stage_block_size_q
                    BDST = cdiv(TDST, BQ)
                    BS = cdiv(BDST, STAGE_STRIDE)
                    left = np.repeat(left, num_split, 1)[:, -BDST:]
                    right = np.repeat(right, num_split, 1)[:, -BDST:]
                    scores = np.repeat(scores, num_split, 1)[:, -BDST:]
                if STAGE_STRIDE != st.stage_stride:
                    assert st.stage_stride < STAGE_STRIDE
                    rep = STAGE_STRIDE // st.stage_stride
                    left = np.repeat(left, rep, 1)[:, -BDST:]
                    right = np.repeat(right, rep, 1)[:, -BDST:]
                    scores = np.repeat(scores, rep, 1)[:, -BDST:]
                    STAGE_STRIDE = st.stage_stride
                    BS = cdiv(BDST, STAGE_STRIDE)
                assert chunk % st.stage_chunk_size == 0
                splits = chunk // st.stage_chunk_size
                w = np.maximum((right - left).astype(np.float32) / np.float32(splits), np.float32(0))
                ar = np.arange(splits, dtype=np.float32)
                left = (left[..., None] + np.floor(ar * w[..., None]).astype(np.int64)).reshape(*left.shape[:-1], -1)
                right = (right[..., None] - np.floor((np.float32(splits - 1) - ar) * w[..., None]).astype(np.int64)
                         ).reshape(*right.shape[:-1], -1)
                scores = np.repeat(scores, splits, -1)
            else:
                assert st.stage_k is None, "first stage always quadratic"
                STAGE_STRIDE = st.stage_stride

            if i >= len(stage_caches):
                if i == 0:
                    stage_caches.append(OStageCache(None, None, None))
                else:
                    stage_caches.append(OStageCache(left.copy(), right.copy(), scores.copy()))

            chunk = st.stage_chunk_size
            n = left.shape[-1]
            BLOCK_CHUNK = max(16, npow2(min(n, BLOCK_CHUNK)))  # :2194
            left = np.ascontiguousarray(left)
            right = np.ascontiguousarray(right)
            scores = np.ascontiguousarray(scores)
            if A.using_extend:  # :2200-2204
                X.scan_backend = st.stage_extend_backend or A.scan_extend_backend
            mask_stage(X, MAX_TSRC, left, right, scores, BS=left.shape[1], BQ=BQ,
                       stride_q=st.stage_block_stride_q, block_chunk=BLOCK_CHUNK,
                       scan_stride=STAGE_STRIDE, sw_eff=sw_eff, terminate=A.stage_early_terminate)
            if A.head_reduce:
                scores = np.broadcast_to(scores.max(axis=2, keepdims=True), scores.shape).copy()
            if i < len(stages) - 1:
                kk = min(stages[i + 1].stage_k // st.stage_chunk_size, n)
                order = topk_order(scores[..., :n], kk)
            else:
                order = topk_order(scores[..., :n], n)
            left = np.take_along_axis(left, order, -1)
            right = np.take_along_axis(right, order, -1)

        if STAGE_STRIDE > 1:
            left = np.repeat(left, STAGE_STRIDE, 1)[:, -BDST:]
            right = np.repeat(right, STAGE_STRIDE, 1)[:, -BDST:]

        assert A.second_stage_k % chunk == 0
        indices = left[..., : A.second_stage_k // chunk] // chunk * chunk  # :2772-2776

        block_size_q = stages[-1].stage_block_size_q
        bsbq = min(A.block_sparse_block_size_q, block_size_q) if A.block_sparse_block_size_q is not None else None
        sw_bsa = sw_eff + mask_k  # :2901
        block_size_k = chunk

        indices = indices.transpose(0, 2, 1, 3).reshape(B * HEAD, indices.shape[1], -1)  # :2907
        indices = np.sort(indices, axis=-1)
        indices = indices // block_size_k * block_size_k
        uniq = np.roll(indices, 1, axis=-1) != indices  # :2912
        indices = np.where(uniq, indices, INT64_MAX)
        indices = np.sort(indices, axis=-1)
        first_pos = np.repeat(pos[:, ::block_size_q, None], HEAD, axis=0)
        active = indices < (first_pos + block_size_q)
        ks = active.astype(np.int32).sum(-1).astype(np.int64)
        ks_count = ks[..., None]
        ks_start_end = np.zeros((ks.shape[0], ks.shape[1], 2), dtype=np.int32)
        ks_start_end[:, :, 1] = ks

        if bsbq is not None and cdiv(TDST, bsbq) != cdiv(TDST, block_size_q):  # :3036-3051
            assert BQ % bsbq == 0
            rep = BQ // bsbq
            indices = np.repeat(indices, rep, 1)
            ks = np.repeat(ks, rep, 1)
            ks_count = np.repeat(ks_count, rep, 1)
            ks_start_end = np.repeat(ks_start_end, rep, 1)
            block_size_q = bsbq
        X.access = user_access
        if A.mask_only:
            X.scan_backend, X.sa_backend = user_backends
            return None, None
    else:
        sw_bsa = sw_eff + mask_k
        block_size_k = stages[-1].stage_chunk_size
        block_size_q = 64  # HiPAttentionArgs.block_size_q default, untouched on this path (:3056-3066)
        indices = cached.indices.copy()
        ks = cached.ks.copy()
        ks_count = cached.ks_count.copy()
        ks_start_end = cached.ks_start_end.copy()

    block_size_q = min(block_size_q, npow2(TDST))  # :3068
    if sw_bsa == 777:  # :3070-3076
        sw_bsa = A.model_context_length - sink - A.second_stage_k - block_size_q

    decode = (TDST == 1) and (not A.disable_flashdecode)
    X.access = sa_access
    user_cap = X.logit_softcap
    X.logit_softcap = float(A.logit_softcap or 0.0)
    X.non_causal = 0 if A.is_causal else (2 if decode else 1)  # attention only; the scan knows no such switch
    try:
        seams = decode_seams(A.second_stage_k, sink, sw_bsa, block_size_k, indices.shape[-1]) if decode else (0, 0)
        sink_share = decode_sink_share(A.second_stage_k, sink, sw_bsa) if decode else 0
        context = bsa(X, MAX_TSRC, indices, ks_start_end, block_size_q, block_size_k, sw_bsa, sink,
                      share_first_head=decode, seams=seams, sink_share=sink_share)
    finally:
        X.access = user_access
        X.logit_softcap = user_cap
        X.non_causal = 0
        X.scan_backend, X.sa_backend = user_backends
    meta = OMetadata(indices=indices, ks=ks, ks_count=ks_count, ks_start_end=ks_start_end,
                     stage_caches=stage_caches, mask_access=mask_access, sa_access=sa_access)
    return context, meta
