"""``hip_attention_12``: hierarchical mask estimation followed by block-sparse attention.

Host-side driver with the call signature and result layout of the reference operator
``dual_stage_quadratic_hip_attention`` (``src/hip_attn/v1_2/attention_extend.py:1918-3133``).
All arithmetic runs in ``libhipattn.so``; this module only sizes buffers and sequences launches
on the current stream.  No host synchronisation happens inside a call.

Differences in representation (not in results):
  * with head reduction on (the default, env ``HIP_HEAD_REDUCE``), every head of a batch item
    works on the same candidate chunk list, so one ``int32 [B, BDST, 1, chunks]`` list is kept
    instead of the reference's ``int64 [B, BDST, HEAD, chunks]`` left/right pair; chunk lists stay
    ascending, which turns the reference's topk + sort + gather into a compaction;
  * stage caches are materialised in the reference layout only as expanded views.
"""
from __future__ import annotations

import os
from typing import List, Optional

import torch
from torch import Tensor

from . import _native as N
from .metadata import (
    HiPAttentionArgs,
    HiPAttentionCacheAccessStatistics,
    HiPAttentionOutputMetadata,
    HiPAttentionStageInputCache,
    NopStage,
    ScanStage,
)

_BIG = (1 << 62)


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


def _npow2(x: int) -> int:
    return 1 if x <= 1 else 1 << (int(x) - 1).bit_length()


def _head_reduce_enabled() -> bool:
    return os.getenv("HIP_HEAD_REDUCE", "1") == "1"


def _reject_unsupported(args: HiPAttentionArgs):
    if args.using_extend and not args.need_apply_rope:
        raise NotImplementedError("using_extend with keys stored WITH rotation (need_apply_rope=False) is not built; "
                                  "store q and k without RoPE and pass need_apply_rope=True")
    if args.logit_softcap is not None and not (args.logit_softcap > 0):
        raise ValueError("logit_softcap must be positive (or None)")
    if args.sliding_window_indices is not None:
        raise NotImplementedError("sliding_window_indices is a research switch and is not built")
    if args.online_update_cache:
        raise NotImplementedError("online_update_cache (in-kernel cache fill) is not built")
    if (args.low_percent > 0) and (args.low_k_ratio < 1):
        raise NotImplementedError("low_percent / low_k_ratio pruning is dead code in the reference and not built")


_ROPE_TABLES = {}  # (cos ptr, sin ptr, versions, dtype) -> (cos, sin) in the compute dtype; tiny, most recent last
_ROPE_TABLES_PINNED = {}  # entries handed out while a stream was capturing: a graph holds their addresses, never freed


def _capturing(device) -> bool:
    return device.type == "cuda" and torch.cuda.is_current_stream_capturing()


def _cached_for_graphs(cache: dict, pinned: dict, key, build, limit: int, device):
    """Look up or build a small read-only helper tensor that later calls share.

    A HIP graph records the address of every tensor its kernels read, so an entry that was handed out while a stream
    was capturing must live as long as the process: it moves to ``pinned`` and is never evicted.  An entry built
    during a capture belongs to that graph's memory pool and is not kept at all.  Only entries no graph has seen
    take part in the oldest-first eviction.
    """
    hit = pinned.get(key)
    if hit is not None:
        return hit
    capturing = _capturing(device)
    hit = cache.get(key)
    if hit is None:
        hit = build()
        if capturing:
            return hit
        if len(cache) >= limit:
            cache.pop(next(iter(cache)))
        cache[key] = hit
    elif capturing:
        pinned[key] = cache.pop(key)
    return hit


def _rope_tables(args: HiPAttentionArgs, dtype: torch.dtype):
    """RoPE tables as 2-D tensors of the query dtype (the reference casts every loaded entry to it,
    attention_extend.py:395-405).  Converted tables are remembered so a serving loop converts once."""
    cos, sin = args.rope_cos, args.rope_sin
    if cos is None or sin is None:
        raise ValueError("using_extend with need_apply_rope needs rope_cos and rope_sin")
    if cos.ndim == 3:
        cos, sin = cos.view(-1, cos.shape[-1]), sin.view(-1, sin.shape[-1])
    assert cos.ndim == 2 and cos.shape == sin.shape, "rope tables are [positions, head_dim]"
    esz = torch.empty((), dtype=dtype).element_size()

    def usable(t):
        return (t.dtype == dtype and t.stride(1) == 1 and (t.stride(0) * esz) % 16 == 0 and t.data_ptr() % 16 == 0)

    if usable(cos) and usable(sin) and cos.stride(0) == sin.stride(0):
        return cos, sin
    key = (cos.data_ptr(), sin.data_ptr(), cos._version, sin._version, tuple(cos.shape), dtype)
    return _cached_for_graphs(_ROPE_TABLES, _ROPE_TABLES_PINNED, key,
                              lambda: (cos.to(dtype).contiguous(), sin.to(dtype).contiguous()), 8, cos.device)


def _check_operands(q: Tensor, k: Optional[Tensor], v: Optional[Tensor], args: HiPAttentionArgs):
    """Refuse K/V storage the kernels would misread.

    The C side derives the element size of every K / V row from q's dtype alone (fp8 caches aside), and takes every
    pointer for memory of q's device: a key tensor of another dtype would be read at the wrong byte offsets, past
    its end.  The reference's Triton kernels cast on load instead; here the caller converts.
    """
    dev, dt = q.device, q.dtype

    def same(name, t, fp8_ok=False):
        if t is None:
            return
        if t.device != dev:
            raise N.HipAttnError(f"{name} is on {t.device}, q is on {dev}: every operand must live on q's device")
        if t.dtype != dt and not (fp8_ok and dt == torch.bfloat16 and t.dtype in N._FP8_DTYPES):
            what = "q's dtype" + (" (or fp8 e5m2 bytes under a bfloat16 q)" if fp8_ok else "")
            raise N.HipAttnError(f"{name} has dtype {t.dtype} but q has {dt}: {name} must have {what}")

    def on_device(name, t):
        if t is not None and t.device != dev:
            raise N.HipAttnError(f"{name} is on {t.device}, q is on {dev}: every operand must live on q's device")

    same("k", k)
    same("v", v)
    same("args.q_mask", args.q_mask)
    same("args.k_mask", args.k_mask)
    same("args.k_cache", args.k_cache, fp8_ok=True)
    same("args.v_cache", args.v_cache, fp8_ok=True)
    on_device("args.block_table", args.block_table)
    on_device("args.cache_seq_lens", args.cache_seq_lens)
    on_device("args.position_ids", args.position_ids)
    if args.using_extend and args.need_apply_rope:
        on_device("args.rope_cos", args.rope_cos)
        on_device("args.rope_sin", args.rope_sin)


def _kv_struct(args: HiPAttentionArgs, k: Optional[Tensor], v: Optional[Tensor], max_tsrc: int,
               masking: bool = False, stats: Optional[HiPAttentionCacheAccessStatistics] = None):
    """Returns (struct, keepalive) describing where K/V rows live.

    ``masking`` picks the key-only cache of an offload cache; ``stats`` attaches access / miss flags.
    """
    if k is not None:
        kk = k if k.stride(-1) == 1 else k.contiguous()
        vv = v if v.stride(-1) == 1 else v.contiguous()
        st, keep = N.make_kv_dense(kk, vv), (kk, vv)
    else:
        bt = args.block_table
        sl = args.cache_seq_lens
        assert bt is not None and bt.ndim == 2, "paged mode needs block_table [B, pages]"
        assert sl is not None and sl.ndim == 1, "paged mode needs cache_seq_lens [B]"
        if bt.dtype not in (torch.int32, torch.int64):
            bt = bt.to(torch.int64)
        if bt.stride(1) != 1:
            bt = bt.contiguous()
        if sl.dtype not in (torch.int32, torch.int64):
            sl = sl.to(torch.int64)
        if sl.stride(0) != 1:
            sl = sl.contiguous()
        if args.k_cache is None and args.offload_cache is not None:
            st, keep = args.offload_cache.kv_struct(bt, sl, max_tsrc, masking), (bt, sl)
        else:
            assert args.k_cache is not None and args.v_cache is not None, "paged mode needs k_cache and v_cache"
            assert args.k_cache.ndim == 4 and args.v_cache.ndim == 4
            st, keep = N.make_kv_paged(args.k_cache, args.v_cache, bt, sl, max_tsrc), (bt, sl)
    if stats is not None and stats.flags()[0] is not None:
        access, miss = stats.flags()
        st = N.set_flags(st, access, miss if st.cache else None)
    return st, keep


_ZERO_FLAG: dict = {}


def _zero_flag(device) -> Tensor:
    """One zero byte per device, the target of the read-only miss flags of calls without an offload cache."""
    key = (device.type, device.index)
    zero = _ZERO_FLAG.get(key)
    if zero is None:
        zero = torch.zeros((1, 1, 1), dtype=torch.uint8, device=device)
        if not (device.type == "cuda" and torch.cuda.is_current_stream_capturing()):
            _ZERO_FLAG[key] = zero  # an allocation made during graph capture belongs to that graph: not kept
    return zero


def _new_statistics(args: HiPAttentionArgs, B: int, head_kv: int, pages: int, device, count: int = 1):
    """Zeroed ``[B, HEAD_KV, pages]`` access and miss flags (attention_extend.py:1994-2006), one byte per page as the
    kernels keep them (``HiPAttentionCacheAccessStatistics`` widens them to int32 when they are read).  Without an
    offload cache nothing can miss: the miss flags are then a read-only view of one zero kept per device, which
    saves clearing ``B * HEAD_KV * pages`` words per call.  ``count`` > 1 returns that many sets whose access flags
    are cleared by one launch (a mask refresh needs one for the scan and one for the attention)."""
    if count > 1:
        if not args.require_cache_statistics or args.offload_cache is not None:
            return [_new_statistics(args, B, head_kv, pages, device) for _ in range(count)]
        both = torch.zeros((count, B, head_kv, pages), dtype=torch.uint8, device=device)
        miss = _zero_flag(device).expand(B, head_kv, pages)
        return [HiPAttentionCacheAccessStatistics(both[i], miss) for i in range(count)]
    if not args.require_cache_statistics:
        return HiPAttentionCacheAccessStatistics(None, None)
    access = torch.zeros((B, head_kv, pages), dtype=torch.uint8, device=device)
    if args.offload_cache is not None:
        return HiPAttentionCacheAccessStatistics(access, torch.zeros_like(access))
    return HiPAttentionCacheAccessStatistics(access, _zero_flag(device).expand(B, head_kv, pages))


def _mask_kv(args: HiPAttentionArgs, k_mask: Optional[Tensor], max_tsrc: int, q: Tensor, programs_rows: int,
             chunk_count: int, device, stats=None, rope_tabs=None, backends=(), first_stage_list=None):
    """KV descriptions for the scan kernels: ``(plain, prescaled or None, keepalive, khat, k_side_delta, first or None)``.

    ``prescaled`` describes keys scaled (and, with RoPE on load under the relative / infllm rules, rotated) once for
    the whole tensor; it is built when the scan will sample far more rows than the key tensor holds.  ``backends``:
    the rotation rules of the stages that will run; ``first_stage_list`` = ``(sink, chunk size)`` when the first of
    them scans the initial list of a dense key tensor under the streaming rule: there a key's rotated position is the
    place of its chunk, whatever the query, and ``first`` describes a copy rotated that way.
    """
    stage0 = args.stages[0]
    iters = max(1, int(stage0.stage_chunk_size).bit_length())
    sampled_rows = 2 * iters * programs_rows * chunk_count  # stage 0 alone
    plain, keep = _kv_struct(args, k_mask, k_mask, max_tsrc, masking=True, stats=stats)
    if q.dtype == torch.bfloat16 and args.offload_cache is None:
        src = k_mask if k_mask is not None else args.k_cache
        if src is not None and src.dtype == torch.bfloat16 and src.ndim == 4 and src.stride(-1) == 1:
            rows_total = src.shape[0] * src.shape[1] * src.shape[2]
            force = os.getenv("HIP_ATTN_PRESCALE_K", "")  # "0" / "1" override the heuristic (testing)
            given = args.k_prescaled if rope_tabs is None else None  # a copy the caller keeps up to date
            if given is not None:
                if given.shape != src.shape or given.dtype != torch.bfloat16 or given.stride(-1) != 1 or given.device != src.device:
                    raise ValueError("k_prescaled must be a bf16 device tensor with the shape of the key storage "
                                     f"({tuple(src.shape)}), got {tuple(given.shape)} {given.dtype}")
            if given is not None or force == "1" or (force != "0" and sampled_rows >= 4 * rows_total):
                delta = 0
                first = None
                if rope_tabs is not None and first_stage_list is not None and k_mask is not None:
                    kfirst = N.prescale_k_rope_chunks(src, rope_tabs[0], rope_tabs[1], first_stage_list[0],
                                                      first_stage_list[1], device)
                    st0, keep0 = _kv_struct(args, kfirst, kfirst, max_tsrc, masking=True, stats=stats)
                    first = (st0, (keep0, kfirst))
                if rope_tabs is not None and not any(b in ("relative", "infllm") for b in backends):
                    return plain, None, keep, None, 0, first  # no stage reads keys rotated to a fixed position
                if given is not None:
                    khat = khat0 = given
                elif rope_tabs is None:
                    # the copy is laid out with the kv head outermost: the rows a search samples then lie within a
                    # few KB instead of spreading over HKV times as much (cfg-2-like prefill: the 256- and 32-token
                    # stages 4.13 -> 3.77 and 5.19 -> 4.82 ms, the same from a page-16 cache)
                    khat = khat0 = N.prescale_k(src, device, head_major=True)
                else:
                    # rotated to position 0 (left samples, and everything under infllm) and 1 (right samples, relative)
                    khat = N.prescale_k_rope(src, rope_tabs[0], rope_tabs[1], (0, 1), device)
                    khat0, delta = khat[0], khat.stride(0)
                if k_mask is not None:
                    st, keep2 = _kv_struct(args, khat0, khat0, max_tsrc, masking=True, stats=stats)
                else:
                    a2 = args.clone()
                    a2.k_cache, a2.v_cache = khat0, khat0
                    st, keep2 = _kv_struct(a2, None, None, max_tsrc, masking=True, stats=stats)
                return plain, st, (keep, keep2, khat), (khat if rope_tabs is None else None), delta, first
    return plain, None, keep, None, 0, None


def _spans_32_gib(t: Optional[Tensor]) -> bool:
    """Whether rows of ``t`` can lie 32 GiB or more beyond its first element (see ``hipattn_mask_stage``)."""
    if t is None:
        return False
    span = sum((n - 1) * abs(s) for n, s in zip(t.shape, t.stride())) + 1
    return span * t.element_size() >= (1 << 35)


_INITIAL_CHUNKS = {}  # read-only stage-0 chunk lists, keyed by their shape parameters
_INITIAL_CHUNKS_PINNED = {}  # those a captured graph reads: kept for the life of the process


def _initial_chunks(chunk_count: int, chunk_size: int, sink: int, B: int, bs: int, hg: int, device) -> Tensor:
    """``int32 [B, bs, hg, chunk_count]``: chunk c starts at ``sink + c * chunk_size`` (attention_extend.py:2020-2035).
    Nothing writes to a chunk list, so the tensor is built once per shape and shared by later calls (a decode loop
    would otherwise pay four small launches per mask refresh for it)."""
    key = (chunk_count, chunk_size, sink, B, bs, hg, str(device))

    def build():
        row = torch.arange(0, chunk_count, device=device, dtype=torch.int32) * chunk_size + sink
        return row[None, None, None, :].expand(B, bs, hg, chunk_count).contiguous()

    return _cached_for_graphs(_INITIAL_CHUNKS, _INITIAL_CHUNKS_PINNED, key, build, 16, device)


_RESET_SCORE: dict = {}


def _reset_scores(device, shape) -> Tensor:
    """The scores a stage starts from (-32000 everywhere) as a view of one element kept per device."""
    key = (device.type, device.index)
    one = _RESET_SCORE.get(key)
    if one is None:
        one = torch.full((1, 1, 1, 1), -32000.0, dtype=torch.float32, device=device)
        if not (device.type == "cuda" and torch.cuda.is_current_stream_capturing()):
            _RESET_SCORE[key] = one  # an allocation made during graph capture belongs to that graph: not kept
    return one.expand(*shape)


def _stage_cache_views(chunk_left: Tensor, HEAD: int, chunk: int, left64: Optional[Tensor] = None,
                       right64: Optional[Tensor] = None) -> HiPAttentionStageInputCache:
    """Reference-layout view of a stage's inputs: int64 left/right and the reset scores.  ``left64 / right64``:
    the same list already written as int64 by the selection kernel."""
    B, BS, hg, n = chunk_left.shape
    left = left64 if left64 is not None else chunk_left.to(torch.int64)
    right = right64 if right64 is not None else left + chunk
    if hg == 1:
        left = left.expand(B, BS, HEAD, n)
        right = right.expand(B, BS, HEAD, n)
    return HiPAttentionStageInputCache(indices_left=left, indices_right=right,
                                       out_scores=_reset_scores(chunk_left.device, (B, BS, HEAD, n)))


def _chunk_list_from_cache(cache: HiPAttentionStageInputCache, hg: int) -> Tensor:
    left = cache.indices_left
    if hg == 1:
        left = left[:, :, :1, :]
    return left.to(torch.int32).contiguous()


@torch.no_grad()
def dual_stage_quadratic_hip_attention(
    q: Tensor,
    k: Optional[Tensor],
    v: Optional[Tensor],
    args: HiPAttentionArgs,
    cached_metadata: Optional[HiPAttentionOutputMetadata] = None,
):
    """HiP attention: returns ``(context, HiPAttentionOutputMetadata)``.

    ``q [B, TDST, HEAD, HID]``; ``k, v [B, TSRC, HEAD_KV, HID]`` or ``None`` with a paged cache in
    ``args``.  ``q`` is used as given: no softmax scale is applied (callers pre-scale).
    Passing ``cached_metadata`` with ``indices`` skips mask estimation; with only
    ``stage_caches`` it resumes estimation from the last cached stage.  Returns ``(None, None)``
    when ``args.mask_only``.
    """
    N.lib()
    if not q.is_cuda:
        raise N.HipAttnError("hip_attention_12 runs on the GPU only: q must be a device tensor")
    _reject_unsupported(args)
    _check_operands(q, k, v, args)
    device = q.device

    q_bsa = q
    if args.q_mask is not None:
        q = args.q_mask
    k_mask = k if args.k_mask is None else args.k_mask

    BSZ, TDST, HEAD, HID = q.shape
    if k is not None:
        _, TSRC, HEAD_KV, _ = k.shape
        assert v is not None and v.shape == k.shape
        MAX_TSRC = TSRC
    else:
        MAX_TSRC = args.extend_context_length
        TSRC = MAX_TSRC
        HEAD_KV = args.k_cache.shape[-2] if args.k_cache is not None else args.offload_cache.head_kv

    stages = args.stages
    assert len(stages) > 0
    STAGE_STRIDE = stages[0].stage_stride
    BLOCK_SIZE_Q = stages[0].stage_block_size_q
    BDST = _cdiv(TDST, BLOCK_SIZE_Q)
    BDST_SCAN = _cdiv(BDST, STAGE_STRIDE)
    BLOCK_CHUNK = args.block_size_k
    chunk_size = stages[0].stage_chunk_size
    chunk_count = _cdiv(max(0, MAX_TSRC - args.sink_token_size - args.sliding_window_size), chunk_size)

    args = args.clone()
    args.mask_k = stages[0].stage_chunk_size
    args.sliding_window_size = max(0, args.sliding_window_size - args.mask_k)
    sw_eff = args.sliding_window_size
    sink = args.sink_token_size

    if args.position_ids is not None:
        position_ids = args.position_ids
        if position_ids.dtype != torch.int64:
            position_ids = position_ids.to(torch.int64)
    else:
        position_ids = (torch.arange(0, TDST, device=device, dtype=torch.int64) + (TSRC - TDST))[None, :].expand(BSZ, TDST)
    assert position_ids.shape == (BSZ, TDST), position_ids.shape

    stage_caches: Optional[List[HiPAttentionStageInputCache]] = (
        [] if (cached_metadata is None) or (cached_metadata.stage_caches is None) else cached_metadata.stage_caches
    )
    if not args.require_stage_caches:
        stage_caches = None

    args.update_flags()
    MAX_PAGE = args.paged_cache_page_count if (k is None and args.using_paged_cache) else MAX_TSRC
    mask_stats = None
    will_scan = (cached_metadata is None) or (cached_metadata.indices is None)
    if will_scan:
        sa_stats, mask_stats_new = _new_statistics(args, BSZ, HEAD_KV, MAX_PAGE, device, count=2)
    else:
        sa_stats = _new_statistics(args, BSZ, HEAD_KV, MAX_PAGE, device)

    qq = q if q.stride(-1) == 1 else q.contiguous()
    rope_tabs = _rope_tables(args, q.dtype) if (args.using_extend and args.need_apply_rope) else None
    hg = 1 if _head_reduce_enabled() else HEAD
    khat = None

    if (cached_metadata is None) or (cached_metadata.indices is None):
        fresh = (cached_metadata is None) or (cached_metadata.stage_caches is None) or (stage_caches is None)
        if (not fresh) and stage_caches[-1].indices_left is None:
            # only the empty stage-0 entry is cached: nothing to resume from
            assert len(stage_caches) == 1
            fresh = True
        if fresh:
            chunk_left = _initial_chunks(chunk_count, chunk_size, sink, BSZ, BDST_SCAN, hg, device)
            right_clamp = MAX_TSRC - sw_eff
        else:
            assert len(stage_caches) <= len(stages)
            chunk_left = _chunk_list_from_cache(stage_caches[-1], hg)
            right_clamp = _BIG

        # Keys are scaled by c_k and re-rounded every time they are sampled.  When the scan will sample
        # far more rows than the key tensor holds (prefill), scale the whole tensor once instead.
        mask_stats = mask_stats_new
        n_cached = len(stage_caches) if stage_caches is not None else 0
        stage_backends = [(st.stage_extend_backend or args.scan_extend_backend) if isinstance(st, ScanStage) else None
                          for i, st in enumerate(stages) if i >= n_cached - 1]
        first_list = None
        if fresh and rope_tabs is not None and stage_backends and stage_backends[0] == "streaming":
            first_list = (sink, chunk_size)
        mask_kv, mask_kv_pre, keep_mask_kv, khat, k_side_delta, mask_kv_first = _mask_kv(
            args, k_mask, MAX_TSRC, q, BSZ * HEAD * BDST_SCAN, chunk_count, device, stats=mask_stats, rope_tabs=rope_tabs,
            backends=stage_backends, first_stage_list=first_list)

        scores = None
        left_out = None
        prev_n = None
        left64 = right64 = None
        query_rows = {}
        for i_stage, stage in enumerate(stages):
            prefilled_scores = None
            if i_stage < n_cached - 1:
                continue
            elif i_stage == n_cached - 1:
                # The reference enters a restarted stage with stage 0's query block size and stage stride (:1960-1965;
                # they are switched, :2092-2124, only on the way into a stage that is not restarted), and its restart
                # test keeps them equal over all stages.  Where they differ its result is not the fresh run's; that
                # state is refused rather than guessed at.
                if i_stage > 0 and ((stage.stage_block_size_q, stage.stage_stride)
                                    != (stages[0].stage_block_size_q, stages[0].stage_stride)):
                    raise NotImplementedError("restart from cached stage inputs at a stage whose stage_block_size_q or "
                                              "stage_stride differs from the first stage's is not built")
            elif i_stage > 0:
                # truncate / realign / sort / re-tile / split (:2072-2165) folded into one selection pass
                assert isinstance(stage, (ScanStage, NopStage)), f"stage type {type(stage).__name__} is not executable"
                if not stage.require_realign_index or not stage.require_reset_score:
                    raise NotImplementedError("stages with require_realign_index/require_reset_score off are not built")
                assert (stage.stage_k % chunk_size) == 0, f"{stage.stage_k} % {chunk_size}"
                keep = min(stage.stage_k // chunk_size, prev_n)
                row_rep = 1
                bs_in = chunk_left.shape[1]
                if BLOCK_SIZE_Q != stage.stage_block_size_q:
                    assert stage.stage_block_size_q > 0 and BLOCK_SIZE_Q > stage.stage_block_size_q
                    assert (BLOCK_SIZE_Q % stage.stage_block_size_q) == 0
                    row_rep *= BLOCK_SIZE_Q // stage.stage_block_size_q
                    BLOCK_SIZE_Q = stage.stage_block_size_q
                    BDST = _cdiv(TDST, BLOCK_SIZE_Q)
                    BDST_SCAN = _cdiv(BDST, STAGE_STRIDE)
                shrunk = row_rep != 1
                if STAGE_STRIDE != stage.stage_stride:
                    assert stage.stage_stride < STAGE_STRIDE and STAGE_STRIDE > 0
                    if stage.stage_stride != 1:
                        raise NotImplementedError("stage_stride may only drop to 1 between stages")
                    # rows repeated for the smaller block and again for the smaller stride, each time keeping the
                    # last BDST rows (:2096-2124): counted from the last row, output row e reads input row
                    # e // (both factors), whether or not the first cut removed anything
                    row_rep *= STAGE_STRIDE // stage.stage_stride
                    STAGE_STRIDE = stage.stage_stride
                    BDST_SCAN = _cdiv(BDST, STAGE_STRIDE)
                if shrunk and STAGE_STRIDE != 1:
                    raise NotImplementedError("a stage may shrink its query block only when its stage_stride is 1")
                bs_out = BDST_SCAN if row_rep == 1 else min(BDST, row_rep * bs_in)
                assert (chunk_size % stage.stage_chunk_size) == 0
                splits = chunk_size // stage.stage_chunk_size
                next_left = torch.empty((BSZ, bs_out, hg, keep * splits), dtype=torch.int32, device=device)
                left64 = right64 = None
                if keep > 0:
                    if (stage_caches is not None) and (i_stage >= len(stage_caches)):
                        # the list is also handed out as this stage's cached inputs: written once, in both widths
                        left64 = torch.empty(next_left.shape, dtype=torch.int64, device=device)
                        right64 = torch.empty(next_left.shape, dtype=torch.int64, device=device)
                    if hg == 1 and isinstance(stage, ScanStage):
                        # the head-reduced scores of the stage that follows have the shape of its chunk list: the
                        # selection pass starts them at -inf, which saves the scan a launch of its own for that
                        prefilled_scores = torch.empty(next_left.shape, dtype=torch.float32, device=device)
                    N.select_stage(scores, chunk_left, BSZ, bs_in, bs_out, row_rep, scores.shape[2], hg, prev_n, keep,
                                   chunk_size, splits, next_left, device, left64=left64, right64=right64,
                                   next_scores=prefilled_scores)
                chunk_left = next_left
                right_clamp = _BIG
            else:
                assert stage.stage_k is None, "first stage always quadratic"
                assert isinstance(stage, ScanStage), f"first stage always scan {stage}"
                STAGE_STRIDE = stage.stage_stride

            if (stage_caches is not None) and (i_stage >= len(stage_caches)):
                if i_stage == 0:
                    stage_caches.append(HiPAttentionStageInputCache(None, None, None))
                else:
                    stage_caches.append(_stage_cache_views(chunk_left, HEAD, stage.stage_chunk_size, left64, right64))

            chunk_size = stage.stage_chunk_size
            chunk_count = chunk_left.shape[-1]
            BLOCK_CHUNK = max(16, _npow2(min(chunk_count, BLOCK_CHUNK)))
            if BLOCK_CHUNK > 64:
                raise NotImplementedError(f"block_size_k (chunks per scan program) above 64 is not built: {BLOCK_CHUNK}")
            bs = chunk_left.shape[1]
            last = i_stage == len(stages) - 1

            if isinstance(stage, ScanStage):
                # one shared chunk list: the scan kernels fold the maximum over heads into their score store
                reduce = hg == 1
                if reduce and prefilled_scores is not None:
                    assert prefilled_scores.shape == (BSZ, bs, 1, chunk_count)
                    scores, reduce = prefilled_scores, 2  # already at -inf
                elif reduce:
                    scores = torch.empty((BSZ, bs, 1, chunk_count), dtype=torch.float32, device=device)  # mask_stage fills it
                else:
                    scores = torch.empty((BSZ, bs, HEAD, chunk_count), dtype=torch.float32, device=device)
                left_out = torch.empty((BSZ, bs, HEAD, chunk_count), dtype=torch.int32, device=device) if last else None
                if chunk_count > 0:
                    rope = None
                    use_pre = mask_kv_pre is not None
                    kv_pre = mask_kv_pre
                    if rope_tabs is not None:  # :2200-2204
                        backend = stage.stage_extend_backend or args.scan_extend_backend
                        use_pre = use_pre and backend in ("relative", "infllm")  # key positions fixed per sample side
                        if i_stage == 0 and fresh and mask_kv_first is not None and backend == "streaming":
                            use_pre, kv_pre = True, mask_kv_first[0]  # keys rotated to the place of their chunk
                        rope = N.make_rope(*rope_tabs, backend, k_side_delta if (use_pre and backend == "relative") else 0,
                                           args.model_context_length)
                    qs = N.make_q(qq, position_ids, rope)
                    # Stages that differ only in their chunks share their averaged, scaled query rows.  Without
                    # rotation only where a row is a mean of several query rows: otherwise a kernel may scale its
                    # rows itself and leave the workspace unwritten.  Rotated rows are always prepared into the
                    # workspace, and only the streaming rule places a query by the stage's chunk count
                    # (attention_extend.py:632-647).
                    if rope is None:
                        shared = stage.stage_block_stride_q > 1 and TDST > 1
                    else:
                        shared = backend != "streaming"
                    ws_key = ((bs, BLOCK_SIZE_Q, stage.stage_block_stride_q, STAGE_STRIDE, backend if rope is not None else None)
                              if shared else None)
                    ws = N.mask_stage(qs, kv_pre if use_pre else mask_kv, chunk_left, hg, chunk_count, chunk_size,
                                      right_clamp, bs, BLOCK_SIZE_Q, stage.stage_block_stride_q, BLOCK_CHUNK, STAGE_STRIDE,
                                      sw_eff, args.stage_early_terminate, scores, left_out, device, k_prescaled=use_pre,
                                      reduce_heads=reduce, workspace=query_rows.get(ws_key),
                                      near_pool=not _spans_32_gib(khat if use_pre else (k_mask if k_mask is not None else args.k_cache)))
                    if ws_key is not None and ws is not None:
                        query_rows[ws_key] = ws
            elif isinstance(stage, NopStage):
                scores = torch.full((BSZ, bs, 1 if hg == 1 else HEAD, chunk_count), -32000.0, dtype=torch.float32,
                                    device=device)
                left_out = chunk_left.expand(BSZ, bs, HEAD, chunk_count).contiguous() if last else None
            else:
                raise NotImplementedError(f"stage type {type(stage).__name__} raises in the reference as well")
            if not stage.require_post_sort:
                raise NotImplementedError("stages without require_post_sort are not built")
            prev_n = chunk_count

        assert (args.second_stage_k % chunk_size) == 0
        K = args.second_stage_k // chunk_size
        BK = min(K, chunk_count)
        indices = torch.empty((BSZ * HEAD, BDST, max(BK, 1)), dtype=torch.int64, device=device)
        ks = torch.empty((BSZ * HEAD, BDST), dtype=torch.int64, device=device)
        ks_start_end = torch.empty((BSZ * HEAD, BDST, 2), dtype=torch.int32, device=device)
        if BK > 0:
            N.finalize_indices(scores, left_out, position_ids, BSZ, chunk_left.shape[1], BDST, STAGE_STRIDE, HEAD,
                               scores.shape[2], hg, chunk_count, K, chunk_size, stages[-1].stage_block_size_q, indices, ks, ks_start_end,
                               device)
        else:
            indices = indices[:, :, :0]
            ks.zero_()
            ks_start_end.zero_()
        ks_count = ks.unsqueeze(-1)

        args = args.clone()
        args.block_size_q = stages[-1].stage_block_size_q
        block_sparse_block_size_q = (
            min(args.block_sparse_block_size_q, args.block_size_q) if args.block_sparse_block_size_q is not None else None
        )
        args.sliding_window_size += args.mask_k
        args.block_size_k = chunk_size
        args.mask_k = args.second_stage_k

        if (block_sparse_block_size_q is not None) and (
            _cdiv(TDST, block_sparse_block_size_q) != _cdiv(TDST, args.block_size_q)
        ):
            assert (BLOCK_SIZE_Q % block_sparse_block_size_q) == 0
            rep = BLOCK_SIZE_Q // block_sparse_block_size_q
            indices = indices.repeat_interleave(rep, 1)
            ks = ks.repeat_interleave(rep, 1)
            ks_count = ks_count.repeat_interleave(rep, 1)
            ks_start_end = ks_start_end.repeat_interleave(rep, 1)
            args.block_size_q = block_sparse_block_size_q

        if args.mask_only:
            return None, None
        fresh_mask = True
        rows_shared = hg == 1  # every head of a batch item carries the same index row
    else:
        args = args.clone()
        args.sliding_window_size += args.mask_k
        args.block_size_k = stages[-1].stage_chunk_size
        args.mask_k = args.second_stage_k
        # The reference clones these four tensors (:3063-3066).  Nothing here writes to them, so the returned
        # metadata shares them with the cached one: four copy kernels less on every cached decode step.
        indices = cached_metadata.indices
        ks = cached_metadata.ks
        ks_count = cached_metadata.ks_count
        ks_start_end = cached_metadata.ks_start_end
        fresh_mask = False
        rows_shared = bool(getattr(cached_metadata, "_rows_shared", False))

    args.block_size_q = min(args.block_size_q, _npow2(TDST))
    if args.sliding_window_size == 777:
        args.sliding_window_size = (
            args.model_context_length - args.sink_token_size - args.second_stage_k - args.block_size_q
        )

    use_decode = (
        (TDST == 1) and (os.environ.get("HIP_DISABLE_FLASHDECODE", "0") != "1") and (not args.disable_flashdecode)
    )
    seq_pos = position_ids[:, -q_bsa.shape[1]:]
    context = block_sparse_attention(
        q_bsa, k, v, seq_pos, indices, ks_start_end, args, MAX_TSRC, decode=use_decode, rows_shared=rows_shared,
        khat=khat if (args.k_mask is None) else None, stats=sa_stats, rope_tables=rope_tabs, operands_checked=True,
    )

    metadata = HiPAttentionOutputMetadata(
        indices=indices,
        ks=ks,
        ks_count=ks_count,
        ks_start_end=ks_start_end,
        mask_cache_statistics=(mask_stats if fresh_mask else None),
        sa_cache_statistics=sa_stats,
        stage_caches=stage_caches,
    )
    # private hint for later calls that reuse this metadata: index rows are identical across heads,
    # so the tile kernel may serve a whole GQA group from one gathered K/V tile
    metadata._rows_shared = rows_shared
    return context, metadata


@torch.no_grad()
def _decode_seams_overlap(args: HiPAttentionArgs, BK: int) -> bool:
    """Whether the reference's decode programs visit some selected block twice (attention_decode_bsa.py:1070-1076,
    1391-1393, 239-247): their share of the index row is not a whole number of their tiles."""
    if args.second_stage_k <= 0 or BK <= 0:
        return False
    chunk = -(-(args.second_stage_k + args.sink_token_size + args.sliding_window_size) // 8)
    programs = min(12, -(-args.second_stage_k // chunk))
    tile = max(1, 16 // args.block_size_k)
    return -(-BK // programs) % tile != 0


def block_sparse_attention(q: Tensor, k: Optional[Tensor], v: Optional[Tensor], position_ids: Tensor, indices: Tensor,
                           ks_start_end: Tensor, args: HiPAttentionArgs, max_tsrc: int, decode: bool = False,
                           impl: int = 0, rows_shared: bool = False, khat: Optional[Tensor] = None,
                           stats: Optional[HiPAttentionCacheAccessStatistics] = None,
                           rope_tables=None, operands_checked: bool = False) -> Tensor:
    """Sparse attention over (selected blocks, sink, sliding window) given the metadata tensors.

    ``position_ids`` are 0-based (the reference passes ``seq_lens = position_ids + 1``,
    attention_extend.py:3092).  ``args.block_size_q / block_size_k / sliding_window_size`` must
    already hold the values the operator derives for this step.  ``decode`` selects the split-KV
    path, which, like the reference's decode kernel, lets every head of a GQA group read the
    index row of the group's first head, and which weights the selected blocks as the reference's decode
    programs do (a block at the seam of two programs' shares of the index row counts twice when
    ``ceil(BK / programs)`` is not a multiple of ``16 // block_size_k``, attention_decode_bsa.py:239-247,1070-1076).
    ``rows_shared`` promises that all heads of a GQA group hold
    identical index rows (true for masks estimated with head reduction), which lets one gathered
    K/V tile serve the whole group.  ``khat`` is an optional ``bf16(k * c_k)`` tensor with the shape and
    strides of the key storage (dense ``k`` or ``args.k_cache``).  ``rope_tables`` = ``(cos, sin)`` in q's dtype
    turns on rotation on load under ``args.sa_extend_backend``.
    """
    device = q.device
    if not q.is_cuda:
        raise N.HipAttnError("block_sparse_attention runs on the GPU only: q must be a device tensor")
    if not operands_checked:  # the operator above has looked at the same tensors already
        _check_operands(q, k, v, args)
    qq = q if q.stride(-1) == 1 else q.contiguous()
    kvs, keep = _kv_struct(args, k, v, max_tsrc, masking=False, stats=stats)
    if position_ids.dtype != torch.int64:
        position_ids = position_ids.to(torch.int64)
    rope = (N.make_rope(*rope_tables, args.sa_extend_backend, 0, args.model_context_length, attention=True)
            if rope_tables is not None else None)
    non_causal = not args.is_causal
    if non_causal and not decode:
        # the reference's query-block kernel takes MAX_TSRC for every row's position when the mask is not causal
        # (attention_extend_bsa.py:743-752); its decode kernel keeps the true ones
        position_ids = torch.full_like(position_ids, max_tsrc - 1)
    qs = N.make_q(qq, position_ids, rope, args.logit_softcap, non_causal)
    if rope is not None or args.logit_softcap is not None:
        khat = None
    if not indices.is_contiguous():
        indices = indices.contiguous()
    if ks_start_end.dtype != torch.int32:  # metadata kept in a HiPMetadataCachePool comes back as int64
        ks_start_end = ks_start_end.to(torch.int32)
    if indices.dtype != torch.int64:
        indices = indices.to(torch.int64)
    if not ks_start_end.is_contiguous():
        ks_start_end = ks_start_end.contiguous()
    BK = indices.shape[-1]
    out = torch.empty(q.shape, dtype=q.dtype, device=device)
    if BK == 0:
        indices = torch.zeros((indices.shape[0], indices.shape[1], 1), dtype=torch.int64, device=device)
    if decode:
        try:
            N.bsa_decode(qs, kvs, indices, ks_start_end, BK, args.block_size_k, args.sliding_window_size,
                         args.sink_token_size, out, device, second_stage_k=args.second_stage_k)
            return out
        except N.HipAttnError as e:
            # the query-block kernel below attends every selected block once: it can stand in only where the
            # reference's decode programs do so too
            if "is not built" not in str(e) or _decode_seams_overlap(args, BK):
                raise
    ksrc = k if k is not None else args.k_cache
    if khat is not None and (ksrc is None or khat.shape != ksrc.shape or kvs.cache):
        khat = None
    if khat is not None and impl != 1:
        # The pre-scaled copy has its own layout (kv head outermost), so the tile kernel gets a description whose K
        # side carries the copy's strides.  Only the tile kernel takes pre-scaled keys: where it does not apply, the
        # call is repeated on the tensors as they are.
        kvs_hat = type(kvs).from_buffer_copy(kvs)
        kvs_hat.k_stride_b, kvs_hat.k_stride_t, kvs_hat.k_stride_h = khat.stride(0), khat.stride(1), khat.stride(2)
        try:
            N.bsa_prefill(qs, kvs_hat, indices, ks_start_end, BK, args.block_size_q, args.block_size_k,
                          args.sliding_window_size, args.sink_token_size, decode or rows_shared, 2, out, device,
                          k_prescaled=khat)
            return out
        except N.HipAttnError as e:
            if "does not cover" not in str(e) or impl == 2:
                raise
    N.bsa_prefill(qs, kvs, indices, ks_start_end, BK, args.block_size_q, args.block_size_k,
                  args.sliding_window_size, args.sink_token_size, decode or rows_shared, impl, out, device)
    del keep
    return out
