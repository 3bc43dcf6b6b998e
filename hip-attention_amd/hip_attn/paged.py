"""``forward_paged_hip``: the entry point a paged-KV serving backend calls per attention layer.

Mirrors ``src/hip_attn/v1_2/paged_hip.py:35-62`` (public wrapper) and ``:327-499`` (argument
assembly): the token-granular KV pool is viewed as a page-size-1 cache, the block table is
``req_to_tokens[req_pool_indices]``, the per-layer preset comes from ``HiPAttentionConfig``, queries
are pre-scaled by ``sm_scale`` (the operator itself applies no softmax scale), and a long prefill is
split so that its last 64 queries attend densely.
"""
from __future__ import annotations

import os
from typing import Optional, Tuple

import torch

from .config import HiPAttentionConfig
from .metadata import HiPAttentionArgs, HiPAttentionOutputMetadata
from .operator import dual_stage_quadratic_hip_attention

from .memory_pool import cuda_graph_capture_configs  # noqa: F401  (paged_hip.py:27-32 keeps it here)

_LAST_DENSE = 64  # trailing prefill queries served with an (effectively) dense window, paged_hip.py:462


def _forward_paged_hip(
    query: torch.Tensor,
    sm_scale: float,
    batch_size: int,
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    offload_cache,
    positions: torch.Tensor,
    seq_lens: torch.Tensor,
    req_to_tokens: torch.Tensor,
    req_pool_indices: torch.Tensor,
    rope_cos: Optional[torch.Tensor],
    rope_sin: Optional[torch.Tensor],
    layer_id: int,
    logit_cap: float,
    orig_context_len: int,
    max_context_len: int,
    is_prefill: bool,
    hip_config: HiPAttentionConfig,
    cached_metadata: Optional[HiPAttentionOutputMetadata] = None,
    k: Optional[torch.Tensor] = None,
    v: Optional[torch.Tensor] = None,
    online_update_cache: bool = False,
    is_decode: bool = False,
    query_for_mask: Optional[torch.Tensor] = None,
    diag_sliding_window_indices: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, HiPAttentionOutputMetadata]:
    """``query [N, H, D]`` -> ``(context [N, H, D], metadata)`` for ``batch_size`` requests.

    ``k_cache / v_cache [tokens, H_kv, D]`` is the serving framework's token pool;
    ``req_to_tokens [requests, max_ctx]`` maps a request's position to its pool slot.
    """
    if diag_sliding_window_indices is not None:
        raise NotImplementedError("diag_sliding_window_indices is a research switch and is not built")
    N, num_heads, hidden = query.shape
    dst_seq_len = N // batch_size

    is_dense = layer_id in hip_config.dense_layers
    presets = hip_config.layers if is_decode else hip_config.prefill_layers
    if is_decode:
        assert dst_seq_len == 1
    layer_config = presets[0 if is_dense else 1] if len(presets) == 2 else presets[layer_id]

    query = query.view(batch_size, dst_seq_len, num_heads, hidden)
    if query_for_mask is not None:
        query_for_mask = query_for_mask.view(batch_size, -1, num_heads, hidden)

    if k_cache is not None:
        n_page, heads_kv, hidden_kv = k_cache.shape
        assert v_cache.shape == k_cache.shape and hidden_kv == hidden
        k_cache = k_cache.view(n_page, 1, heads_kv, hidden)
        v_cache = v_cache.view(n_page, 1, heads_kv, hidden)

    block_table = req_to_tokens.index_select(dim=0, index=req_pool_indices)
    assert block_table.shape[0] == batch_size

    if k_cache is not None:
        hidden_size = k_cache.shape[-1]
    elif k is not None:
        hidden_size = k.shape[-1]
    elif offload_cache is not None:
        hidden_size = offload_cache.head_dim
    else:
        raise ValueError("forward_paged_hip needs k_cache, k or offload_cache")
    wide_heads = hidden_size > 128

    want_stats = (cached_metadata is None) or (cached_metadata.indices is None) or (
        os.getenv("HIP_DISABLE_COMPUTE_STATISTICS", "1") == "0")

    if is_dense:
        default_scan_backend = "relative" if hip_config.apply_v_dot else "streaming"
    else:
        default_scan_backend = "relative"

    args = HiPAttentionArgs(
        k_cache=k_cache,
        v_cache=v_cache,
        offload_cache=offload_cache,
        block_table=block_table,
        cache_seq_lens=seq_lens,
        position_ids=positions.view(batch_size, dst_seq_len),
        block_size_k=32 if wide_heads else 64,
        sliding_window_size=layer_config.sliding_window_size,
        sink_token_size=layer_config.sink_token_size,
        using_extend=hip_config.using_extend,
        need_apply_rope=hip_config.using_extend,
        rope_cos=rope_cos,
        rope_sin=rope_sin,
        logit_softcap=logit_cap if logit_cap != 0.0 else None,
        second_stage_k=layer_config.second_stage_k,
        stages=layer_config.stages,
        model_context_length=orig_context_len,
        extend_context_length=max_context_len,
        block_sparse_block_size_q=hip_config.block_sparse_block_size_q,
        scan_extend_backend=(default_scan_backend if layer_config.scan_extend_backend is None
                             else layer_config.scan_extend_backend),
        sa_extend_backend=layer_config.sa_extend_backend,
        online_update_cache=online_update_cache,
        require_cache_statistics=want_stats,
        disable_flashdecode=not is_decode,
        q_mask=((query_for_mask * sm_scale).to(query.dtype) if query_for_mask is not None else None),
        layer_id=layer_id,
    )

    def scaled(qpart: torch.Tensor) -> torch.Tensor:
        return (qpart * sm_scale).to(query.dtype)

    if is_decode or (query.shape[1] < (_LAST_DENSE * 2)):
        context, metadata = dual_stage_quadratic_hip_attention(scaled(query), k, v, args=args,
                                                               cached_metadata=cached_metadata)
        context = context.to(query.dtype)[:, -query.shape[1]:, :, :].contiguous()
    else:
        assert query_for_mask is None
        position_ids = args.position_ids
        args.position_ids = position_ids[:, :-_LAST_DENSE]
        sparse_ctx, metadata = dual_stage_quadratic_hip_attention(
            scaled(query[:, :-_LAST_DENSE]), k, v, args=args, cached_metadata=cached_metadata)
        # 777 is the reference's sentinel for "window = whatever is left of the model context"
        args.sliding_window_size = 777
        args.position_ids = position_ids[:, -_LAST_DENSE:]
        dense_ctx, metadata = dual_stage_quadratic_hip_attention(
            scaled(query[:, -_LAST_DENSE:]), k, v, args=args, cached_metadata=cached_metadata)
        context = torch.cat([sparse_ctx.to(query.dtype), dense_ctx.to(query.dtype)], dim=1)

    return context.view(N, num_heads, hidden), metadata


def _sse(a: torch.Tensor, b: torch.Tensor) -> float:
    return float(((a.float() - b.float()) ** 2).sum())


def forward_paged_hip(
    query: torch.Tensor,
    sm_scale: float,
    batch_size: int,
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    offload_cache,
    positions: torch.Tensor,
    seq_lens: torch.Tensor,
    req_to_tokens: torch.Tensor,
    req_pool_indices: torch.Tensor,
    rope_cos: Optional[torch.Tensor],
    rope_sin: Optional[torch.Tensor],
    layer_id: int,
    logit_cap: float,
    orig_context_len: int,
    max_context_len: int,
    is_prefill: bool,
    hip_config: HiPAttentionConfig,
    cached_metadata: Optional[HiPAttentionOutputMetadata] = None,
    k: Optional[torch.Tensor] = None,
    v: Optional[torch.Tensor] = None,
    online_update_cache: bool = False,
    offloading_metadata=None,
    is_decode: bool = False,
    query_for_mask: Optional[torch.Tensor] = None,
    diag_sliding_window_indices: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, HiPAttentionOutputMetadata]:
    """The serving entry point (``paged_hip.py:35-320``): ``query [N, H, D]`` -> ``(context [N, H, D], metadata)``.

    ``offloading_metadata`` turns on the reference's self-check of an offloaded run (``:95-320``): it is the resident
    copy of the K / V token pools that ``HiPModelOffloadCache`` keeps under ``HIP_OFFLOAD_CACHE_VALIDATION=1``.  The
    call is repeated on that copy and the two outputs must agree (squared error below 1e-6 for prefill, 1e-7 for
    decode); for decode the host pools are compared with the copy as well.
    """
    common = dict(sm_scale=sm_scale, batch_size=batch_size, positions=positions, seq_lens=seq_lens,
                  req_to_tokens=req_to_tokens, req_pool_indices=req_pool_indices, rope_cos=rope_cos, rope_sin=rope_sin,
                  layer_id=layer_id, logit_cap=logit_cap, orig_context_len=orig_context_len,
                  max_context_len=max_context_len, is_prefill=is_prefill, hip_config=hip_config,
                  cached_metadata=cached_metadata, k=k, v=v, online_update_cache=online_update_cache,
                  is_decode=is_decode, query_for_mask=query_for_mask,
                  diag_sliding_window_indices=diag_sliding_window_indices)
    o, metadata = _forward_paged_hip(query, k_cache=k_cache, v_cache=v_cache, offload_cache=offload_cache, **common)
    if offloading_metadata is None:
        return o, metadata
    k_valid, v_valid = offloading_metadata
    if is_prefill:
        o_valid, _ = _forward_paged_hip(query, k_cache=k_valid, v_cache=v_valid, offload_cache=offload_cache, **common)
        err = _sse(o, o_valid)
        assert err < 1e-6, f"prefill on the validation pools differs: sse={err}"
        return o, metadata
    o_valid, metadata_valid = _forward_paged_hip(query, k_cache=k_valid, v_cache=v_valid, offload_cache=None, **common)
    err = _sse(o, o_valid)
    if err >= 1e-7:
        pool_k, pool_v = offload_cache.k_uvm.bank_cpu, offload_cache.v_uvm.bank_cpu
        n = min(pool_k.shape[0], k_valid.shape[0])
        wide = (lambda t: t.view(torch.float8_e5m2) if t.dtype == torch.uint8 else t)
        err_k = _sse(wide(pool_k[:n]).to(k_valid.device), wide(k_valid[:n]))
        err_v = _sse(wide(pool_v[:n]).to(v_valid.device), wide(v_valid[:n]))
        same_mask = (metadata.indices is not None and metadata_valid.indices is not None
                     and torch.equal(metadata.indices, metadata_valid.indices))
        raise AssertionError(f"decode on the offload cache differs from the validation pools: sse={err}, "
                             f"pool K / V against the copy: {err_k} / {err_v}, same block indices: {same_mask}")
    return o, metadata
