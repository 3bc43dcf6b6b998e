"""Host-side logic that needs no GPU: config parsing, refresh schedule, argument defaults, exports."""
import json

import pytest


def test_refresh_schedule_matches_reference_rule():
    # mask_refresh_interval.py:8-29: -1 on step 0, else the first stage whose interval divides the step
    from hip_attn import HiPAttentionConfig, HiPMaskRefreshState

    st = HiPMaskRefreshState(HiPAttentionConfig())
    seq = [st.update() for _ in range(65)]
    assert seq[0] == -1
    for i in range(1, 65):
        want = 0 if i % 32 == 0 else 1 if i % 16 == 0 else 2 if i % 8 == 0 else None
        assert seq[i] == want, i
    cfg = HiPAttentionConfig(json_or_path='{"mask_refresh_interval": 4}')
    assert cfg.mask_refresh_interval == [4, 4, 4]
    st = HiPMaskRefreshState(cfg)
    assert [st.update() for _ in range(6)] == [-1, None, None, None, 0, None]


def test_config_json_defaults_and_unknown_keys(tmp_path):
    from hip_attn import HiPAttentionConfig
    from hip_attn.v1_2.hip_config import HiPAttentionPerLayerConfig

    cfg = HiPAttentionConfig()
    assert cfg.dense_layers == [0, 1, 2, 3, 31] and cfg.block_sparse_block_size_q == 64
    assert cfg.mask_refresh_interval == [32, 16, 8] and cfg.using_extend is True
    assert cfg.layers[0].second_stage_k == 4096 and cfg.layers[0].scan_extend_backend == "streaming"
    assert cfg.layers[1].second_stage_k == 2048 and cfg.layers[1].scan_extend_backend == "relative"
    assert cfg.layers[1].sliding_window_size == 1024 and cfg.layers[1].sink_token_size == 256
    assert [s.stage_chunk_size for s in cfg.layers[0].stages] == [256, 32, 8]
    spec = {"dense_layers": [0], "using_extend": False, "layers": [
        {"second_stage_k": 1024, "stages": [
            {"stage_block_size_q": 32, "stage_block_stride_q": 2, "stage_chunk_size": 64, "stage_k": None, "stage_stride": 1},
            {"stage_block_size_q": 32, "stage_block_stride_q": 1, "stage_chunk_size": 8, "stage_k": 4096, "stage_stride": 1}]},
        {"sliding_window_size": 256, "stages": [
            {"stage_block_size_q": 32, "stage_block_stride_q": 2, "stage_chunk_size": 64, "stage_k": None, "stage_stride": 1},
            {"stage_block_size_q": 32, "stage_block_stride_q": 1, "stage_chunk_size": 8, "stage_k": 4096, "stage_stride": 1}]}]}
    path = tmp_path / "hip.json"
    path.write_text(json.dumps(spec))
    for src in (json.dumps(spec), str(path)):
        cfg = HiPAttentionConfig(json_or_path=src)
        assert cfg.dense_layers == [0] and not cfg.using_extend
        assert cfg.layers[0].second_stage_k == 1024 and cfg.layers[1].sliding_window_size == 256
        assert cfg.layers[0].stages[1].stage_chunk_size == 8 and cfg.mask_refresh_interval == [32, 16, 8]
    with pytest.raises(ValueError):
        HiPAttentionConfig(json_or_path='{"no_such_key": 1}')
    with pytest.raises(ValueError):
        HiPAttentionPerLayerConfig(parsed_json={"second_stage_k": 1, "typo": 2})


def test_operator_argument_defaults_match_reference():
    # attention_metadata.py:133-215
    from hip_attn import HiPAttentionArgs12, ScanStage12

    a = HiPAttentionArgs12()
    assert (a.sink_token_size, a.sliding_window_size, a.block_size_k, a.second_stage_k) == (256, 512, 64, 2048)
    assert (a.model_context_length, a.extend_context_length) == (131072, 524288)
    assert a.block_sparse_block_size_q == 64 and a.stage_early_terminate == 1 and a.is_causal
    assert a.require_cache_statistics and a.require_stage_caches and not a.disable_flashdecode
    assert [(s.stage_block_size_q, s.stage_block_stride_q, s.stage_chunk_size, s.stage_k, s.stage_stride)
            for s in a.stages] == [(64, 4, 256, None, 1), (64, 4, 32, 32768, 1), (64, 1, 8, 8192, 1)]
    s = ScanStage12(64, 4, 256, None, 1)
    assert s.require_realign_index and s.require_reset_score and s.require_post_sort
    assert HiPAttentionArgs12(logit_softcap=0).logit_softcap is None
    b = a.clone()
    b.sliding_window_size = 7
    assert a.sliding_window_size == 512


def test_reference_import_paths_resolve():
    import hip_attn
    from hip_attn.v1_2 import HiPAttentionConfig, HiPMaskRefreshState, forward_paged_hip, hip_attention  # noqa: F401
    from hip_attn.v1_2.attention_extend import dual_stage_quadratic_hip_attention
    from hip_attn.v1_2.attention_metadata import HiPAttentionArgs, HiPAttentionOutputMetadata, ScanStage  # noqa: F401
    from hip_attn.v1_2.paged_hip import forward_paged_hip as f2  # noqa: F401

    assert hip_attn.hip_attention_12 is dual_stage_quadratic_hip_attention
    assert hip_attn.hip_attention is hip_attn.hip_attention_12
    assert hip_attn.HiPAttentionArgs is hip_attn.HiPAttentionArgs12


def test_unsupported_options_fail_loudly():
    import torch
    from hip_attn import HiPAttentionArgs12
    from hip_attn.operator import _reject_unsupported

    for kw in (dict(using_extend=True),
               dict(online_update_cache=True), dict(sliding_window_indices=torch.zeros(1))):
        with pytest.raises(NotImplementedError):
            _reject_unsupported(HiPAttentionArgs12(**kw))


def test_metadata_cache_pool_round_trip_on_cpu():
    """HiPMetadataCachePool: storage formats, batch slicing and stage-level getters (hip_memory_pool.py:55-409)."""
    import torch
    from hip_attn import HiPAttentionConfig, HiPMetadataCachePool, cuda_graph_capture_configs
    from hip_attn.metadata import HiPAttentionOutputMetadata, HiPAttentionStageInputCache

    cfg = HiPAttentionConfig()
    assert cuda_graph_capture_configs(cfg) == [(None,), (0,), (1,), (2,)]
    H, B = 4, 3
    pool = HiPMetadataCachePool(max_total_num_tokens=1 << 16, query_head_num=H, layer_num=2, context_length=1 << 17,
                                device="cpu", hip_config=cfg)
    lc = pool.layer_configs[1]
    nblk = lc.second_stage_k // lc.stages[-1].stage_chunk_size
    assert pool.cache[1]["indices"].buffer.dtype == torch.uint32
    assert pool.cache[1]["indices"].buffer.shape == (cfg.metadata_cache_max_batch_size * H, 1, nblk)
    assert pool.cache[1]["stage_1_out_scores"].buffer.dtype == torch.bfloat16
    assert pool.compute_allocated_bytes() == pool.allocated_gpu_bytes > 0
    g = torch.Generator().manual_seed(0)
    idx = torch.randint(0, 1 << 20, (B * H, 1, nblk), generator=g, dtype=torch.int64).sort(-1).values
    idx[:, :, -5:] = torch.iinfo(torch.int64).max  # padding entries wrap to 2^32 - 1 in storage
    ks = torch.full((B * H, 1), nblk - 5, dtype=torch.int64)
    kse = torch.zeros((B * H, 1, 2), dtype=torch.int32); kse[..., 1] = nblk - 5
    stage = lambda n: HiPAttentionStageInputCache(
        torch.randint(0, 1 << 20, (B, 1, H, n), generator=g), torch.randint(0, 1 << 20, (B, 1, H, n), generator=g),
        torch.randn((B, 1, H, n), generator=g))
    n1 = pool.cache[1]["stage_1_indices_left"].buffer.shape[-1]
    n2 = pool.cache[1]["stage_2_indices_left"].buffer.shape[-1]
    meta = HiPAttentionOutputMetadata(indices=idx, ks=ks, ks_count=ks.unsqueeze(-1), ks_start_end=kse,
                                      mask_cache_statistics=None, sa_cache_statistics=None,
                                      stage_caches=[HiPAttentionStageInputCache(None, None, None), stage(n1), stage(n2)])
    pool.set_hip_metadata_cache(1, B, B, meta)
    back = pool.get_hip_metadata_cache(1, B, B, None)
    assert back.indices.dtype == torch.int64 and back.indices.shape == idx.shape
    assert torch.equal(back.indices[:, :, :-5], idx[:, :, :-5]) and (back.indices[:, :, -5:] == 2 ** 32 - 1).all()
    assert torch.equal(back.ks, ks) and torch.equal(back.ks_start_end, kse.to(torch.int64))
    assert back.stage_caches is None
    assert pool.get_hip_metadata_cache(1, B, B, 0) is None
    part = pool.get_hip_metadata_cache(1, B, B, 2)
    assert part.indices is None and len(part.stage_caches) == 3 and part.stage_caches[0].indices_left is None
    assert torch.equal(part.stage_caches[2].indices_left, meta.stage_caches[2].indices_left)
    assert torch.equal(part.stage_caches[1].out_scores, meta.stage_caches[1].out_scores.to(torch.bfloat16).float())
    # a smaller batch reads a prefix; a larger one than the pool holds is refused
    small = pool.get_hip_metadata_cache(1, 2, 2, None)
    assert torch.equal(small.indices, back.indices[: 2 * H])
    with pytest.raises(ValueError):
        pool.get_buffer(1, "stage_1_indices_left", cfg.metadata_cache_max_batch_size + 1)
    with pytest.raises(KeyError):
        pool.get_buffer(1, "nope", 1)


def test_operands_of_another_dtype_or_device_are_refused():
    # the C side sizes every K / V row from q's dtype: a mismatch must never reach a kernel
    import torch
    from hip_attn import HiPAttentionArgs12
    from hip_attn._native import HipAttnError
    from hip_attn.operator import _check_operands, dual_stage_quadratic_hip_attention

    q = torch.zeros((1, 4, 4, 64), dtype=torch.float32)
    k = torch.zeros((1, 64, 1, 64), dtype=torch.float32)
    _check_operands(q, k, k, HiPAttentionArgs12())
    for bad in (k.to(torch.bfloat16), k.to(torch.float16), k.to(torch.float64)):
        with pytest.raises(HipAttnError, match="dtype"):
            _check_operands(q, bad, k, HiPAttentionArgs12())
        with pytest.raises(HipAttnError, match="dtype"):
            _check_operands(q, k, bad, HiPAttentionArgs12())
    kc = torch.zeros((8, 16, 1, 64), dtype=torch.bfloat16)
    with pytest.raises(HipAttnError, match="k_cache"):
        _check_operands(q, None, None, HiPAttentionArgs12(k_cache=kc, v_cache=kc))
    qb = q.to(torch.bfloat16)
    _check_operands(qb, None, None, HiPAttentionArgs12(k_cache=kc, v_cache=kc))
    _check_operands(qb, None, None, HiPAttentionArgs12(k_cache=kc.view(torch.uint8)[..., :64], v_cache=kc.view(torch.uint8)[..., :64]))
    with pytest.raises(HipAttnError, match="k_cache"):  # fp8 bytes need bf16 queries
        _check_operands(q, None, None, HiPAttentionArgs12(k_cache=kc.view(torch.uint8), v_cache=kc.view(torch.uint8)))
    with pytest.raises(HipAttnError, match="q_mask"):
        _check_operands(q, k, k, HiPAttentionArgs12(q_mask=qb))
    meta = torch.zeros((1, 64, 1, 64), dtype=torch.float32, device="meta")
    with pytest.raises(HipAttnError, match="device"):
        _check_operands(q, meta, k, HiPAttentionArgs12())
    with pytest.raises(HipAttnError, match="block_table"):
        _check_operands(qb, None, None, HiPAttentionArgs12(
            k_cache=kc, v_cache=kc, block_table=torch.zeros((1, 8), dtype=torch.int64, device="meta")))
    with pytest.raises(HipAttnError, match="GPU only"):
        dual_stage_quadratic_hip_attention(q, k, k, HiPAttentionArgs12())


def test_helper_tensors_a_graph_has_seen_are_never_evicted(monkeypatch):
    # a captured graph records addresses: what was handed out during a capture must outlive every eviction
    import torch
    from hip_attn import operator as op

    cache, pinned, capturing = {}, {}, [False]
    monkeypatch.setattr(op, "_capturing", lambda device: capturing[0])
    dev = torch.device("cpu")
    built = []

    def get(key):
        return op._cached_for_graphs(cache, pinned, key, lambda: built.append(key) or torch.full((1,), key), 4, dev)

    a = get(0)                       # eager warm-up builds and keeps it
    capturing[0] = True
    assert get(0) is a and 0 in pinned and 0 not in cache   # the capture sees the kept tensor: pinned from now on
    b = get(100)                     # built inside a capture: the graph's pool owns it, not kept
    assert 100 not in cache and 100 not in pinned and get(100) is not b
    capturing[0] = False
    for key in range(1, 40):         # far more shapes than the limit
        get(key)
    assert len(cache) == 4 and get(0) is a and built.count(0) == 1
    assert 1 not in cache and get(1) is not None and built.count(1) == 2   # unpinned entries are evicted oldest first


def test_key_buffers_of_32_gib_are_reported_to_the_scan():
    """Scan launches that pass the places of key rows between lanes as 31-bit piece numbers must be told when a
    buffer is too large for that; the span counts strides, not elements."""
    import torch
    from hip_attn import operator as op

    small = torch.empty((1, 1 << 20, 8, 128), dtype=torch.bfloat16, device="meta")
    assert not op._spans_32_gib(small) and not op._spans_32_gib(None)
    pool = torch.empty(((1 << 20) + 1, 16, 8, 128), dtype=torch.bfloat16, device="meta")  # 32 KiB pages: one more than 32 GiB
    assert op._spans_32_gib(pool)
    assert not op._spans_32_gib(pool[: 1 << 19])
    assert op._spans_32_gib(pool[:: 1 << 19])  # three pages, 16 GiB apart
