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

    for kw in (dict(using_extend=True), dict(is_causal=False),
               dict(online_update_cache=True), dict(sliding_window_indices=torch.zeros(1))):
        with pytest.raises(NotImplementedError):
            _reject_unsupported(HiPAttentionArgs12(**kw))
