"""GPU parity of forward_paged_hip (the serving entry point) against the oracle."""
import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs
from gpu_utils import assert_context_close, assert_metadata_equal, from_torch, to_torch

pytestmark = pytest.mark.gpu


def _pool(X, seed):
    """Token-granular KV pool + req_to_tokens as a serving framework keeps them (page size 1)."""
    B, TK, HKV, D = X.k.shape
    rng = np.random.default_rng(seed)
    slots = rng.permutation(np.arange(1, B * TK + 8))[: B * TK].reshape(B, TK)
    kc = np.zeros((B * TK + 8, HKV, D), dtype=X.k.dtype)
    vc = np.zeros_like(kc)
    for b in range(B):
        kc[slots[b]] = X.k[b]
        vc[slots[b]] = X.v[b]
    req_to_tokens = np.zeros((B + 3, TK), dtype=np.int32)
    pool_idx = np.array([2, 0, 4][:B])
    req_to_tokens[pool_idx] = slots
    return kc, vc, req_to_tokens, pool_idx


def _config(sw):
    from hip_attn import HiPAttentionConfig

    spec = ('{"using_extend": false, "dense_layers": [0], "layers": [{"second_stage_k": 256, "sliding_window_size": %d},'
            '{"second_stage_k": 128, "sliding_window_size": %d}], "prefill_layers": [{"second_stage_k": 256, '
            '"sliding_window_size": %d}, {"second_stage_k": 128, "sliding_window_size": %d}]}') % (sw, sw, sw, sw)
    return HiPAttentionConfig(json_or_path=spec)


def _oracle(X, kc, vc, r2t, pool_idx, lens, sm_scale, second_k, sw, max_ctx, disable_flashdecode, model_ctx=131072):
    qs = O.bf16_bits_to_f32(X.q) * np.float32(sm_scale)
    XP = O.OInputs("bf16", O.f32_to_bf16_bits(qs), X.pos, k_cache=kc[:, None], v_cache=vc[:, None],
                   block_table=r2t[pool_idx].astype(np.int64), cache_seq_lens=lens.astype(np.int64))
    A = O.OArgs(sliding_window_size=sw, second_stage_k=second_k, extend_context_length=max_ctx,
                model_context_length=model_ctx, disable_flashdecode=disable_flashdecode)
    return XP, A


def test_forward_paged_hip_decode_and_short_prefill():
    from hip_attn import forward_paged_hip

    print("[case] forward_paged_hip decode", flush=True)
    B, TK, H, HKV, D, sw = 2, 3072, 8, 2, 128, 512
    lens = np.array([3072, 2000])
    X = make_inputs(21, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=(lens - 1)[:, None])
    kc, vc, r2t, pool_idx = _pool(X, 1)
    cfg = _config(sw)
    sm = D ** -0.5
    dev = "cuda"
    common = dict(sm_scale=sm, batch_size=B, k_cache=to_torch(kc, "bf16", dev), v_cache=to_torch(vc, "bf16", dev),
                  offload_cache=None, seq_lens=torch.from_numpy(lens).to(dev), req_to_tokens=torch.from_numpy(r2t).to(dev),
                  req_pool_indices=torch.from_numpy(pool_idx).to(dev), rope_cos=None, rope_sin=None, logit_cap=0.0,
                  orig_context_len=131072, max_context_len=TK, hip_config=cfg)
    q = to_torch(X.q, "bf16", dev).view(B, H, D)
    for layer_id, second_k in ((0, 256), (5, 128)):
        out, meta = forward_paged_hip(q, positions=torch.from_numpy(X.pos.reshape(-1)).to(dev), layer_id=layer_id,
                                      is_prefill=False, is_decode=True, **common)
        XP, A = _oracle(X, kc, vc, r2t, pool_idx, lens, sm, second_k, sw, TK, False)
        octx, ometa = O.hip_attention_12(XP, A)
        assert out.shape == (B, H, D)
        assert_metadata_equal(meta, ometa)
        assert_context_close(out.view(B, 1, H, D), octx, "bf16")
        out2, meta2 = forward_paged_hip(q, positions=torch.from_numpy(X.pos.reshape(-1)).to(dev), layer_id=layer_id,
                                        is_prefill=False, is_decode=True, cached_metadata=meta, **common)
        assert_context_close(out2.view(B, 1, H, D), octx, "bf16")


def test_forward_paged_hip_long_prefill_splits_off_last_64_queries():
    from hip_attn import forward_paged_hip

    print("[case] forward_paged_hip prefill", flush=True)
    B, TK, TQ, H, HKV, D, sw = 1, 2048, 192, 4, 2, 64, 256
    X = make_inputs(22, B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16")
    kc, vc, r2t, pool_idx = _pool(X, 2)
    lens = np.array([TK])
    cfg = _config(sw)
    sm = D ** -0.5
    dev = "cuda"
    out, meta = forward_paged_hip(
        to_torch(X.q, "bf16", dev).view(B * TQ, H, D), sm_scale=sm, batch_size=B, k_cache=to_torch(kc, "bf16", dev),
        v_cache=to_torch(vc, "bf16", dev), offload_cache=None, positions=torch.from_numpy(X.pos.reshape(-1)).to(dev),
        seq_lens=torch.from_numpy(lens).to(dev), req_to_tokens=torch.from_numpy(r2t).to(dev),
        req_pool_indices=torch.from_numpy(pool_idx).to(dev), rope_cos=None, rope_sin=None, layer_id=7, logit_cap=0.0,
        orig_context_len=4096, max_context_len=TK, is_prefill=True, hip_config=cfg)
    # oracle: same two calls
    XP, A = _oracle(X, kc, vc, r2t, pool_idx, lens, sm, 128, sw, TK, True, model_ctx=4096)
    first = O.OInputs("bf16", XP.q[:, :-64], XP.pos[:, :-64], k_cache=XP.k_cache, v_cache=XP.v_cache,
                      block_table=XP.block_table, cache_seq_lens=XP.cache_seq_lens)
    octx1, _ = O.hip_attention_12(first, A)
    last = O.OInputs("bf16", XP.q[:, -64:], XP.pos[:, -64:], k_cache=XP.k_cache, v_cache=XP.v_cache,
                     block_table=XP.block_table, cache_seq_lens=XP.cache_seq_lens)
    A2 = O.OArgs(**{**A.__dict__, "sliding_window_size": 777})
    octx2, ometa2 = O.hip_attention_12(last, A2)
    assert_metadata_equal(meta, ometa2)
    got = out.view(B, TQ, H, D)
    assert_context_close(got[:, :-64], octx1, "bf16")
    assert_context_close(got[:, -64:], octx2, "bf16")


def test_forward_paged_hip_decode_with_rope_applied_on_load():
    """using_extend on (the configuration default): the KV pool holds keys without rotation and the serving stack
    hands over its cos/sin tables; dense layers scan with the streaming rule, the others with the relative one."""
    from hip_attn import HiPAttentionConfig, forward_paged_hip
    from helpers import rope_tables

    print("[case] forward_paged_hip decode, rope on load", flush=True)
    B, TK, H, HKV, D, sw = 2, 3072, 8, 2, 128, 512
    lens = np.array([3072, 2000])
    X = make_inputs(23, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=(lens - 1)[:, None])
    kc, vc, r2t, pool_idx = _pool(X, 3)
    spec = ('{"dense_layers": [0], "layers": [{"second_stage_k": 256, "sliding_window_size": %d},'
            '{"second_stage_k": 128, "sliding_window_size": %d}]}') % (sw, sw)
    cfg = HiPAttentionConfig(json_or_path=spec)
    assert cfg.using_extend
    cos, sin, _ = rope_tables(4096, D, "bf16")
    sm = D ** -0.5
    dev = "cuda"
    common = dict(sm_scale=sm, batch_size=B, k_cache=to_torch(kc, "bf16", dev), v_cache=to_torch(vc, "bf16", dev),
                  offload_cache=None, seq_lens=torch.from_numpy(lens).to(dev), req_to_tokens=torch.from_numpy(r2t).to(dev),
                  req_pool_indices=torch.from_numpy(pool_idx).to(dev),
                  rope_cos=to_torch(O.f32_to_bf16_bits(cos), "bf16", dev), rope_sin=to_torch(O.f32_to_bf16_bits(sin), "bf16", dev),
                  logit_cap=0.0, orig_context_len=131072, max_context_len=TK, hip_config=cfg)
    q = to_torch(X.q, "bf16", dev).view(B, H, D)
    for layer_id, second_k, scan in ((0, 256, "streaming"), (5, 128, "relative")):
        out, meta = forward_paged_hip(q, positions=torch.from_numpy(X.pos.reshape(-1).copy()).to(dev), layer_id=layer_id,
                                      is_prefill=False, is_decode=True, **common)
        XP, A = _oracle(X, kc, vc, r2t, pool_idx, lens, sm, second_k, sw, TK, False)
        XP.rope_cos, XP.rope_sin = cos, sin
        A.using_extend = A.need_apply_rope = True
        A.scan_extend_backend, A.sa_extend_backend = scan, "streaming"
        octx, ometa = O.hip_attention_12(XP, A)
        assert_metadata_equal(meta, ometa)
        assert_context_close(out.view(B, 1, H, D), octx, "bf16")


def test_metadata_cache_pool_hands_masks_between_decode_steps():
    """A mask stored in HiPMetadataCachePool after a refresh step drives the next steps (finished mask, or the
    inputs of a later stage) exactly like the metadata object itself."""
    from hip_attn import HiPAttentionArgs12, HiPAttentionConfig, HiPMetadataCachePool, hip_attention_12
    from helpers import to_paged

    print("[case] metadata cache pool", flush=True)
    B, TK, H, HKV, D = 2, 16384, 8, 2, 128
    lens = np.array([16384, 9000])
    X = make_inputs(24, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=(lens - 1)[:, None])
    XP = to_paged(X, 16, seed=9, seq_lens=lens)
    dev = "cuda"
    cfg = HiPAttentionConfig()
    pool = HiPMetadataCachePool(max_total_num_tokens=B * TK, query_head_num=H, layer_num=2, context_length=TK,
                                device=dev, hip_config=cfg)
    layer = pool.layer_configs[1]

    def args():
        return HiPAttentionArgs12(
            k_cache=to_torch(XP.k_cache, "bf16", dev), v_cache=to_torch(XP.v_cache, "bf16", dev),
            block_table=torch.from_numpy(XP.block_table).to(dev), cache_seq_lens=torch.from_numpy(XP.cache_seq_lens).to(dev),
            position_ids=torch.from_numpy(XP.pos.copy()).to(dev), sliding_window_size=layer.sliding_window_size,
            sink_token_size=layer.sink_token_size, second_stage_k=layer.second_stage_k, stages=layer.stages,
            extend_context_length=TK)

    q = to_torch(X.q, "bf16", dev)
    out, meta = hip_attention_12(q, None, None, args())
    pool.set_hip_metadata_cache(1, B, B, meta)
    # finished mask out of the pool
    cached = pool.get_hip_metadata_cache(1, B, B, None)
    assert torch.equal(cached.ks, meta.ks)
    out_c, _ = hip_attention_12(q, None, None, args(), cached_metadata=cached)
    assert torch.equal(out_c, out)
    # inputs of the last stage out of the pool: estimation resumes there and ends in the same mask
    resumed = pool.get_hip_metadata_cache(1, B, B, len(layer.stages) - 1)
    out_r, meta_r = hip_attention_12(q, None, None, args(), cached_metadata=resumed)
    assert torch.equal(meta_r.indices, meta.indices) and torch.equal(meta_r.ks, meta.ks)
    assert torch.equal(out_r, out)
