"""Randomly drawn calls of ``hip_attention_12`` against the oracle.

Forty draws over dtype (bf16 / f32), head dim, GQA group, batch, query length (1 to 777), key length, page size
(dense, 1, 4, 16), sliding window, ragged sequence lengths and statistics on / off: selected blocks, ``ks`` and access
flags must equal the oracle's, the context must lie within the accepted tolerance, and a second call that reuses the
mask must give the same context.  (Longer runs of the same draw, 2510 cases over eleven seeds, found no difference.)
"""
import random

import numpy as np
import pytest

from oracle import hip12 as O
from helpers import make_inputs, to_paged
from gpu_utils import assert_context_close, assert_metadata_equal, run_product

pytestmark = pytest.mark.gpu


def test_random_calls_match_the_oracle():
    rng = random.Random(11)
    for it in range(40):
        D = rng.choice([64, 128, 128])
        HKV = rng.choice([1, 2, 4])
        H = HKV * rng.choice([1, 2, 4, 4, 8])
        decode = rng.random() < 0.4
        TK = rng.choice([1500, 3000, 4096, 6000, 8192, 12000, 16384])
        TQ = 1 if decode else rng.choice([1, 17, 64, 130, 200, 300, 512, 777])
        B = rng.choice([1, 2, 3])
        paged = rng.choice([0, 0, 1, 4, 16])
        sw = rng.choice([128, 256, 512, 1024])
        dtype = rng.choice(["bf16", "bf16", "bf16", "f32"])
        if D == 128 and dtype == "f32" and TK > 8192:
            TK = 8192
        stats = rng.random() < 0.6
        if decode:
            lens = np.array([rng.randint(max(TK // 2, sw + 300), TK) for _ in range(B)])
            if not paged:
                lens[:] = TK
            X = make_inputs(1000 + it, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, pos=(lens - 1)[:, None])
        else:
            lens = None
            X = make_inputs(1000 + it, B=B, TQ=min(TQ, TK), TK=TK, H=H, HKV=HKV, D=D, dtype=dtype)
        A = O.OArgs(sliding_window_size=sw)
        if paged:
            X = to_paged(X, paged, seed=it, seq_lens=lens) if decode else to_paged(X, paged, seed=it)
            A.extend_context_length = TK
        print(f"[case {it}] {dtype} D={D} H={H}/{HKV} B={B} TQ={TQ} TK={TK} paged={paged} sw={sw} decode={decode} "
              f"stats={stats}", flush=True)
        ctx, meta = run_product(X, A, require_cache_statistics=stats)
        octx, ometa = O.hip_attention_12(X, A)
        assert_metadata_equal(meta, ometa)
        assert_context_close(ctx, octx, dtype)
        ctx2, _ = run_product(X, A, cached=meta, require_cache_statistics=stats)
        assert_context_close(ctx2, octx, dtype)


def test_random_calls_with_rotation_on_load_match_the_oracle():
    """Thirty draws over the rotation rules of the scan (relative / streaming / infllm / dynamic_extend) and of the
    attention (streaming / infllm / dynamic_extend), model context lengths below and above the key length, logit
    soft-capping on / off, prefill and ragged paged decode.  (1980 cases of the same draw over six seeds, 400 of them with the prescaled and coalesced variants forced, found no difference.)"""
    from helpers import tiny_args, with_rope

    rng = random.Random(21)
    for it in range(30):
        D = rng.choice([64, 128])
        HKV = rng.choice([1, 2])
        H = HKV * rng.choice([1, 2, 4])
        decode = rng.random() < 0.4
        TK = rng.choice([1500, 2048, 3000, 4096])
        TQ = 1 if decode else rng.choice([1, 40, 130, 200, 256])
        B = rng.choice([1, 2])
        paged = rng.choice([0, 1, 16]) if not decode else rng.choice([1, 16])
        dtype = rng.choice(["bf16", "bf16", "f32"])
        scan = rng.choice(["relative", "streaming", "infllm", "dynamic_extend"])
        sa = rng.choice(["streaming", "infllm", "dynamic_extend"])
        model_ctx = rng.choice([1024, 2048, 131072])
        cap = rng.choice([None, None, 30.0])
        if decode:
            lens = np.array([rng.randint(TK // 2, TK) for _ in range(B)])
            X = make_inputs(2000 + it, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, pos=(lens - 1)[:, None],
                            scale=0.5)
        else:
            lens = None
            X = make_inputs(2000 + it, B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=0.5)
        kw = dict(using_extend=True, need_apply_rope=True, scan_extend_backend=scan, sa_extend_backend=sa,
                  model_context_length=model_ctx)
        if cap:
            kw["logit_softcap"] = cap
        if paged:
            X = to_paged(X, paged, seed=it, seq_lens=lens) if decode else to_paged(X, paged, seed=it)
            kw["extend_context_length"] = TK
        X = with_rope(X, 8192)
        print(f"[case {it}] {dtype} D={D} H={H}/{HKV} B={B} TQ={TQ} TK={TK} paged={paged} scan={scan} sa={sa} "
              f"model_ctx={model_ctx} softcap={cap} decode={decode}", flush=True)
        A = tiny_args(**kw)
        octx, ometa = O.hip_attention_12(X, A)
        ctx, meta = run_product(X, A)
        assert_metadata_equal(meta, ometa)
        assert_context_close(ctx, octx, dtype)


def _draw_later_options(rng, it):
    """One draw over the options beyond the plain call: non-causal attention, head dim 256, a caller-kept pre-scaled key
    copy, the self_extend scan rule and the dynamic_extend attention rule (bf16: on the matrix-core kernels)."""
    from helpers import tiny_args, with_rope

    D = rng.choice([64, 128, 128, 256])
    HKV = rng.choice([1, 2])
    H = HKV * rng.choice([1, 2, 4])
    decode = rng.random() < 0.4
    TK = rng.choice([1500, 2048, 3000, 4096, 9000])
    TQ = 1 if decode else rng.choice([1, 40, 130, 200, 256])
    B = rng.choice([1, 2])
    paged = rng.choice([0, 1, 16]) if not decode else rng.choice([0, 16])
    dtype = "f32" if (D != 256 and rng.random() < 0.2) else "bf16"
    rope = rng.random() < 0.5
    causal = rng.random() < 0.7
    prescaled = (not rope) and dtype == "bf16" and rng.random() < 0.5
    cap = rng.choice([None, None, 30.0])
    big = rng.random() < 0.3
    if decode:
        lens = np.array([rng.randint(TK // 2, TK) for _ in range(B)])
        if not paged:
            lens[:] = TK
        X = make_inputs(5000 + it, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, pos=(lens - 1)[:, None], scale=0.5)
    else:
        lens = None
        X = make_inputs(5000 + it, B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=0.5)
    kw = dict(is_causal=causal)
    desc = f"{dtype} D={D} H={H}/{HKV} B={B} TQ={TQ} TK={TK} paged={paged} causal={causal} prescaled={prescaled} softcap={cap}"
    if rope:
        scan = rng.choice(["self_extend", "self_extend", "dynamic_extend", "relative", "streaming"])
        sa = rng.choice(["dynamic_extend", "dynamic_extend", "streaming", "infllm"])
        model_ctx = rng.choice([1024, 2048, 131072])
        kw.update(using_extend=True, need_apply_rope=True, scan_extend_backend=scan, sa_extend_backend=sa,
                  model_context_length=model_ctx, extend_context_length=TK)
        desc += f" scan={scan} sa={sa} model_ctx={model_ctx}"
    if cap:
        kw["logit_softcap"] = cap
    if paged:
        X = to_paged(X, paged, seed=it, seq_lens=lens) if decode else to_paged(X, paged, seed=it)
        kw["extend_context_length"] = TK
    if rope:
        X = with_rope(X, 16384)
    A = O.OArgs(sliding_window_size=rng.choice([256, 512]), **kw) if big else tiny_args(**kw)
    return X, A, dtype, prescaled, desc + f" default_stages={big}"


def test_random_calls_with_the_later_options_match_the_oracle():
    """Twenty-eight draws over non-causal attention, head dim 256 (two column passes per head in the tile kernel), a
    caller-kept pre-scaled key copy, the self_extend scan rule and the dynamic_extend attention rule.  (1350 cases of the
    same draw over four seeds found no difference.)"""
    from gpu_utils import to_torch
    from hip_attn import prescale_keys

    rng = random.Random(61)
    for it in range(28):
        X, A, dtype, prescaled, desc = _draw_later_options(rng, it)
        print(f"[case {it}] {desc}", flush=True)
        extra = {}
        if prescaled:
            extra["k_prescaled"] = prescale_keys(to_torch(X.k if X.k is not None else X.k_cache, "bf16"))
        octx, ometa = O.hip_attention_12(X, A)
        ctx, meta = run_product(X, A, **extra)
        assert_metadata_equal(meta, ometa)
        assert_context_close(ctx, octx, dtype)


def test_random_calls_on_fp8_caches_match_the_oracle():
    """Twenty-four draws on fp8 (e5m2) paged caches: head dims 64 / 128 / 256, page sizes 1 / 4 / 16, prefill and ragged
    decode, with and without rotation on load and soft-capping, small and default stage settings; the oracle runs on the
    same values held as bf16.  (420 cases of the same draw over two seeds found no difference.)"""
    from helpers import tiny_args, with_rope
    from test_gpu_fp8 import _quantise, _run

    rng = random.Random(41)
    for it in range(24):
        D = rng.choice([64, 128, 128, 256])
        HKV = rng.choice([1, 2])
        H = HKV * rng.choice([1, 2, 4])
        decode = rng.random() < 0.5
        TK = rng.choice([1500, 2048, 3000, 4096])
        TQ = 1 if decode else rng.choice([1, 40, 130, 200, 256])
        B = rng.choice([1, 2, 3])
        page = rng.choice([1, 4, 16])
        rope = rng.random() < 0.3
        cap = rng.choice([None, None, 30.0])
        big = rng.random() < 0.4
        if decode:
            lens = np.array([rng.randint(TK // 2, TK) for _ in range(B)])
            X = make_inputs(3000 + it, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=(lens - 1)[:, None],
                            scale=0.5)
        else:
            lens = None
            X = make_inputs(3000 + it, B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", scale=0.5)
        XP = to_paged(X, page, seed=it, seq_lens=lens) if decode else to_paged(X, page, seed=it)
        kw = dict(extend_context_length=TK)
        if rope:
            XP = with_rope(XP, 8192)
            kw.update(using_extend=True, need_apply_rope=True,
                      scan_extend_backend=rng.choice(["relative", "streaming", "infllm"]),
                      sa_extend_backend=rng.choice(["streaming", "infllm"]))
        if cap:
            kw["logit_softcap"] = cap
        A = O.OArgs(sliding_window_size=rng.choice([256, 512]), **kw) if big else tiny_args(**kw)
        as_bytes = rng.random() < 0.5
        print(f"[case {it}] D={D} H={H}/{HKV} B={B} TQ={TQ} TK={TK} page={page} rope={rope} softcap={cap} "
              f"decode={decode} default_stages={big}", flush=True)
        XQ, kc, vc = _quantise(XP)
        octx, ometa = O.hip_attention_12(XQ, A)
        ctx, meta = _run(XQ, A, kc, vc, as_bytes)
        assert_metadata_equal(meta, ometa)
        assert_context_close(ctx, octx, "bf16")


def test_random_offload_caches_equal_resident_keys_and_the_oracle():
    """Sixteen draws of an offloaded key pool behind device caches of random sizes (from far too small, so that blocks
    are evicted in every step, to holding everything), block sizes 8 / 16 / 32, ragged batches, prefill and decode:
    over four steps with a commit after each, masks must equal the oracle's and contexts the resident run's bit for
    bit.  (250 cases of the same draw over two seeds found no difference.)"""
    import torch
    from gpu_utils import to_torch
    from hip_attn import HiPOffloadCache, hip_attention_12
    from test_gpu_offload import _args, _bits, _fill, _offloaded_case

    rng = random.Random(51)
    for it in range(16):
        D = rng.choice([64, 128])
        HKV = rng.choice([1, 2, 4])
        H = HKV * rng.choice([1, 2, 4])
        B = rng.choice([1, 2, 3])
        TK = rng.choice([1024, 2048, 3000, 4096])
        TQ = rng.choice([1, 1, 1, 17, 64])
        lens = np.array([rng.randint(max(TK // 2, 600), TK) for _ in range(B)])
        mask_tokens = rng.choice([1 << 20, 4096, 1024, 256])
        sa_tokens = rng.choice([1 << 20, 4096, 1024, 512])
        block_tokens = rng.choice([16, 16, 8, 32])
        print(f"[case {it}] D={D} H={H}/{HKV} B={B} TQ={TQ} TK={TK} lens={lens.tolist()} mask_tokens={mask_tokens} "
              f"sa_tokens={sa_tokens} block_tokens={block_tokens}", flush=True)
        X, XP = _offloaded_case(4000 + it, B, TK, H, HKV, D, lens, TQ)
        A = O.OArgs(sliding_window_size=256, second_stage_k=512, extend_context_length=TK,
                    stages=[O.OStage(64, 4, 64, None, 1), O.OStage(64, 4, 16, 1024, 1), O.OStage(64, 1, 8, 512, 1)])
        octx, ometa = O.hip_attention_12(XP, A)
        rows = XP.k_cache.shape[0]
        cache = HiPOffloadCache(0, rows, mask_tokens, sa_tokens, HKV, D, torch.bfloat16, torch.device("cuda"),
                                block_tokens=block_tokens)
        _fill(cache, XP)
        q = to_torch(X.q, "bf16")
        res_args = _args(XP, A, k_cache=to_torch(XP.k_cache, "bf16"), v_cache=to_torch(XP.v_cache, "bf16"))
        ctx_res, meta_res = hip_attention_12(q, None, None, res_args)
        assert_metadata_equal(meta_res, ometa)
        for step in range(4):
            ctx, meta = hip_attention_12(q, None, None, _args(XP, A, offload_cache=cache))
            torch.cuda.synchronize()
            assert_metadata_equal(meta, ometa)
            assert torch.equal(_bits(ctx), _bits(ctx_res)), f"case {it}, step {step}: offloaded context differs"
            cache.handle_cache_miss(meta)
        assert_context_close(ctx, octx, "bf16")
        del cache
