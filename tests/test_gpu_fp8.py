"""fp8 (e5m2) paged KV caches: rows are widened to bf16 on load, exactly, so the product on the fp8 cache must equal the
oracle run on the same values held as bf16 (``paged_hip.py:409-418``, ``uvm_gpu_cache.py:1043-1046``)."""
import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, tiny_args, to_paged, with_rope
from gpu_utils import assert_context_close, assert_metadata_equal, from_torch, product_args, to_torch

pytestmark = pytest.mark.gpu


def _quantise(XP):
    """Round the paged K/V of an OInputs to e5m2; returns (oracle inputs holding the rounded values as bf16, fp8 caches)."""
    kc = to_torch(XP.k_cache, "bf16", "cpu").to(torch.float8_e5m2)
    vc = to_torch(XP.v_cache, "bf16", "cpu").to(torch.float8_e5m2)
    XQ = O.OInputs("bf16", XP.q, XP.pos, k_cache=from_torch(kc.to(torch.bfloat16), "bf16"),
                   v_cache=from_torch(vc.to(torch.bfloat16), "bf16"), block_table=XP.block_table,
                   cache_seq_lens=XP.cache_seq_lens)
    XQ.rope_cos, XQ.rope_sin = XP.rope_cos, XP.rope_sin
    return XQ, kc, vc


def _run(XQ, A, kc, vc, view_u8, cached=None):
    from hip_attn import hip_attention_12
    args = product_args(A, XQ)
    kcd, vcd = kc.cuda(), vc.cuda()
    args.k_cache = kcd.view(torch.uint8) if view_u8 else kcd
    args.v_cache = vcd.view(torch.uint8) if view_u8 else vcd
    ctx, meta = hip_attention_12(to_torch(XQ.q, "bf16"), None, None, args, cached_metadata=cached)
    torch.cuda.synchronize()
    return ctx, meta


def test_widening_is_exact_for_every_byte():
    # all 256 bit patterns through the decode kernel's loader would need a kernel of its own; the operator-level tests
    # below exercise every loader.  Here: the premise that e5m2 -> bf16 loses nothing (NaN patterns aside).
    b = torch.arange(256, dtype=torch.uint8)
    f8 = b.view(torch.float8_e5m2)
    wide = f8.to(torch.float32)
    ok = ~torch.isnan(wide)
    assert torch.equal(wide[ok].to(torch.bfloat16).to(torch.float32), wide[ok])


@pytest.mark.parametrize("D,view_u8", [(128, True), (64, False)])
def test_prefill_on_fp8_cache(D, view_u8):
    print(f"[case] fp8 prefill D={D}", flush=True)
    X = make_inputs(51, B=2, TQ=200, TK=2048, H=4, HKV=2, D=D, dtype="bf16", scale=0.5)
    XQ, kc, vc = _quantise(to_paged(X, 16, seed=8))
    A = tiny_args(extend_context_length=2048)
    octx, ometa = O.hip_attention_12(XQ, A)
    ctx, meta = _run(XQ, A, kc, vc, view_u8)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")


@pytest.mark.parametrize("D", [128, 64, 256])
def test_decode_on_fp8_cache(D):
    print(f"[case] fp8 decode D={D}", flush=True)
    lens = np.array([3000, 1500, 700])
    X = make_inputs(52, B=3, TQ=1, TK=3000, H=8, HKV=2, D=D, dtype="bf16", pos=(lens - 1)[:, None], scale=0.5)
    XQ, kc, vc = _quantise(to_paged(X, 16, seed=9, seq_lens=lens))
    A = tiny_args(extend_context_length=3072)
    octx, ometa = O.hip_attention_12(XQ, A)
    ctx, meta = _run(XQ, A, kc, vc, True)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    ctx2, _ = _run(XQ, A, kc, vc, True, cached=meta)
    assert_context_close(ctx2, octx, "bf16")


def test_fp8_cache_with_rope_on_load_and_softcap():
    print("[case] fp8 + rope + softcap", flush=True)
    X = make_inputs(53, B=1, TQ=96, TK=2048, H=4, HKV=1, D=128, dtype="bf16", scale=0.7)
    XP = with_rope(to_paged(X, 16, seed=10), 4096)
    XQ, kc, vc = _quantise(XP)
    for scan in ("relative", "streaming"):
        A = tiny_args(extend_context_length=2048, using_extend=True, need_apply_rope=True, scan_extend_backend=scan,
                      logit_softcap=5.0)
        octx, ometa = O.hip_attention_12(XQ, A)
        ctx, meta = _run(XQ, A, kc, vc, True)
        assert_metadata_equal(meta, ometa)
        assert_context_close(ctx, octx, "bf16")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("cap", [None, 20.0])
def test_fp8_cache_with_the_dynamic_rule_inside_attention(D, cap):
    """dynamic_extend inside attention on an fp8 cache (the tile kernel's and the decode kernel's variants that blend
    two table rows while they stage widened key rows), prefill and ragged decode, with and without soft-capping."""
    print(f"[case] fp8 + dynamic_extend attention D={D} softcap={cap}", flush=True)
    kw = dict(extend_context_length=3000, using_extend=True, need_apply_rope=True, scan_extend_backend="relative",
              sa_extend_backend="dynamic_extend", model_context_length=1024)
    if cap:
        kw["logit_softcap"] = cap
    X = make_inputs(57, B=2, TQ=100, TK=3000, H=4, HKV=2, D=D, dtype="bf16", scale=0.5)
    XQ, kc, vc = _quantise(with_rope(to_paged(X, 16, seed=12), 4096))
    A = tiny_args(**kw)
    octx, ometa = O.hip_attention_12(XQ, A)
    ctx, meta = _run(XQ, A, kc, vc, True)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    lens = np.array([3000, 1700])
    Xd = make_inputs(58, B=2, TQ=1, TK=3000, H=4, HKV=2, D=D, dtype="bf16", pos=(lens - 1)[:, None], scale=0.5)
    XQ, kc, vc = _quantise(with_rope(to_paged(Xd, 8, seed=13, seq_lens=lens), 4096))
    octx, ometa = O.hip_attention_12(XQ, A)
    ctx, meta = _run(XQ, A, kc, vc, False)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")


def test_portable_attention_kernel_on_fp8_cache():
    from hip_attn import HiPAttentionArgs12
    from hip_attn.operator import block_sparse_attention
    from test_oracle_bsa import random_indices

    print("[case] fp8 portable bsa", flush=True)
    rng = np.random.default_rng(3)
    TK, TQ, H, HKV, D, bq, bk, BK, sw, sink = 1024, 80, 4, 2, 64, 16, 8, 12, 48, 16
    X = make_inputs(54, B=2, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", scale=0.5)
    XQ, kc, vc = _quantise(to_paged(X, 8, seed=11))
    idx, ks, kse = random_indices(rng, 2, H, O.cdiv(TQ, bq), BK, bk, TK)
    ref = O.bsa(XQ, 1024, idx, kse, bq, bk, sw, sink)
    dev = "cuda"
    for impl in (1, 2):
        args = HiPAttentionArgs12(sink_token_size=sink, sliding_window_size=sw, k_cache=kc.cuda().view(torch.uint8),
                                  v_cache=vc.cuda().view(torch.uint8), block_table=torch.from_numpy(XQ.block_table).to(dev),
                                  cache_seq_lens=torch.from_numpy(XQ.cache_seq_lens).to(dev))
        args.block_size_q, args.block_size_k = bq, bk
        out = block_sparse_attention(to_torch(XQ.q, "bf16"), None, None, torch.from_numpy(XQ.pos.copy()).to(dev),
                                     torch.from_numpy(idx).to(dev), torch.from_numpy(kse).to(dev), args, 1024, impl=impl,
                                     rows_shared=True)
        torch.cuda.synchronize()
        assert_context_close(out, ref, "bf16")


@pytest.mark.parametrize("TQ,sa_tokens", [(1, 1 << 20), (96, 1 << 20), (1, 1024)])
def test_fp8_pools_behind_the_offload_cache(TQ, sa_tokens):
    """fp8 rows in pinned host pools behind the device block caches (``model_offload_cache.py:39-41``): the same
    kernels read the same bytes, so the offloaded run equals the resident fp8 run bit for bit, hit or miss, and both
    match the oracle on the widened values."""
    from hip_attn import HiPOffloadCache, hip_attention_12

    print(f"[case] fp8 offload TQ={TQ} sa_tokens={sa_tokens}", flush=True)
    B, TK, H, HKV, D = 2, 2048, 8, 2, 128
    lens = np.array([2048, 1500])
    pos = np.stack([np.arange(TQ) + l - TQ for l in lens])
    X = make_inputs(60 + TQ, B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=pos, scale=0.5)
    XQ, kc, vc = _quantise(to_paged(X, 1, seed=12, seq_lens=lens))
    A = O.OArgs(sliding_window_size=256, second_stage_k=512, extend_context_length=TK,
                stages=[O.OStage(64, 4, 64, None, 1), O.OStage(64, 4, 16, 1024, 1), O.OStage(64, 1, 8, 512, 1)])
    octx, ometa = O.hip_attention_12(XQ, A)
    ctx_res, meta_res = _run(XQ, A, kc, vc, True)
    assert_metadata_equal(meta_res, ometa)
    assert_context_close(ctx_res, octx, "bf16")

    rows = kc.shape[0]
    cache = HiPOffloadCache(0, rows, 1 << 20, sa_tokens, HKV, D, torch.float8_e5m2, torch.device("cuda"))
    assert cache.k_uvm.bank_cpu.dtype == torch.uint8
    table = torch.arange(rows, dtype=torch.int64)
    cache.set_kv_buffer(table, table.cuda(), kc[:, 0], vc[:, 0])  # float8_e5m2 rows from the host
    hits = 0
    for step in range(3):
        args = product_args(A, XQ)
        args.k_cache = args.v_cache = None
        args.offload_cache = cache
        ctx, meta = hip_attention_12(to_torch(XQ.q, "bf16"), None, None, args)
        torch.cuda.synchronize()
        assert_metadata_equal(meta, ometa)
        assert torch.equal(ctx.view(torch.int16), ctx_res.view(torch.int16)), f"step {step}: offloaded != resident"
        cache.handle_cache_miss(meta)
        hits += cache.sa_kv_cache.statistics()["last_hit"]
    assert hits > 0  # later steps were served from the device cache
    # rows written from the device in a wider dtype are rounded to e5m2 on the way in
    new = torch.randn((4, HKV, D), device="cuda", dtype=torch.bfloat16)
    at = torch.tensor([5, 6, 7, 8], device="cuda")
    cache.set_kv_buffer(at, at, new, new)
    torch.cuda.synchronize()
    assert torch.equal(cache.k_uvm.bank_cpu[5:9], new.to(torch.float8_e5m2).view(torch.uint8).cpu())
