"""GPU parity of RoPE applied on load (the "extend" modes): mask stage rules relative / streaming / infllm /
dynamic_extend / self_extend, sparse
attention rules streaming / infllm, through every kernel that loads query or key rows (scan on the matrix cores and
portable scan, tile kernel, portable attention kernel, decode kernel).

Indices must match the oracle bit for bit; outputs within 2e-2 abs / 1e-2 rel (bf16) or 1e-4 (f32).
"""
import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, tiny_args, to_paged, with_rope
from gpu_utils import assert_context_close, assert_metadata_equal, run_product, to_torch
from test_oracle_bsa import random_indices

pytestmark = pytest.mark.gpu


def _ext(**kw):
    return tiny_args(using_extend=True, need_apply_rope=True, **kw)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("scan", ["relative", "streaming", "infllm"])
def test_prefill_with_rope_matches_oracle(dtype, scan):
    print(f"[case] rope prefill {dtype} scan={scan}", flush=True)
    # ragged last query block, GQA, strided query mean in the first two stages
    X = with_rope(make_inputs(31, B=2, TQ=200, TK=2048, H=4, HKV=2, D=64, dtype=dtype, scale=0.5), 4096)
    A = _ext(scan_extend_backend=scan, sa_extend_backend="streaming")
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)


@pytest.mark.parametrize("dtype,D", [("f32", 64), ("bf16", 64), ("bf16", 128)])
@pytest.mark.parametrize("model_ctx", [1024, 131072])
def test_dynamic_extend_scan_prefill_and_paged_decode(dtype, D, model_ctx):
    """The dynamic_extend rule of the scan: queries beyond model_context_length squeeze the keys older than a quarter
    of it into the rest (1024 against 3000 keys); below it (131072) every key keeps its own position."""
    print(f"[case] rope dynamic_extend {dtype} D={D} model_ctx={model_ctx}", flush=True)
    X = with_rope(make_inputs(51, B=2, TQ=200, TK=3000, H=4, HKV=2, D=D, dtype=dtype, scale=0.5), 4096)
    A = _ext(scan_extend_backend="dynamic_extend", sa_extend_backend="streaming", model_context_length=model_ctx)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)
    if model_ctx == 1024:  # the squeeze really changes what is selected
        _, plain = O.hip_attention_12(X, _ext(scan_extend_backend="dynamic_extend", sa_extend_backend="streaming"))
        assert not np.array_equal(plain.indices, ometa.indices)
    lens = np.array([3000, 1777])
    XD = make_inputs(52, B=2, TQ=1, TK=3000, H=4, HKV=2, D=D, dtype=dtype, pos=(lens - 1)[:, None], scale=0.5)
    XP = with_rope(to_paged(XD, 16, seed=5, seq_lens=lens), 4096)
    A = _ext(scan_extend_backend="dynamic_extend", sa_extend_backend="infllm", model_context_length=model_ctx,
             extend_context_length=3072)
    octx, ometa = O.hip_attention_12(XP, A)
    ctx, meta = run_product(XP, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)


@pytest.mark.parametrize("D", [64, 128])
def test_prefill_with_rope_paged_bf16_default_like_stages(D):
    print(f"[case] rope prefill paged D={D}", flush=True)
    X = with_rope(make_inputs(32, B=1, TQ=256, TK=4096, H=8, HKV=2, D=D, dtype="bf16", scale=0.5), 8192)
    XP = with_rope(to_paged(X, 16, seed=4), 8192)
    A = _ext(scan_extend_backend="relative", sa_extend_backend="streaming", extend_context_length=4096,
             sliding_window_size=512, second_stage_k=1024, block_sparse_block_size_q=64,
             stages=[O.OStage(64, 4, 256, None, 1), O.OStage(64, 4, 32, 2048, 1, "streaming"), O.OStage(64, 1, 8, 1024, 1)])
    octx, ometa = O.hip_attention_12(XP, A)
    ctx, meta = run_product(XP, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("sa", ["streaming", "infllm"])
def test_batched_paged_decode_with_rope(dtype, sa):
    print(f"[case] rope decode {dtype} sa={sa}", flush=True)
    B, TK, H, HKV, D = 3, 3000, 8, 2, 128 if dtype == "bf16" else 64
    lens = np.array([3000, 1777, 900])
    X = make_inputs(33, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, pos=(lens - 1)[:, None], scale=0.5)
    XP = with_rope(to_paged(X, 16, seed=5, seq_lens=lens), 4096)
    A = _ext(scan_extend_backend="relative", sa_extend_backend=sa, extend_context_length=3072)
    octx, ometa = O.hip_attention_12(XP, A)
    ctx, meta = run_product(XP, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)
    # cached mask: attention only
    octx2, _ = O.hip_attention_12(XP, A, cached=O.OMetadata(ometa.indices, ometa.ks, ometa.ks_count, ometa.ks_start_end, None))
    ctx2, _ = run_product(XP, A, cached=meta)
    assert_context_close(ctx2, octx2, dtype)


@pytest.mark.parametrize("D,G", [(128, 8), (128, 6), (64, 8), (128, 3)])
def test_decode_with_rope_and_wide_groups(D, G):
    """Groups of more heads than one pass of the decode kernel's query preparation holds (head dim 128: four), of as
    many (head dim 64: eight), and of a number that does not divide a pass."""
    print(f"[case] rope decode D={D} G={G}", flush=True)
    B, TK, HKV = 2, 2500, 2
    lens = np.array([2500, 1300])
    X = make_inputs(37, B=B, TQ=1, TK=TK, H=HKV * G, HKV=HKV, D=D, dtype="bf16", pos=(lens - 1)[:, None], scale=0.5)
    XP = with_rope(to_paged(X, 16, seed=6, seq_lens=lens), 4096)
    A = _ext(scan_extend_backend="relative", sa_extend_backend="streaming", extend_context_length=3072)
    octx, ometa = O.hip_attention_12(XP, A)
    ctx, meta = run_product(XP, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    octx2, _ = O.hip_attention_12(XP, A, cached=O.OMetadata(ometa.indices, ometa.ks, ometa.ks_count, ometa.ks_start_end, None))
    ctx2, _ = run_product(XP, A, cached=meta)
    assert_context_close(ctx2, octx2, "bf16")


def _run_bsa(X, max_tsrc, idx, kse, bq, bk, sw, sink, impl, backend, share=True, decode=False):
    from hip_attn import HiPAttentionArgs12
    from hip_attn.operator import block_sparse_attention

    dev = "cuda"
    bits = (lambda a: O.f32_to_bf16_bits(a)) if X.dtype == "bf16" else (lambda a: a)
    args = HiPAttentionArgs12(sink_token_size=sink, sliding_window_size=sw, sa_extend_backend=backend)
    args.block_size_q, args.block_size_k = bq, bk
    tabs = (to_torch(bits(X.rope_cos), X.dtype, dev), to_torch(bits(X.rope_sin), X.dtype, dev))
    out = block_sparse_attention(to_torch(X.q, X.dtype, dev), to_torch(X.k, X.dtype, dev), to_torch(X.v, X.dtype, dev),
                                 torch.from_numpy(X.pos.copy()).to(dev), torch.from_numpy(idx).to(dev),
                                 torch.from_numpy(kse).to(dev), args, max_tsrc, decode=decode, impl=impl,
                                 rows_shared=share, rope_tables=tabs)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("backend", ["streaming", "infllm"])
@pytest.mark.parametrize("D,bq,TQ,bk", [(64, 64, 200, 8), (128, 32, 96, 2), (128, 16, 40, 16), (256, 64, 100, 8)])
def test_attention_kernels_with_rope_given_indices(backend, D, bq, TQ, bk):
    print(f"[case] rope bsa {backend} D={D} bq={bq} TQ={TQ} bk={bk}", flush=True)
    rng = np.random.default_rng(D + bq + bk)
    TK, H, HKV, BK, sw, sink = 1536, 8, 2, 24, 100, 32
    X = with_rope(make_inputs(34, B=2, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", scale=0.5), 2048,
                  sa_backend=backend)
    idx, ks, kse = random_indices(rng, 2, H, O.cdiv(TQ, bq), BK, bk, TK, same_heads=True)
    ref = O.bsa(X, TK, idx, kse, bq, bk, sw, sink)
    assert_context_close(_run_bsa(X, TK, idx, kse, bq, bk, sw, sink, 2, backend), ref, "bf16")
    assert_context_close(_run_bsa(X, TK, idx, kse, bq, bk, sw, sink, 1, backend), ref, "bf16")


def test_float32_tables_with_bf16_queries_are_cast_like_the_reference():
    print("[case] rope f32 tables, bf16 q", flush=True)
    # tables handed over in float32 (and as [1, L, D]): entries are cast to the query dtype on use
    X = with_rope(make_inputs(35, B=1, TQ=64, TK=1024, H=2, HKV=1, D=64, dtype="bf16", scale=0.5), 2048, dtype="f32")
    A = _ext(scan_extend_backend="relative", sa_extend_backend="streaming")
    cos32 = torch.from_numpy(X.rope_cos.copy()).cuda()[None]
    sin32 = torch.from_numpy(X.rope_sin.copy()).cuda()[None]
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A, rope_cos=cos32, rope_sin=sin32)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")


@pytest.mark.parametrize("dtype,D", [("f32", 64), ("bf16", 64), ("bf16", 128)])
@pytest.mark.parametrize("model_ctx", [1024, 131072])
def test_dynamic_extend_inside_attention_prefill_and_paged_decode(dtype, D, model_ctx):
    """The dynamic_extend rule of block sparse attention: sink and selected keys are rotated with 0.75 of the table row
    of their streaming position and 0.25 of the row of their own position squeezed into the model's context
    (attention_extend_bsa.py:271-292, :323-357).  With model_ctx = 1024 the 3000-token context reaches beyond the
    model's and the squeeze is active; with 131072 the second row is the key's own position."""
    print(f"[case] rope dynamic_extend in attention {dtype} D={D} model_ctx={model_ctx}", flush=True)
    X = with_rope(make_inputs(51, B=2, TQ=100, TK=3000, H=4, HKV=2, D=D, dtype=dtype, scale=0.5), 4096)
    A = _ext(scan_extend_backend="relative", sa_extend_backend="dynamic_extend", model_context_length=model_ctx)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)
    ref_stream, _ = O.hip_attention_12(X, _ext(scan_extend_backend="relative", sa_extend_backend="streaming"))
    widen = O.bf16_bits_to_f32 if dtype == "bf16" else (lambda a: a)
    assert np.abs(widen(octx) - widen(ref_stream)).max() > 0.05  # the rule really changes the result
    lens = np.array([3000, 1400])
    Xd = make_inputs(52, B=2, TQ=1, TK=3000, H=4, HKV=2, D=D, dtype=dtype, pos=(lens - 1)[:, None], scale=0.5)
    XP = with_rope(to_paged(Xd, 8, seed=9, seq_lens=lens), 4096)
    A = _ext(scan_extend_backend="streaming", sa_extend_backend="dynamic_extend", model_context_length=model_ctx,
             extend_context_length=3000)
    octx, ometa = O.hip_attention_12(XP, A)
    ctx, meta = run_product(XP, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)


@pytest.mark.parametrize("dtype,D", [("f32", 64), ("bf16", 64), ("bf16", 128)])
@pytest.mark.parametrize("model_ctx", [4096, 131072])
def test_self_extend_scan_prefill_and_paged_decode(dtype, D, model_ctx):
    """The self_extend rule of the scan (attention_extend.py:275-289): once a query block reaches beyond the model's
    context (4096 against 9000 keys), keys older than 8192 positions are grouped by sixteen; below it (131072) every
    key keeps its own position.  The oracle's rule is pinned by the closed form in tests/test_oracle_rope.py and by
    an execution of the reference (tests/golden/reference_f32_prefill_rope_self_extend.npz)."""
    print(f"[case] rope self_extend {dtype} D={D} model_ctx={model_ctx}", flush=True)
    X = with_rope(make_inputs(61, B=1, TQ=200, TK=9000, H=4, HKV=2, D=D, dtype=dtype, scale=0.5), 9216)
    A = _ext(scan_extend_backend="self_extend", sa_extend_backend="streaming", model_context_length=model_ctx)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)
    if model_ctx == 4096:  # the grouping really changes what is selected
        _, plain = O.hip_attention_12(X, _ext(scan_extend_backend="self_extend", sa_extend_backend="streaming"))
        assert not np.array_equal(plain.indices, ometa.indices)
    lens = np.array([9000, 8800])
    XD = make_inputs(62, B=2, TQ=1, TK=9000, H=4, HKV=2, D=D, dtype=dtype, pos=(lens - 1)[:, None], scale=0.5)
    XP = with_rope(to_paged(XD, 16, seed=5, seq_lens=lens), 9216)
    A = _ext(scan_extend_backend="self_extend", sa_extend_backend="infllm", model_context_length=model_ctx,
             extend_context_length=9008)
    octx, ometa = O.hip_attention_12(XP, A)
    ctx, meta = run_product(XP, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)


def test_unbuilt_rules_fail_loudly():
    from hip_attn import _native as N
    print("[case] rope unbuilt rules", flush=True)
    X = with_rope(make_inputs(36, B=1, TQ=32, TK=512, H=2, HKV=1, D=32, dtype="f32"), 1024)
    with pytest.raises(NotImplementedError):  # the reference's attention kernels raise on these two as well
        run_product(X, _ext(sa_extend_backend="self_extend"))
    with pytest.raises(NotImplementedError):
        run_product(X, _ext(sa_extend_backend="relative"))
    with pytest.raises(N.HipAttnError):  # the squeeze divides by pmin - model_context_length / 4: tiny lengths are refused
        run_product(X, _ext(scan_extend_backend="dynamic_extend", model_context_length=64))
    with pytest.raises(NotImplementedError):
        run_product(X, tiny_args(using_extend=True, need_apply_rope=False))


@pytest.mark.parametrize("scan", ["relative", "infllm"])
@pytest.mark.parametrize("force", ["0", "1"])
def test_keys_rotated_and_scaled_ahead_give_identical_masks(scan, force, monkeypatch):
    """relative / infllm rotate sampled keys to position 0 or 1 whatever the token: rotating and scaling the whole
    key tensor once per position must give the same mask as rotating every sample (one stage keeps the streaming
    rule, which cannot be prepared ahead, to cover the mix)."""
    print(f"[case] rope prescaled scan={scan} force={force}", flush=True)
    monkeypatch.setenv("HIP_ATTN_PRESCALE_K", force)
    X = with_rope(make_inputs(37, B=2, TQ=200, TK=2048, H=4, HKV=2, D=64, dtype="bf16", scale=0.5), 4096)
    A = _ext(scan_extend_backend=scan, sa_extend_backend="streaming",
             stages=[O.OStage(32, 2, 64, None, 1), O.OStage(32, 2, 16, 2048, 1, "streaming"), O.OStage(32, 1, 2, 1024, 1)])
    octx, ometa = O.hip_attention_12(X, A)
    for XX in (X, with_rope(to_paged(X, 16, seed=6), 4096)):
        AA = A if XX is X else O.OArgs(**{**A.__dict__, "extend_context_length": 2048})
        ctx, meta = run_product(XX, AA)
        assert np.array_equal(meta.indices.cpu().numpy(), ometa.indices)
        assert_context_close(ctx, octx, "bf16")


def test_keys_rotated_to_the_place_of_their_chunk():
    """hipattn_prescale_k_rope_chunks: every key row rotated to (t - first) // chunk, clamped into the tables, and
    scaled, against the oracle's row rotation followed by its scaling."""
    import torch
    from hip_attn import _native as N
    from gpu_utils import to_torch

    print("[case] keys rotated to the place of their chunk", flush=True)
    B, T, HKV, D, first, chunk, table_len = 2, 300, 2, 64, 16, 64, 4
    X = with_rope(make_inputs(71, B=B, TQ=8, TK=T, H=HKV, HKV=HKV, D=D, dtype="bf16", scale=0.7), table_len,
                  scan_backend="relative")
    k = to_torch(X.k, "bf16")
    cos = torch.from_numpy(X.rope_cos).to(torch.bfloat16).cuda().contiguous()
    sin = torch.from_numpy(X.rope_sin).to(torch.bfloat16).cuda().contiguous()
    out = N.prescale_k_rope_chunks(k, cos, sin, first, chunk, k.device)
    torch.cuda.synchronize()
    got = out.view(torch.int16).cpu().numpy().view(np.uint16)
    _, ck = O.scale_constants(D, "bf16")
    kf = O.bf16_bits_to_f32(X.k)
    for b in range(B):
        for t in (0, 15, 16, 79, 80, 143, 271, 272, 299):   # below `first`, chunk edges, beyond the table (clamped)
            pos = min((t - first) // chunk if t >= first else 0, table_len - 1)
            for h in range(HKV):
                rot = O.rope_row(X, kf[b, t, h], pos)
                want = O.f32_to_bf16_bits((rot * np.float32(ck)).astype(np.float32))
                assert np.array_equal(got[b, t, h], want), (b, t, h)

