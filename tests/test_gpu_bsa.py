"""GPU parity of the block-sparse attention kernels given indices (tile kernel, portable kernel, decode)."""
import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, to_paged
from gpu_utils import assert_context_close, to_torch
from test_oracle_bsa import random_indices

pytestmark = pytest.mark.gpu


def _run(X, max_tsrc, idx, kse, bq, bk, sw, sink, impl, share=False, decode=False, softcap=None, second_k=0,
         causal=True):
    from hip_attn import HiPAttentionArgs12
    from hip_attn.operator import block_sparse_attention

    dev = "cuda"
    q = to_torch(X.q, X.dtype, dev)
    kw = {}
    if X.k is None:
        kw = dict(k_cache=to_torch(X.k_cache, X.dtype, dev), v_cache=to_torch(X.v_cache, X.dtype, dev),
                  block_table=torch.from_numpy(X.block_table).to(dev),
                  cache_seq_lens=torch.from_numpy(X.cache_seq_lens).to(dev))
    args = HiPAttentionArgs12(sink_token_size=sink, sliding_window_size=sw, logit_softcap=softcap, is_causal=causal, **kw)
    args.block_size_q, args.block_size_k = bq, bk
    args.second_stage_k = second_k  # decode only: sizes the reference's own split of the index row
    out = block_sparse_attention(q, to_torch(X.k, X.dtype, dev), to_torch(X.v, X.dtype, dev),
                                 torch.from_numpy(X.pos.copy()).to(dev), torch.from_numpy(idx).to(dev),
                                 torch.from_numpy(kse).to(dev), args, max_tsrc, decode=decode, impl=impl,
                                 rows_shared=share)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("bq,TQ,bk", [(64, 200, 8), (32, 96, 2), (16, 40, 16)])
@pytest.mark.parametrize("paged", [False, True])
def test_tile_kernel_matches_oracle_and_portable_kernel(D, bq, TQ, bk, paged):
    print(f"[case] bsa mfma D={D} bq={bq} TQ={TQ} bk={bk} paged={paged}", flush=True)
    rng = np.random.default_rng(D + bq + bk)
    TK, H, HKV, BK, sw, sink = 1536, 8, 2, 24, 100, 24
    X = make_inputs(12, B=2, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", scale=0.5)
    nbq = O.cdiv(TQ, bq)
    idx, ks, kse = random_indices(rng, 2, H, nbq, BK, bk, TK, same_heads=True)
    max_tsrc = TK
    if paged:
        X = to_paged(X, 16, seed=7)
        max_tsrc = 4096
    ref = O.bsa(X, max_tsrc, idx, kse, bq, bk, sw, sink)
    out_tile = _run(X, max_tsrc, idx, kse, bq, bk, sw, sink, impl=2, share=True)
    out_port = _run(X, max_tsrc, idx, kse, bq, bk, sw, sink, impl=1, share=True)
    assert_context_close(out_tile, ref, "bf16")
    assert_context_close(out_port, ref, "bf16")


def test_tile_kernel_per_head_rows():
    print("[case] bsa mfma per-head rows", flush=True)
    rng = np.random.default_rng(5)
    TK, TQ, H, HKV, D, bq, bk, BK, sw, sink = 1024, 128, 8, 2, 128, 64, 8, 20, 64, 16
    X = make_inputs(13, B=1, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", scale=0.5)
    idx, ks, kse = random_indices(rng, 1, H, 2, BK, bk, TK, same_heads=False)
    ref = O.bsa(X, TK, idx, kse, bq, bk, sw, sink)
    out = _run(X, TK, idx, kse, bq, bk, sw, sink, impl=2, share=False)
    assert_context_close(out, ref, "bf16")
    ref_shared = O.bsa(X, TK, idx, kse, bq, bk, sw, sink, share_first_head=True)
    out_shared = _run(X, TK, idx, kse, bq, bk, sw, sink, impl=2, share=True)
    assert_context_close(out_shared, ref_shared, "bf16")


def test_tile_kernel_empty_rows_and_early_positions():
    print("[case] bsa mfma early positions", flush=True)
    # queries at the very start of the sequence: window and sink are clipped by the position, ks = 0
    X = make_inputs(14, B=1, TQ=64, TK=64, H=4, HKV=1, D=64, dtype="bf16", scale=0.5)
    idx = np.full((4, 1, 4), O.INT64_MAX, dtype=np.int64)
    kse = np.zeros((4, 1, 2), dtype=np.int32)
    ref = O.bsa(X, 64, idx, kse, 64, 8, 16, 4)
    out = _run(X, 64, idx, kse, 64, 8, 16, 4, impl=2, share=True)
    assert_context_close(out, ref, "bf16")


@pytest.mark.parametrize("second_k", [0, 320, 2048])
@pytest.mark.parametrize("dtype,D,G", [("bf16", 128, 4), ("bf16", 64, 2), ("f32", 64, 4), ("bf16", 128, 1)])
def test_decode_kernel_matches_oracle(dtype, D, G, second_k):
    """``second_k`` 0: every selected block once; 320: the reference's programs take 8 index entries each in tiles
    of 2, no seams; 2048: 5 entries each, so the first entry of every later share is attended twice."""
    print(f"[case] decode {dtype} D={D} G={G} second_k={second_k}", flush=True)
    rng = np.random.default_rng(D + G)
    B, HKV, TK, bk, BK, sw, sink = 3, 2, 3000, 8, 40, 200, 32
    H = HKV * G
    lens = np.array([3000, 1500, 257])
    X = make_inputs(15, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=0.5, pos=(lens - 1)[:, None])
    idx, ks, kse = random_indices(rng, B, H, 1, BK, bk, 1400, same_heads=True)
    seams = O.decode_seams(second_k, sink, sw, bk, BK) if second_k else (0, 0)
    assert seams == {0: (0, 0), 320: (8, 0), 2048: (5, 1)}[second_k]
    ref = O.bsa(X, TK, idx, kse, 1, bk, sw, sink, share_first_head=True, seams=seams)
    out = _run(X, TK, idx, kse, 1, bk, sw, sink, impl=0, decode=True, second_k=second_k)
    assert_context_close(out, ref, dtype)
    if seams[1]:
        once = O.bsa(X, TK, idx, kse, 1, bk, sw, sink, share_first_head=True)
        w = (lambda a: O.bf16_bits_to_f32(a)) if dtype == "bf16" else (lambda a: a)
        assert np.abs(w(ref) - w(once)).max() > 0.025  # the seams matter on this input


@pytest.mark.parametrize("dtype,D", [("bf16", 128), ("bf16", 64), ("f32", 64)])
def test_logit_softcap_in_every_attention_kernel(dtype, D):
    print(f"[case] bsa softcap {dtype} D={D}", flush=True)
    rng = np.random.default_rng(D)
    TK, TQ, H, HKV, bq, bk, BK, sw, sink = 1024, 96, 8, 2, 32, 8, 16, 64, 16
    X = make_inputs(42, B=2, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=1.5)
    X.logit_softcap = 3.0
    idx, ks, kse = random_indices(rng, 2, H, O.cdiv(TQ, bq), BK, bk, TK, same_heads=True)
    ref = O.bsa(X, TK, idx, kse, bq, bk, sw, sink)
    uncapped = O.OInputs(X.dtype, X.q, X.pos, k=X.k, v=X.v)
    assert np.abs(O.bf16_bits_to_f32(ref) - O.bf16_bits_to_f32(O.bsa(uncapped, TK, idx, kse, bq, bk, sw, sink))).max() > 0.05 \
        if dtype == "bf16" else True
    assert_context_close(_run(X, TK, idx, kse, bq, bk, sw, sink, impl=1, share=True, softcap=3.0), ref, dtype)
    if dtype == "bf16":
        assert_context_close(_run(X, TK, idx, kse, bq, bk, sw, sink, impl=2, share=True, softcap=3.0), ref, dtype)
    # decode: one query at the end of each sequence
    Xd = make_inputs(43, B=2, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=1.5)
    Xd.logit_softcap = 3.0
    idx, ks, kse = random_indices(rng, 2, H, 1, BK, bk, TK, same_heads=True)
    ref = O.bsa(Xd, TK, idx, kse, 1, bk, sw, sink, share_first_head=True)
    assert_context_close(_run(Xd, TK, idx, kse, 1, bk, sw, sink, impl=0, decode=True, softcap=3.0), ref, dtype)


@pytest.mark.parametrize("dtype,D", [("bf16", 64), ("bf16", 128), ("bf16", 256), ("f32", 64)])
def test_non_causal_attention_in_every_kernel(dtype, D):
    """is_causal = False (attention_extend_bsa.py:511-523, :743-752): the mask keeps validity only; the query-block
    kernels put every row at the end of the keys, the decode kernels keep the row's position.  Blocks selected inside
    the last window are attended twice, by the kernels as by the oracle."""
    print(f"[case] bsa non-causal {dtype} D={D}", flush=True)
    rng = np.random.default_rng(D)
    TK, TQ, H, HKV, bq, bk, BK, sw, sink = 1536, 200, 8, 2, 64, 8, 24, 100, 24
    X = make_inputs(15, B=2, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=0.5)
    nbq = O.cdiv(TQ, bq)
    idx, ks, kse = random_indices(rng, 2, H, nbq, BK, bk, TK, same_heads=True)
    idx[:, :, 0] = 64  # one early block, and one inside the last sw + bq tokens
    idx[:, :, 1] = TK - 96
    idx[:, :, 2:] = O.INT64_MAX
    kse[..., 1] = 2
    X.non_causal = 1
    ref = O.bsa(X, TK, idx, kse, bq, bk, sw, sink)
    X.non_causal = 0
    assert np.abs(widen_any(ref, dtype) - widen_any(O.bsa(X, TK, idx, kse, bq, bk, sw, sink), dtype)).max() > 1e-2
    impls = (2, 1) if dtype == "bf16" else (1,)
    for impl in impls:
        out = _run(X, TK, idx, kse, bq, bk, sw, sink, impl=impl, share=True, causal=False)
        assert_context_close(out, ref, dtype)
    # decode: one query token per sequence, true positions kept
    lens = np.array([TK, 1000])
    XD = make_inputs(16, B=2, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, pos=(lens - 1)[:, None], scale=0.5)
    XP = to_paged(XD, 16, seed=3, seq_lens=lens)
    idx, ks, kse = random_indices(rng, 2, H, 1, BK, bk, 900, same_heads=True)
    XP.non_causal = 2
    ref = O.bsa(XP, 2048, idx, kse, 1, bk, sw, sink, share_first_head=True)
    XP.non_causal = 0
    out = _run(XP, 2048, idx, kse, 1, bk, sw, sink, impl=0, decode=True, causal=False)
    assert_context_close(out, ref, dtype)


def widen_any(a, dtype):
    return O.bf16_bits_to_f32(a) if dtype == "bf16" else a
