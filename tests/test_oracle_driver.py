"""Pins the oracle's stage glue, selection and metadata layout (attention_extend.py:2058-2165,2710-2728,2906-2924)."""
import copy

import numpy as np

from oracle import hip12 as O
from helpers import make_inputs, tiny_args, to_paged, widen


def test_topk_order_is_score_desc_position_asc():
    rng = np.random.default_rng(0)
    s = rng.integers(0, 5, size=(3, 40)).astype(np.float32)  # many ties
    got = O.topk_order(s, 17)
    for r in range(3):
        ref = np.lexsort((np.arange(40), -s[r]))[:17]
        assert np.array_equal(got[r], ref)


def test_single_stage_chunk2_selection_equals_brute_force():
    # one stage, chunk size 2, stride_q 1: every token of an active chunk is scored, so the selected set
    # is maxpool(chunk) -> max over heads -> top-k over chunks that start at or before p_min - sw'
    X = make_inputs(1, B=1, TQ=32, TK=256, H=4, HKV=2, D=32, dtype="f32")
    sink, sw, K = 4, 8, 40
    A = O.OArgs(sink_token_size=sink, sliding_window_size=sw, second_stage_k=K, block_sparse_block_size_q=16,
                stages=[O.OStage(16, 1, 2, None, 1)])
    _, meta = O.hip_attention_12(X, A)
    cq, ck = O.scale_constants(32, "f32")
    qh = (X.q * np.float32(cq)).astype(np.float32); kh = (X.k * np.float32(ck)).astype(np.float32)
    L = O.lib()
    n = O.cdiv(256 - sink - sw, 2)
    sw_eff = max(0, sw - 2)
    for qb in range(2):
        pmin = int(X.pos[0, qb * 16])
        sc = np.full(n, -32000.0, dtype=np.float32)
        for c in range(n):
            cl = sink + 2 * c
            if cl > pmin - sw_eff:
                continue
            best = -np.inf
            for t in (cl, cl + 1):
                if t >= 256 - sw_eff:
                    continue
                for h in range(4):
                    for r in range(qb * 16, qb * 16 + 16):
                        a = np.ascontiguousarray(qh[0, r, h]); b = np.ascontiguousarray(kh[0, t, h // 2])
                        best = max(best, L.hipo_dot(a.ctypes.data, b.ctypes.data, 32))
            sc[c] = best
        order = np.lexsort((np.arange(n), -sc))[: K // 2]
        want = np.sort(sink + 2 * order) // 2 * 2
        want = want[want < pmin + 16]
        for h in range(4):
            ks = int(meta.ks[h, qb])
            assert ks == len(want)
            assert np.array_equal(meta.indices[h, qb, :ks], want)


def _check_layout(meta, X, A, B, H):
    bk = A.stages[-1].stage_chunk_size
    bq = A.stages[-1].stage_block_size_q
    idx, ks = meta.indices, meta.ks
    assert idx.dtype == np.int64 and ks.dtype == np.int64 and meta.ks_start_end.dtype == np.int32
    assert np.array_equal(meta.ks_count, ks[..., None])
    assert (meta.ks_start_end[..., 0] == 0).all() and np.array_equal(meta.ks_start_end[..., 1], ks)
    first = np.repeat(X.pos[:, ::bq], H, axis=0)
    for r in range(idx.shape[0]):
        for qb in range(idx.shape[1]):
            row = idx[r, qb]; n = int(ks[r, qb])
            act = row[:n]
            assert (np.diff(act) > 0).all() and (act % bk == 0).all()
            assert (act < first[r, qb] + bq).all() and (row[n:] >= first[r, qb] + bq).all()
            real = row[row != O.INT64_MAX]
            assert (np.diff(real) > 0).all()
    per_head = idx.reshape(B, H, *idx.shape[1:])
    assert all(np.array_equal(per_head[:, 0], per_head[:, h]) for h in range(H))


def test_metadata_layout_invariants_dense_and_paged():
    X = make_inputs(0, B=2, TQ=96, TK=1024, H=4, HKV=2, D=32, dtype="bf16")
    A = tiny_args(sliding_window_size=128, second_stage_k=128)
    _, meta = O.hip_attention_12(X, A)
    assert meta.indices.shape == (8, 3, 64)
    _check_layout(meta, X, A, 2, 4)
    # paged with the same tokens and extend_context_length == TK selects the same blocks
    XP = to_paged(X, 8, seed=2)
    A2 = copy.deepcopy(A); A2.extend_context_length = 1024
    ctx_d, _ = O.hip_attention_12(X, A)
    ctx_p, meta_p = O.hip_attention_12(XP, A2)
    assert np.array_equal(meta.indices, meta_p.indices) and np.array_equal(meta.ks, meta_p.ks)
    assert np.array_equal(ctx_d, ctx_p)


def test_stage_cache_replay_and_cached_indices_reuse():
    # reference invariant: restarting from stage_caches[:i+1] reproduces the result
    # (tests/v1_2/test_gen3_stage_caching.py:166-186); passing indices skips estimation entirely
    X = make_inputs(2, B=1, TQ=64, TK=2048, H=4, HKV=1, D=32, dtype="f32")
    A = tiny_args()
    ctx, meta = O.hip_attention_12(X, A)
    assert len(meta.stage_caches) == 3 and meta.stage_caches[0].indices_left is None
    for i in range(3):
        part = O.OMetadata(None, None, None, None, stage_caches=list(meta.stage_caches[: i + 1]))
        ctx_i, meta_i = O.hip_attention_12(X, A, cached=part)
        assert np.array_equal(meta_i.indices, meta.indices) and np.array_equal(ctx_i, ctx)
        assert len(part.stage_caches) == 3  # appended to in place
    ctx_c, meta_c = O.hip_attention_12(X, A, cached=meta)
    assert np.array_equal(meta_c.indices, meta.indices)
    # cached path uses block_size_q = 64 while the fresh path used 32: same attended sets here because
    # indices rows are identical per 32-row block?  No -- rows differ, so only compare with a matching layout
    A64 = tiny_args(block_sparse_block_size_q=64,
                    stages=[O.OStage(64, 2, 64, None, 1), O.OStage(64, 2, 16, 2048, 1), O.OStage(64, 1, 2, 1024, 1)])
    ctx64, meta64 = O.hip_attention_12(X, A64)
    ctx64c, _ = O.hip_attention_12(X, A64, cached=meta64)
    assert np.array_equal(ctx64, ctx64c)


def test_decode_shape_and_flashdecode_head_sharing_is_neutral_under_head_reduce():
    X = make_inputs(3, B=3, TQ=1, TK=1500, H=4, HKV=2, D=32, dtype="bf16",
                    pos=np.array([[1499], [700], [1200]]))
    # window 256: the decode kernel's 2 programs take 16 index entries each, a whole number of their tiles of 8
    A = tiny_args(sliding_window_size=256, second_stage_k=64)
    assert O.decode_seams(64, A.sink_token_size, 256, 2, 32) == (16, 0)
    ctx, meta = O.hip_attention_12(X, A)
    assert meta.indices.shape == (12, 1, 32) and ctx.shape == (3, 1, 4, 32)
    A.disable_flashdecode = True
    ctx2, meta2 = O.hip_attention_12(X, A)
    assert np.array_equal(meta.indices, meta2.indices) and np.array_equal(ctx, ctx2)
    # window 128: 3 programs of 11 entries, each walking 16: five entries per seam are attended twice, and the
    # decode kernel's output departs from the query-block kernel's
    A = tiny_args(sliding_window_size=128, second_stage_k=64)
    assert O.decode_seams(64, A.sink_token_size, 128, 2, 32) == (11, 5)
    ctx, meta = O.hip_attention_12(X, A)
    A.disable_flashdecode = True
    ctx2, meta2 = O.hip_attention_12(X, A)
    assert np.array_equal(meta.indices, meta2.indices)
    assert np.abs(O.bf16_bits_to_f32(ctx) - O.bf16_bits_to_f32(ctx2)).max() > 0.02


def test_restart_at_a_stage_with_another_block_size_is_refused():
    import pytest

    X = make_inputs(2, B=1, TQ=128, TK=2048, H=2, HKV=1, D=32, dtype="f32")
    A = tiny_args(stages=[O.OStage(64, 2, 64, None, 1), O.OStage(32, 2, 16, 1024, 1), O.OStage(32, 1, 2, 1024, 1)])
    ctx, meta = O.hip_attention_12(X, A)
    part = O.OMetadata(None, None, None, None, stage_caches=list(meta.stage_caches[:2]))
    with pytest.raises(NotImplementedError):
        O.hip_attention_12(X, A, cached=part)
