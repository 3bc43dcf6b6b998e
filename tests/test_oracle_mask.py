"""Pins hipo_mask_stage: lane-literal Python form, brute force for chunk sizes 1 and 2, invariants."""
import numpy as np
import pytest

from oracle import hip12 as O
from oracle import literal
from helpers import make_inputs, to_paged, widen


def _stage0(X, max_tsrc, sink, sw_eff, sw_orig, chunk, BQ, scan_stride=1):
    B, TDST, HEAD, _ = X.q.shape
    BDST = O.cdiv(TDST, BQ)
    BS = O.cdiv(BDST, scan_stride)
    n = O.cdiv(max(0, max_tsrc - sink - sw_orig), chunk)
    left = np.zeros((B, BS, HEAD, n), dtype=np.int64)
    left[...] = sink + np.arange(n) * chunk
    right = np.minimum(left + chunk, max_tsrc - sw_eff)
    scores = np.full((B, BS, HEAD, O.npow2(n)), -32000.0, dtype=np.float32)
    return left, right, scores


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("paged", [False, True])
def test_c_oracle_equals_lane_literal(dtype, paged):
    # ragged TDST (50 rows, BQ 16), strided query mean, two heads per kv head, ragged last chunk (sw_eff=0)
    X = make_inputs(3, B=2, TQ=50, TK=300, H=4, HKV=2, D=32, dtype=dtype)
    max_tsrc = 300
    if paged:
        X = to_paged(X, page_size=4, seed=1)
        max_tsrc = 320
    for (chunk, sw_orig, sw_eff, stride_q, scan_stride, bc) in [(32, 20, 0, 2, 1, 16), (16, 64, 48, 4, 2, 16), (8, 8, 0, 1, 1, 32)]:
        l0, r0, s0 = _stage0(X, max_tsrc, 4, sw_eff, sw_orig, chunk, 16, scan_stride)
        l1, r1, s1 = l0.copy(), r0.copy(), s0.copy()
        O.mask_stage(X, max_tsrc, l0, r0, s0, BS=l0.shape[1], BQ=16, stride_q=stride_q, block_chunk=bc,
                     scan_stride=scan_stride, sw_eff=sw_eff)
        literal.mask_stage(X, max_tsrc, l1, r1, s1, BQ=16, stride_q=stride_q, block_chunk=bc,
                           scan_stride=scan_stride, sw_eff=sw_eff)
        assert np.array_equal(l0, l1) and np.array_equal(r0, r1)
        assert np.array_equal(s0.view(np.uint32), s1.view(np.uint32))
        assert (s0 > -32000).any()


def _brute_scores(X, chunk_lefts, chunk, BQ, qb):
    """max over rows of q^.k^ for every token, max-pooled over each chunk (float64 dot, rounded like T)."""
    cq, ck = O.scale_constants(X.q.shape[-1], X.dtype)
    q = widen(X.q, X.dtype); k = widen(X.k, X.dtype)
    rnd = (lambda a: O.bf16_bits_to_f32(O.f32_to_bf16_bits(a))) if X.dtype == "bf16" else (lambda a: a.astype(np.float32))
    qh = rnd(q * np.float32(cq)); kh = rnd(k * np.float32(ck))
    return qh, kh


@pytest.mark.parametrize("chunk", [1, 2])
def test_small_chunks_equal_brute_force_maxpool(chunk):
    # With chunk size 1 or 2 and stride_q=1 every token of an active chunk is sampled, so the chunk
    # score must be the exact max over (rows, tokens) of the rounded logits.
    X = make_inputs(5, B=1, TQ=32, TK=128, H=2, HKV=1, D=16, dtype="f32")
    sink, sw_eff, BQ = 8, 0, 16
    L = O.lib()
    left, right, scores = _stage0(X, 128, sink, sw_eff, 0, chunk, BQ)
    l_in = left.copy()
    O.mask_stage(X, 128, left, right, scores, BS=left.shape[1], BQ=BQ, stride_q=1, block_chunk=16,
                 scan_stride=1, sw_eff=sw_eff)
    qh, kh = _brute_scores(X, None, chunk, BQ, None)
    B, TQ, H, D = X.q.shape
    for h in range(H):
        for qb in range(TQ // BQ):
            pmin = int(X.pos[0, qb * BQ])
            for c in range(left.shape[-1]):
                cl = int(l_in[0, qb, h, c])
                if cl > pmin - sw_eff:
                    # chunk starts after the first row's position: inactive, or skipped by the program gate
                    assert scores[0, qb, h, c] == -32000.0
                    continue
                best = -np.inf
                for t in range(cl, min(cl + chunk, 128)):
                    for r in range(qb * BQ, (qb + 1) * BQ):
                        a = np.ascontiguousarray(qh[0, r, h]); b = np.ascontiguousarray(kh[0, t, 0])
                        best = max(best, L.hipo_dot(a.ctypes.data, b.ctypes.data, D))
                assert scores[0, qb, h, c] == np.float32(best), (h, qb, c)
                # and the interval collapsed onto the arg-max token of the chunk (ties -> right)
                assert right[0, qb, h, c] - left[0, qb, h, c] <= 1


def test_invariants_nesting_and_inactive_lanes():
    X = make_inputs(7, B=1, TQ=64, TK=1024, H=4, HKV=2, D=64, dtype="bf16")
    sink, chunk, BQ = 16, 64, 32
    left, right, scores = _stage0(X, 1024, sink, 64, 128, chunk, BQ)
    l0, r0 = left.copy(), right.copy()
    O.mask_stage(X, 1024, left, right, scores, BS=left.shape[1], BQ=BQ, stride_q=2, block_chunk=16,
                 scan_stride=1, sw_eff=64)
    assert (left >= l0).all() and (right <= r0).all() and (left <= right).all()
    scores = scores[..., : left.shape[-1]]
    active = scores > -32000
    # active lanes end on an interval of width <= 1, unless the search moved their left edge past
    # p_min - sw' (the activity test is re-evaluated every iteration); inactive lanes are untouched
    lim = np.broadcast_to((X.pos[0, ::BQ] - 64)[None, :, None, None], left.shape)
    done = ((right - left) <= 1) | (left > lim)
    assert done[active].all()
    assert (left > lim)[active].any()  # the case does occur in this input
    assert np.array_equal(left[~active], l0[~active]) and np.array_equal(right[~active], r0[~active])
    # activity rule: a chunk is scored iff it starts at or before p_min - sw' of its query block
    pmin = X.pos[0, ::BQ]
    expect = l0 <= (pmin[None, :, None, None] - 64)
    assert np.array_equal(active, expect)
    # bf16 scores are bf16-representable
    assert np.array_equal(O.bf16_bits_to_f32(O.f32_to_bf16_bits(scores)), scores)


def test_program_level_iteration_count_rescoring():
    # a ragged (narrower) chunk shares the iteration count of the widest chunk in its program
    X = make_inputs(11, B=1, TQ=16, TK=200, H=1, HKV=1, D=16, dtype="f32")
    left = np.array([[[[0, 64, 128]]]], dtype=np.int64)
    right = np.array([[[[64, 128, 131]]]], dtype=np.int64)  # last chunk width 3
    scores = np.full((1, 1, 1, 4), -32000.0, dtype=np.float32)
    O.mask_stage(X, 200, left, right, scores, BS=1, BQ=16, stride_q=1, block_chunk=16, scan_stride=1, sw_eff=0)
    l2 = np.array([[[[128]]]], dtype=np.int64); r2 = np.array([[[[131]]]], dtype=np.int64)
    s2 = np.full((1, 1, 1, 1), -32000.0, dtype=np.float32)
    O.mask_stage(X, 200, l2, r2, s2, BS=1, BQ=16, stride_q=1, block_chunk=16, scan_stride=1, sw_eff=0)
    # alone, the width-3 chunk runs floor(log2(3))+1 = 2 iterations; in company it runs 7 and can only gain
    assert scores[0, 0, 0, 2] >= s2[0, 0, 0, 0]
    assert right[0, 0, 0, 2] - left[0, 0, 0, 2] <= 1
