"""Pins hipo_bsa against dense masked softmax in float64 and against textbook special cases."""
import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, to_paged, widen


def dense_reference(X, indices, ks, bq, bk, sw, sink, max_tsrc, share_first_head=False, softcap=None, visits=None):
    """softmax over the attended set written as an explicit boolean mask, float64 arithmetic.

    Built from the set definition only (no tiling): sink tokens and selected-block tokens at
    distance >= sw from the query, window tokens at distance < sw, everything clipped by the
    query block's largest position.  ``visits[j]``: weight of the tokens of index entry j (default 1).
    """
    B, TQ, H, D = X.q.shape
    k = widen(X.k, X.dtype).astype(np.float64)
    v = widen(X.v, X.dtype).astype(np.float64)
    TK = k.shape[1]
    G = H // k.shape[2]
    cq, ck = O.scale_constants(D, X.dtype)
    rnd = (lambda a: O.bf16_bits_to_f32(O.f32_to_bf16_bits(a.astype(np.float32))).astype(np.float64)) \
        if X.dtype == "bf16" else (lambda a: a.astype(np.float32).astype(np.float64))
    qh = rnd(widen(X.q, X.dtype) * np.float32(cq))
    kh = rnd(widen(X.k, X.dtype) * np.float32(ck))
    out = np.zeros((B, TQ, H, D))
    t = np.arange(TK)
    for b in range(B):
        for h in range(H):
            hrow = (h // G) * G if share_first_head else h
            for qb in range(O.cdiv(TQ, bq)):
                rows = np.arange(qb * bq, min(TQ, (qb + 1) * bq))
                p = X.pos[b, rows]
                curr = p.max() + 1
                sel = np.zeros(TK, dtype=bool)
                weight = np.ones(TK)
                for j in range(int(ks[b * H + hrow, qb])):
                    st = int(indices[b * H + hrow, qb, j])
                    sel[max(st, 0): max(min(st + bk, TK, max_tsrc), 0)] = True
                    if visits is not None:
                        weight[max(st, 0): max(min(st + bk, TK, max_tsrc), 0)] = visits[j]
                sel &= (t >= sink)
                far = (t[None, :] + sw <= p[:, None]) & (t[None, :] < curr)
                near = (t[None, :] <= p[:, None]) & (t[None, :] + sw > p[:, None]) & \
                       (t[None, :] >= max(0, curr - sw - bq)) & (sw > 0)
                mask = (far & (sel | (t < sink))[None, :]) | near
                logits = qh[b, rows, h] @ kh[b, :, h // G].T
                if softcap is not None:
                    logits = np.tanh(logits / softcap) * softcap
                logits = np.where(mask, logits, -np.inf)
                m = logits.max(axis=1, keepdims=True)
                m = np.where(np.isfinite(m), m, 0.0)
                pr = np.exp(logits - m) * np.where(near, 1.0, weight[None, :])
                den = pr.sum(axis=1, keepdims=True)
                den = np.where(den == 0, 1.0, den)
                out[b, rows, h] = (pr / den) @ v[b, :, h // G]
    return out


def random_indices(rng, B, H, nbq, BK, bk, tk, same_heads=True):
    idx = np.full((B * H, nbq, BK), O.INT64_MAX, dtype=np.int64)
    ks = np.zeros((B * H, nbq), dtype=np.int64)
    for b in range(B):
        for qb in range(nbq):
            for h in range(H):
                if same_heads and h > 0:
                    idx[b * H + h, qb] = idx[b * H, qb]; ks[b * H + h, qb] = ks[b * H, qb]
                    continue
                n = int(rng.integers(0, BK + 1))
                st = np.sort(rng.choice(tk // bk, size=n, replace=False)) * bk
                idx[b * H + h, qb, :n] = st
                ks[b * H + h, qb] = n
    kse = np.zeros((B * H, nbq, 2), dtype=np.int32)
    kse[..., 1] = ks
    return idx, ks, kse


@pytest.mark.parametrize("dtype,tol", [("f32", 2e-5), ("bf16", 1.5e-2)])
@pytest.mark.parametrize("bq,TQ", [(16, 40), (1, 1), (64, 64)])
def test_bsa_equals_dense_masked_softmax(dtype, tol, bq, TQ):
    rng = np.random.default_rng(2)
    TK, H, HKV, D, bk, BK, sw, sink = 192, 4, 2, 32, 4, 12, 24, 8
    X = make_inputs(4, B=2, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=0.3)
    nbq = O.cdiv(TQ, bq)
    idx, ks, kse = random_indices(rng, 2, H, nbq, BK, bk, TK, same_heads=False)
    got = widen(O.bsa(X, TK, idx, kse, bq, bk, sw, sink), dtype)
    ref = dense_reference(X, idx, ks, bq, bk, sw, sink, TK)
    assert np.abs(got - ref).max() < tol
    # decode flavour: every head of a GQA group reads the first head's index row
    got2 = widen(O.bsa(X, TK, idx, kse, bq, bk, sw, sink, share_first_head=True), dtype)
    ref2 = dense_reference(X, idx, ks, bq, bk, sw, sink, TK, share_first_head=True)
    assert np.abs(got2 - ref2).max() < tol
    assert np.abs(ref2 - ref).max() > 1e-3  # the two flavours really differ on this input


def test_no_selected_blocks_is_streaming_attention():
    # ks = 0 everywhere -> sink + sliding window (StreamingLLM)
    TK, TQ, H, D, sw, sink, bq = 160, 48, 2, 32, 32, 4, 16
    X = make_inputs(6, B=1, TQ=TQ, TK=TK, H=H, HKV=2, D=D, dtype="f32", scale=0.3)
    idx = np.full((H, 3, 4), O.INT64_MAX, dtype=np.int64)
    kse = np.zeros((H, 3, 2), dtype=np.int32)
    got = O.bsa(X, TK, idx, kse, bq, 4, sw, sink)
    q = torch.from_numpy(X.q).permute(0, 2, 1, 3).double()
    k = torch.from_numpy(X.k).permute(0, 2, 1, 3).double()
    v = torch.from_numpy(X.v).permute(0, 2, 1, 3).double()
    p = torch.from_numpy(X.pos[0])[:, None]; t = torch.arange(TK)[None, :]
    mask = ((t <= p) & (t > p - sw)) | ((t < sink) & (t <= p - sw))
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask[None, None], scale=1.0)
    assert np.abs(got - ref.permute(0, 2, 1, 3).numpy()).max() < 2e-5


def test_huge_window_is_plain_causal_attention():
    TK, TQ, H, D = 96, 96, 2, 64
    X = make_inputs(8, B=1, TQ=TQ, TK=TK, H=H, HKV=1, D=D, dtype="f32", scale=0.3)
    idx = np.full((H, 6, 2), O.INT64_MAX, dtype=np.int64)
    kse = np.zeros((H, 6, 2), dtype=np.int32)
    got = O.bsa(X, TK, idx, kse, 16, 2, 4096, 0)
    q = torch.from_numpy(X.q).permute(0, 2, 1, 3).double()
    k = torch.from_numpy(X.k).permute(0, 2, 1, 3).double().repeat(1, 2, 1, 1)
    v = torch.from_numpy(X.v).permute(0, 2, 1, 3).double().repeat(1, 2, 1, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=1.0)
    assert np.abs(got - ref.permute(0, 2, 1, 3).numpy()).max() < 2e-5


def test_empty_row_gives_zero_and_sink_only_rows():
    # sw = 0, sink = 0, no blocks: nothing attended -> output 0 (l keeps its initial 1.0)
    X = make_inputs(9, B=1, TQ=8, TK=32, H=1, HKV=1, D=16, dtype="f32")
    idx = np.full((1, 1, 1), O.INT64_MAX, dtype=np.int64)
    kse = np.zeros((1, 1, 2), dtype=np.int32)
    got = O.bsa(X, 32, idx, kse, 8, 2, 0, 0)
    assert (got == 0).all()


@pytest.mark.parametrize("page_size", [1, 2, 4, 8, 16, 32])
def test_paged_equals_dense_bit_exact(page_size):
    rng = np.random.default_rng(3)
    TK, TQ, H, HKV, D, bk, BK = 128, 32, 4, 2, 32, 4, 6
    X = make_inputs(10, B=2, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", scale=0.3)
    idx, ks, kse = random_indices(rng, 2, H, 2, BK, bk, TK)
    dense = O.bsa(X, TK, idx, kse, 16, bk, 16, 4)
    XP = to_paged(X, page_size, seed=page_size)
    paged = O.bsa(XP, 4096, idx, kse, 16, bk, 16, 4)
    assert np.array_equal(dense, paged)


@pytest.mark.parametrize("dtype,tol", [("f32", 2e-5), ("bf16", 1.5e-2)])
def test_logit_softcap_is_tanh_capping_of_the_logits(dtype, tol):
    rng = np.random.default_rng(9)
    B, TQ, TK, H, HKV, D, bq, bk, sw, sink = 1, 40, 256, 4, 2, 32, 16, 8, 24, 8
    X = make_inputs(41, B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=1.5)
    idx, ks, kse = random_indices(rng, B, H, O.cdiv(TQ, bq), 6, bk, TK)
    plain = widen(O.bsa(X, TK, idx, kse, bq, bk, sw, sink), dtype)
    X.logit_softcap = 2.0
    got = widen(O.bsa(X, TK, idx, kse, bq, bk, sw, sink), dtype)
    want = dense_reference(X, idx, ks, bq, bk, sw, sink, TK, softcap=2.0)
    assert np.abs(got - want).max() <= tol
    assert np.abs(got - plain).max() > 10 * tol  # the cap matters at this scale


def programs_walk(BK, second_k, sink, sw, bk, rs, re):
    """How often each entry of an index row is visited when the decode kernel's programs run their loops as written
    (attention_decode_bsa.py:239-247) with the launcher's constants (:1070-1076, :1391-1393)."""
    counts = np.zeros(BK, dtype=np.int64)
    chunk = O.cdiv(second_k + sink + sw, 8)
    programs = min(12, O.cdiv(second_k, chunk))
    tile = max(1, min(16, 16 // bk))
    share = O.cdiv(BK, programs)
    for s in range(programs):
        start, end = share * s, min(share * s + share, BK)
        if end > start:
            for i in range(start, end, tile):
                for j in range(i, i + tile):
                    if rs <= j < min(rs + BK, re):
                        counts[j] += 1
    return counts


def test_seam_multiplicity_equals_a_walk_of_the_programs():
    rng = np.random.default_rng(0)
    seen = set()
    for _ in range(400):
        bk = int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
        BK = int(rng.integers(1, 300))
        second_k = int(rng.choice([BK * bk, 2048, 512, 128, 4096]))
        sink, sw = int(rng.choice([0, 4, 128, 256])), int(rng.choice([0, 64, 1024, 4096]))
        re = int(rng.integers(0, BK + 1))
        want = programs_walk(BK, second_k, sink, sw, bk, 0, re)
        share, over = O.decode_seams(second_k, sink, sw, bk, BK)
        got = np.array([O.seam_multiplicity(j, share, over) if j < re else 0 for j in range(BK)])
        assert np.array_equal(got, want), (BK, second_k, sink, sw, bk, re)
        seen.add(int(want.max(initial=0)))
    assert {1, 2, 3} <= seen  # plain, doubled and (tiny rows) tripled entries all occurred
    # the reference's default preset: 2048 tokens in blocks of 8 among 5 programs of 52 entries, tiles of 2 -> no seams
    assert O.decode_seams(2048, 256, 1024, 8, 256) == (52, 0)


@pytest.mark.parametrize("dtype,tol", [("f32", 2e-5), ("bf16", 1.5e-2)])
def test_decode_seams_weigh_the_blocks_at_the_seams_twice(dtype, tol):
    rng = np.random.default_rng(8)
    TK, H, HKV, D, bk, BK, sw, sink, second_k = 512, 4, 2, 32, 2, 40, 24, 8, 80
    lens = np.array([512, 300])
    X = make_inputs(9, B=2, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype, scale=0.3, pos=(lens - 1)[:, None])
    idx, ks, kse = random_indices(rng, 2, H, 1, BK, bk, 280, same_heads=True)
    ks[:] = BK - 3
    kse[..., 1] = BK - 3
    for r in range(idx.shape[0]):
        idx[r, 0] = np.sort(rng.choice(280 // bk, size=BK, replace=False)) * bk
    seams = O.decode_seams(second_k, sink, sw, bk, BK)
    assert seams == (7, 1)  # 6 programs of 7 entries walking tiles of 8: 1 entry of overhang
    visits = programs_walk(BK, second_k, sink, sw, bk, 0, BK - 3)
    assert visits.max() == 2 and visits[:BK - 3].min() == 1
    got = widen(O.bsa(X, TK, idx, kse, 1, bk, sw, sink, share_first_head=True, seams=seams), dtype)
    ref = dense_reference(X, idx, ks, 1, bk, sw, sink, TK, share_first_head=True, visits=visits)
    once = dense_reference(X, idx, ks, 1, bk, sw, sink, TK, share_first_head=True)
    assert np.abs(got - ref).max() < tol
    assert np.abs(ref - once).max() > 5 * tol


def test_sink_numbering_of_the_decode_programs_equals_a_walk_of_their_loops():
    """attention_decode_bsa.py:514-520 and :740: a program over the sink starts at ``share * s``, steps by its tile of
    ``BLOCK_BK * bk`` tokens and numbers the tile's entries ``arange(BLOCK_BK) + i_tsrc // bk``."""
    rng = np.random.default_rng(1)
    slipped = 0
    for _ in range(200):
        bk = int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
        sink = int(rng.choice([4, 16, 100, 256, 1024]))
        second_k, sw = int(rng.choice([128, 256, 2048])), int(rng.choice([0, 256, 1024]))
        chunk = O.cdiv(second_k + sink + sw, 8)
        programs = min(12, O.cdiv(sink, chunk))
        share = O.cdiv(sink, programs)
        assert share == O.decode_sink_share(second_k, sink, sw)
        block_bk = max(1, min(16, 16 // bk))
        slot = np.full(sink, -1, dtype=np.int64)
        for s in range(programs):
            start, end = share * s, min(share * s + share, sink)
            for i in range(start, end, block_bk * bk):
                for x in range(block_bk * bk):
                    if i + x < end:
                        slot[i + x] = (x // bk + i // bk) * bk + x % bk
        t = np.arange(sink)
        assert np.array_equal(slot, t - ((t // share) * share) % bk), (bk, sink, second_k, sw)
        slipped += int((slot != t).any())
    assert slipped > 20


def _non_causal_reference(X, indices, ks, bq, bk, sw, sink, max_tsrc, decode):
    """is_causal = False written from its description (attention_extend_bsa.py:511-523, :743-752): the mask keeps
    nothing but validity.  Query-block form: every row sits at position max_tsrc - 1, so all rows of a block attend
    the same multiset: the tokens of their selected blocks (at or above the sink), the sink, and the last
    sw + bq tokens; a token that is selected and in that window counts twice.  Decode form: the same with the row's
    true position in place of max_tsrc - 1.  float64."""
    B, TQ, H, D = X.q.shape
    k = widen(X.k, X.dtype).astype(np.float64)
    v = widen(X.v, X.dtype).astype(np.float64)
    TK = k.shape[1]
    G = H // k.shape[2]
    cq, ck = O.scale_constants(D, X.dtype)
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    qh, kh = f32(widen(X.q, X.dtype) * np.float32(cq)), f32(widen(X.k, X.dtype) * np.float32(ck))
    out = np.zeros((B, TQ, H, D))
    for b in range(B):
        for h in range(H):
            for qb in range(O.cdiv(TQ, bq)):
                rows = np.arange(qb * bq, min(TQ, (qb + 1) * bq))
                curr = (int(X.pos[b, rows].max()) + 1) if decode else max_tsrc
                count = np.zeros(TK)
                for j in range(int(ks[b * H + h, qb])):
                    st = int(indices[b * H + h, qb, j])
                    for t in range(st, st + bk):
                        if 0 <= t < min(TK, max_tsrc) and sink <= t < curr:
                            count[t] += 1
                count[:min(sink, curr)] += 1
                if sw > 0:
                    count[max(0, curr - sw - bq):curr] += 1
                logits = np.where(count[None, :] > 0, qh[b, rows, h] @ kh[b, :, h // G].T, -np.inf)
                pr = np.exp(logits - logits.max(axis=1, keepdims=True)) * count[None, :]
                out[b, rows, h] = (pr / pr.sum(axis=1, keepdims=True)) @ v[b, :, h // G]
    return out


@pytest.mark.parametrize("decode", [False, True])
def test_non_causal_mask_keeps_validity_only(decode):
    rng = np.random.default_rng(5)
    TK, H, HKV, D, bk, BK, sw, sink = 192, 4, 2, 32, 4, 12, 24, 8
    bq, TQ = (1, 1) if decode else (16, 40)
    pos = np.array([[150], [99]]) if decode else None
    X = make_inputs(14, B=2, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="f32", scale=0.3, pos=pos)
    nbq = O.cdiv(TQ, bq)
    idx, ks, kse = random_indices(rng, 2, H, nbq, BK, bk, TK, same_heads=False)
    idx[0, 0, :3] = [TK - 40, TK - 24, TK - 8]  # blocks inside the last sw + bq tokens: attended twice
    idx[0, 0, 3:] = O.INT64_MAX
    ks[0, 0] = 3; kse[0, 0, 1] = 3
    X.non_causal = 2 if decode else 1
    got = O.bsa(X, TK, idx, kse, bq, bk, sw, sink)
    ref = _non_causal_reference(X, idx, ks, bq, bk, sw, sink, TK, decode)
    assert np.abs(got - ref).max() < 2e-5
    X.non_causal = 0
    causal = O.bsa(X, TK, idx, kse, bq, bk, sw, sink)
    assert np.abs(causal - got).max() > 1e-3  # the switch really changes the result


def test_non_causal_with_a_huge_window_is_plain_bidirectional_attention():
    TK, TQ, H, D = 96, 96, 2, 64
    X = make_inputs(8, B=1, TQ=TQ, TK=TK, H=H, HKV=1, D=D, dtype="f32", scale=0.3)
    idx = np.full((H, 6, 2), O.INT64_MAX, dtype=np.int64)
    kse = np.zeros((H, 6, 2), dtype=np.int32)
    X.non_causal = 1
    got = O.bsa(X, TK, idx, kse, 16, 2, 4096, 0)
    q = torch.from_numpy(X.q).permute(0, 2, 1, 3).double()
    k = torch.from_numpy(X.k).permute(0, 2, 1, 3).double().repeat(1, 2, 1, 1)
    v = torch.from_numpy(X.v).permute(0, 2, 1, 3).double().repeat(1, 2, 1, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=False, scale=1.0)
    assert np.abs(got - ref.permute(0, 2, 1, 3).numpy()).max() < 2e-5
