"""Pins the oracle's RoPE-on-load ("extend") paths against the complex-number form of rotary embeddings.

A row x of width D is read as D/2 complex numbers z_d = x[d] + i*x[d + D/2]; rotating the row to position p
multiplies z_d by exp(i * p * w_d).  The logit of a rotated query/key pair is Re(sum_d zq_d * conj(zk_d) *
exp(i * (pq - pk) * w_d)).  The expectations below are built from that identity and from a plain description of
where each rule puts the keys, in float64, without the oracle's table lookups or rotate-half arithmetic.
"""
import numpy as np
import pytest

from oracle import hip12 as O
from helpers import make_inputs, rope_tables, to_paged, widen, with_rope


def _cplx(x):
    D = x.shape[-1]
    return x[..., : D // 2].astype(np.float64) + 1j * x[..., D // 2:].astype(np.float64)


def _rot(x, pos, D, theta=10000.0):
    """rows [..., D] rotated to integer positions pos [...]: float64 complex arithmetic, back to real layout."""
    inv = theta ** (-np.arange(0, D, 2, dtype=np.float64) / D)
    z = _cplx(x) * np.exp(1j * np.asarray(pos, dtype=np.float64)[..., None] * inv)
    return np.concatenate([z.real, z.imag], axis=-1)


@pytest.mark.parametrize("dtype,tol", [("f32", 2e-6), ("bf16", 2e-2)])
def test_row_rotation_is_complex_multiplication(dtype, tol):
    X = with_rope(make_inputs(1, B=1, TQ=4, TK=8, H=1, HKV=1, D=32, dtype=dtype), 300, scan_backend="relative")
    x = widen(X.q, dtype)[0, :, 0]
    for r, pos in enumerate([0, 1, 17, 299]):
        got = O.rope_row(X, x[r], pos)
        want = _rot(x[r], pos, 32)
        assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), (pos, np.abs(got - want).max())
    # position 0 is the identity
    assert np.array_equal(O.rope_row(X, x[0], 0), x[0])
    # norms of the complex pairs are kept
    z0, z1 = _cplx(x[1]), _cplx(O.rope_row(X, x[1], 123))
    assert np.allclose(np.abs(z0), np.abs(z1), rtol=4 * tol, atol=4 * tol)


def _stage0(TK, sink, sw_eff, chunk, B, BS, H):
    n = O.cdiv(TK - sink - sw_eff, chunk)
    left = np.zeros((B, BS, H, n), dtype=np.int64)
    left[...] = sink + np.arange(n) * chunk
    right = np.minimum(left + chunk, TK - sw_eff)
    scores = np.full((B, BS, H, O.npow2(n)), -32000.0, dtype=np.float32)
    return left, right, scores


@pytest.mark.parametrize("backend", ["relative", "streaming", "infllm", "dynamic_extend", "dynamic_extend squeezed",
                                     "self_extend", "self_extend grouped"])
def test_mask_stage_chunk_size_one_scores(backend):
    # Chunks of one token: the scan evaluates token t once as the "left" and once as the "right" candidate and
    # keeps the larger score.  relative: key at 0 (left) or 1 (right), query at 1 + window; streaming: key at its
    # chunk number, query at min(position, chunks + window); infllm: key at 0, query at the window; dynamic_extend:
    # every query row at its own position, and the key at its own token while the block ends inside the model's
    # context -- plain rotary scores -- or, beyond it (model context 32 against positions 48..63), keys older than
    # a quarter of that context squeezed linearly into the rest (attention_extend.py:249-274).  self_extend: like
    # dynamic_extend, except that beyond the model's context a key older than 8192 positions moves to
    # pmin + trunc((t - pmin) / 16): sixteen neighbours share a position (attention_extend.py:275-289; the quotient
    # of the negative numerator truncates toward zero, as the compiled kernel's int32 division does).  8192 is fixed
    # in the reference, so the grouped case needs positions beyond it.
    D, BQ, sink, sw_eff = 32, 8, 4, 6
    squeezed = backend.endswith("squeezed")
    grouped = backend.endswith("grouped")
    backend = backend.split()[0]
    TK = 8400 if grouped else 64
    X = make_inputs(11, B=1, TQ=16, TK=TK, H=2, HKV=1, D=D, dtype="f32")
    X = with_rope(X, TK + 64 if grouped else 256, scan_backend=backend)
    if squeezed:
        X.model_context_length = 32
    if grouped:
        X.model_context_length = 4096
    left, right, scores = _stage0(TK, sink, sw_eff, 1, 1, 2, 2)
    l_in = left.copy()
    n = left.shape[-1]
    O.mask_stage(X, TK, left, right, scores, BS=2, BQ=BQ, stride_q=1, block_chunk=16, scan_stride=1, sw_eff=sw_eff)
    cq, ck = O.scale_constants(D, "f32")
    q = widen(X.q, "f32").astype(np.float64)
    k = widen(X.k, "f32").astype(np.float64)
    checked = 0
    for h in range(2):
        for qb in range(2):
            rows = np.arange(qb * BQ, (qb + 1) * BQ)
            p = X.pos[0, rows]
            if backend == "relative":
                qpos, kpos = np.full(BQ, 1 + sw_eff), (lambda c: (0, 1))
            elif backend == "infllm":
                qpos, kpos = np.full(BQ, sw_eff), (lambda c: (0, 0))
            elif backend == "dynamic_extend":
                def kpos(c, t, pmin=int(p.min()), pmax=int(p.min()) + BQ, ctx=int(X.model_context_length)):
                    w = ctx // 4
                    if t >= pmax - w or pmax <= ctx:
                        return (t, t)
                    moved = int((np.float32(t) - np.float32(pmin - w)) * (np.float32(ctx - w) / np.float32(pmin - w)))
                    return (max(pmax - ctx, moved + pmin - w),) * 2
                qpos = p
            elif backend == "self_extend":
                def kpos(c, t, pmin=int(p.min()), pmax=int(p.min()) + BQ, ctx=int(X.model_context_length)):
                    if t >= pmax - 8192 or pmax <= ctx:
                        return (t, t)
                    return (max(0, pmin - (pmin - t) // 16),) * 2  # t < pmin: truncation of (t - pmin) / 16
                qpos = p
            else:
                qpos, kpos = np.minimum(p, n + sw_eff), (lambda c: (c, c))
            qr = _rot(q[0, rows, h], qpos, D) * cq
            for c in range(n):
                t = int(l_in[0, qb, h, c])
                if t > p.min() - sw_eff:
                    assert scores[0, qb, h, c] == -32000.0
                    continue
                if grouped and 300 < t < TK - 300:
                    continue  # the grouped case checks both ends of the key range, not all 8400 tokens
                kps = kpos(c, t) if backend in ("dynamic_extend", "self_extend") else kpos(c)
                if squeezed and t < 40:
                    assert kps[0] != t  # the squeeze really moves these keys
                if grouped and t < 190:
                    assert kps[0] != t
                    assert int(p.min()) - kps[0] == (int(p.min()) - t) // 16  # sixteen keys share a position
                best = max(float((qr @ (_rot(k[0, t, 0], kp, D) * ck)).max()) for kp in kps)
                assert abs(scores[0, qb, h, c] - best) <= 2e-5 * max(1.0, abs(best)), (backend, h, qb, c)
                checked += 1
    assert checked > 50


def test_mask_stage_infllm_is_plain_scan_of_rotated_queries():
    # infllm rotates every key to position 0 (the identity) and every query row to the window size: the stage must
    # equal, bit for bit, the unrotated stage run on queries rotated beforehand.  Strided rows included.
    for dtype in ("f32", "bf16"):
        X = make_inputs(12, B=2, TQ=40, TK=200, H=4, HKV=2, D=32, dtype=dtype)
        Xr = with_rope(make_inputs(12, B=2, TQ=40, TK=200, H=4, HKV=2, D=32, dtype=dtype), 128, scan_backend="infllm")
        sw_eff = 24
        qw = widen(X.q, dtype)
        qrot = np.stack([[[O.rope_row(Xr, qw[b, t, h], sw_eff) for h in range(4)] for t in range(40)]
                         for b in range(2)]).astype(np.float32)
        X.q = O.f32_to_bf16_bits(qrot) if dtype == "bf16" else qrot
        a = _stage0(200, 8, sw_eff, 16, 2, 3, 4)
        b_ = tuple(x.copy() for x in a)
        kw = dict(BS=3, BQ=16, stride_q=2, block_chunk=16, scan_stride=1, sw_eff=sw_eff)
        O.mask_stage(X, 200, *a, **kw)
        O.mask_stage(Xr, 200, *b_, **kw)
        for x, y in zip(a, b_):
            assert np.array_equal(x, y)
        assert (a[2] > -32000).any()


def _expected_bsa(X, indices, ks, bq, bk, sw, sink, backend, share_first_head=False):
    """Dense float64 softmax over the attended set, keys placed by the rule's plain description:
    sink tokens and the tokens of the selected blocks, in the order of the index row, fill consecutive slots;
    "streaming" rotates slot s to (first query position of the block - window) - (last slot - s), "infllm" rotates
    all of them to (first query position - window); negative positions clamp to 0; window keys and queries keep
    their own positions."""
    B, TQ, H, D = X.q.shape
    dt = X.dtype
    cq, ck = O.scale_constants(D, dt)
    q = widen(X.q, dt).astype(np.float64)
    k = widen(X.k, dt).astype(np.float64)
    v = widen(X.v, dt).astype(np.float64)
    G = H // k.shape[2]
    TK = k.shape[1]
    out = np.zeros((B, TQ, H, D))
    for b in range(B):
        for h in range(H):
            hrow = (h // G) * G if share_first_head else h
            for qb in range(O.cdiv(TQ, bq)):
                rows = np.arange(qb * bq, min(TQ, (qb + 1) * bq))
                p = X.pos[b, rows]
                curr, pmin = int(p.max()) + 1, int(p.min())
                nsel = int(ks[b * H + hrow, qb])
                slots = list(range(sink))
                for j in range(nsel):
                    st = int(indices[b * H + hrow, qb, j])
                    slots += list(range(st, st + bk))
                last = len(slots) - 1
                toks, kpos, far = [], [], []
                for s, t in enumerate(slots):
                    if t < 0 or t >= TK or t >= curr or (s >= sink and t < sink):
                        continue
                    toks.append(t)
                    kpos.append(max(0, (pmin - sw) - (last - s) if backend == "streaming" else pmin - sw))
                    far.append(True)
                if sw > 0:
                    for t in range(max(0, curr - sw - bq), curr):
                        toks.append(t); kpos.append(t); far.append(False)
                if not toks:
                    continue
                toks, kpos, far = np.array(toks), np.array(kpos), np.array(far)
                kr = _rot(k[b, toks, h // G], kpos, D) * ck
                qr = _rot(q[b, rows, h], p, D) * cq
                logits = qr @ kr.T
                att = np.where(far[None, :], toks[None, :] + sw <= p[:, None],
                               (toks[None, :] <= p[:, None]) & (p[:, None] < toks[None, :] + sw))
                logits = np.where(att, logits, -np.inf)
                m = logits.max(axis=1, keepdims=True)
                m = np.where(np.isfinite(m), m, 0.0)
                pr = np.exp(logits - m)
                den = pr.sum(axis=1, keepdims=True)
                den = np.where(den == 0, 1.0, den)
                out[b, rows, h] = (pr / den) @ v[b, toks, h // G]
    return out


def _random_indices(rng, B, H, nbq, BK, bk, lo, hi):
    idx = np.full((B * H, nbq, BK), O.INT64_MAX, dtype=np.int64)
    ks = np.zeros((B * H, nbq), dtype=np.int64)
    for r in range(B * H):
        for qb in range(nbq):
            n = int(rng.integers(1, BK + 1))
            st = lo + np.sort(rng.choice((hi - lo) // bk, size=n, replace=False)) * bk
            idx[r, qb, :n] = st
            ks[r, qb] = n
    kse = np.zeros((B * H, nbq, 2), dtype=np.int32)
    kse[..., 1] = ks
    return idx, ks, kse


@pytest.mark.parametrize("backend", ["streaming", "infllm"])
# bf16: tables, products and sums are all rounded to 8 bits, so only gross agreement is asked; f32 is the pin
@pytest.mark.parametrize("dtype,tol", [("f32", 5e-5), ("bf16", 1e-1)])
@pytest.mark.parametrize("bq,TQ", [(16, 40), (1, 1)])
def test_bsa_with_rope_equals_dense_softmax_of_packed_positions(backend, dtype, tol, bq, TQ):
    rng = np.random.default_rng(21)
    B, H, HKV, D, TK, bk, sink, sw = 2, 4, 2, 32, 256, 8, 16, 24
    X = with_rope(make_inputs(22, B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype=dtype), 512, sa_backend=backend)
    nbq = O.cdiv(TQ, bq)
    idx, ks, kse = _random_indices(rng, B, H, nbq, 6, bk, sink, TK)
    if bq == 1:  # decode: every head of a group reads the first head's row
        got = widen(O.bsa(X, TK, idx, kse, bq, bk, sw, sink, share_first_head=True), dtype)
        want = _expected_bsa(X, idx, ks, bq, bk, sw, sink, backend, share_first_head=True)
    else:
        got = widen(O.bsa(X, TK, idx, kse, bq, bk, sw, sink), dtype)
        want = _expected_bsa(X, idx, ks, bq, bk, sw, sink, backend)
    assert np.abs(got - want).max() <= tol, np.abs(got - want).max()


def test_bsa_streaming_with_every_block_selected_is_causal_rope_attention():
    # One query block whose index row lists every key block between the sink and the window: the packed positions
    # coincide with the true ones, so the result is ordinary causal attention over rotary-embedded q and k (rows
    # after the first lose the few tokens between the last block and their own window, as without RoPE).
    B, H, HKV, D, bk, sink, sw, bq = 1, 2, 1, 32, 8, 16, 16, 8
    TK = 16 + 12 * 8 + 16 + 7  # sink + blocks + window + (rows after the first)
    X = with_rope(make_inputs(23, B=B, TQ=bq, TK=TK, H=H, HKV=HKV, D=D, dtype="f32"), 512, sa_backend="streaming")
    pmin = int(X.pos[0, 0])
    assert pmin - sw + 1 == sink + 12 * bk
    idx = np.broadcast_to(sink + np.arange(12) * bk, (B * H, 1, 12)).astype(np.int64).copy()
    kse = np.zeros((B * H, 1, 2), dtype=np.int32); kse[..., 1] = 12
    got = O.bsa(X, TK, idx, kse, bq, bk, sw, sink)
    q = widen(X.q, "f32").astype(np.float64); k = widen(X.k, "f32").astype(np.float64)
    v = widen(X.v, "f32").astype(np.float64)
    cq, ck = O.scale_constants(D, "f32")
    for h in range(H):
        qr = _rot(q[0, :, h], X.pos[0], D) * cq
        kr = _rot(k[0, :, 0], np.arange(TK), D) * ck
        logits = qr @ kr.T
        t = np.arange(TK)[None, :]
        p = X.pos[0][:, None]
        logits = np.where((t <= p) & ((t + sw > p) | (t < sink + 12 * bk)), logits, -np.inf)
        pr = np.exp(logits - logits.max(axis=1, keepdims=True))
        want = (pr / pr.sum(axis=1, keepdims=True)) @ v[0, :, 0]
        assert np.abs(got[0, :, h] - want).max() <= 5e-5


def test_driver_with_rope_runs_and_differs_from_plain():
    from helpers import tiny_args
    X = with_rope(make_inputs(24, B=1, TQ=64, TK=1024, H=2, HKV=1, D=32, dtype="f32"), 2048)
    plain, meta_p = O.hip_attention_12(X, tiny_args())
    for scan in ("relative", "streaming", "infllm"):
        ctx, meta = O.hip_attention_12(X, tiny_args(using_extend=True, need_apply_rope=True,
                                                    scan_extend_backend=scan, sa_extend_backend="streaming"))
        assert np.isfinite(ctx).all() and ctx.shape == X.q.shape
        assert not np.array_equal(ctx, plain)
        assert X.scan_backend is None and X.sa_backend is None
        # paged and dense agree bit for bit
        XP = with_rope(to_paged(X, 8, seed=2), 2048)
        ctx_p, meta_pg = O.hip_attention_12(XP, tiny_args(using_extend=True, need_apply_rope=True, extend_context_length=1024,
                                                          scan_extend_backend=scan, sa_extend_backend="streaming"))
        assert np.array_equal(meta.indices, meta_pg.indices)
        assert np.array_equal(ctx, ctx_p)
