"""Selection between scan stages and the final index layout, called directly through the C ABI.

Both kernels of each entry point (the throughput kernel of wide launches and the latency kernel of launches with a
few workgroups, as in decode) are checked against the definition written out in numpy: the k best chunks by (score
descending, position ascending) in position order (reference: `topk(sorted=False)` followed by a sort of the positions,
attention_extend.py:2710-2728), and for the final layout the block-aligned left edges with repeats dropped, padded
with the largest int64, and the count of entries before the end of the query block
(attention_extend.py:2757-2776, 2906-2924).
"""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

INT64_MAX = np.iinfo(np.int64).max


def _scores(rng, shape, kind):
    if kind == "bf16":  # scores as the bf16 scan kernels store them: low 16 bits zero, many ties
        s = rng.standard_normal(shape).astype(np.float32) * 3
        s = (s.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)
    elif kind == "ties":  # a handful of distinct values, both zeros among them
        s = rng.choice(np.array([-2.0, -0.0, 0.0, 0.5, 0.5000001, 3.0], dtype=np.float32), size=shape)
    else:  # full-precision scores
        s = rng.standard_normal(shape).astype(np.float32)
    return np.ascontiguousarray(s)


def _top_positions(key, k):
    """positions of the k best entries by (score descending, position ascending), ascending"""
    order = np.lexsort((np.arange(key.size), -key.astype(np.float64)))
    return np.sort(order[:k])


@pytest.fixture(params=["1", "0"], ids=["latency_kernel", "throughput_kernel"])
def select_fast(request):
    old = os.environ.get("HIPATTN_SELECT_FAST")
    os.environ["HIPATTN_SELECT_FAST"] = request.param
    yield request.param
    if old is None:
        del os.environ["HIPATTN_SELECT_FAST"]
    else:
        os.environ["HIPATTN_SELECT_FAST"] = old


@pytest.mark.parametrize("B,bs_in,bs_out,row_rep,HEAD,hg,n,k,splits,kind", [
    (1, 1, 1, 1, 1, 1, 4091, 128, 8, "bf16"),     # 1M-key decode, first stage (four entries per thread)
    (1, 1, 1, 1, 1, 1, 1024, 256, 4, "bf16"),     # one entry per thread
    (2, 1, 1, 1, 4, 1, 1000, 100, 2, "f32"),      # maximum over four heads, four radix passes
    (2, 2, 4, 2, 8, 8, 777, 33, 1, "ties"),       # a list per head, rows repeated, ties across the threshold
    (1, 1, 1, 1, 2, 1, 5000, 4999, 2, "ties"),    # sixteen entries per thread, all but one selected
    (3, 1, 1, 1, 1, 1, 640, 640, 4, "bf16"),      # everything selected
    (1, 1, 1, 1, 1, 1, 16384, 8192, 1, "f32"),    # the largest list the latency kernel holds
    (1, 1, 1, 1, 1, 1, 16384, 9000, 1, "bf16"),   # beyond it: the throughput kernel in both settings
    (1, 3, 3, 1, 2, 1, 65, 1, 3, "f32"),
])
def test_select_stage_against_its_definition(select_fast, B, bs_in, bs_out, row_rep, HEAD, hg, n, k, splits, kind):
    from hip_attn import _native as N

    rng = np.random.default_rng(n * 31 + k)
    chunk = 8 * splits
    sub = chunk // splits
    scores = _scores(rng, (B, bs_in, HEAD, n), kind)
    left = np.sort(rng.choice(n * 4, size=(B, bs_in, hg, n)).astype(np.int32) * chunk, axis=-1)
    dev = torch.device("cuda")
    t_scores, t_left = torch.from_numpy(scores).to(dev), torch.from_numpy(left).to(dev)
    nxt = torch.full((B, bs_out, hg, k * splits), -7, dtype=torch.int32, device=dev)
    l64 = torch.full((B, bs_out, hg, k * splits), -7, dtype=torch.int64, device=dev)
    r64 = torch.full((B, bs_out, hg, k * splits), -7, dtype=torch.int64, device=dev)
    nsc = torch.zeros((B, bs_out, 1, k * splits), dtype=torch.float32, device=dev) if hg == 1 else None
    N.select_stage(t_scores, t_left, B, bs_in, bs_out, row_rep, HEAD, hg, n, k, chunk, splits, nxt, dev,
                   left64=l64, right64=r64, next_scores=nsc)
    torch.cuda.synchronize()
    nheads = HEAD // hg
    want = np.empty((B, bs_out, hg, k * splits), dtype=np.int64)
    for b in range(B):
        for o in range(bs_out):
            i = (o + row_rep * bs_in - bs_out) // row_rep
            for g in range(hg):
                key = scores[b, i, g * nheads:(g + 1) * nheads].max(axis=0)
                sel = _top_positions(key, k)
                want[b, o, g] = (left[b, i, g, sel].astype(np.int64)[:, None] + np.arange(splits) * sub).reshape(-1)
    assert np.array_equal(nxt.cpu().numpy(), want)
    assert np.array_equal(l64.cpu().numpy(), want)
    assert np.array_equal(r64.cpu().numpy(), want + sub)
    if nsc is not None:
        assert bool(torch.isneginf(nsc).all())


@pytest.mark.parametrize("B,bs,bdst,stride,HEAD,score_heads,hg,n,K,chunk,kind", [
    (1, 1, 1, 1, 32, 1, 1, 1024, 256, 8, "bf16"),    # decode: head-reduced scores, one list, a row per head
    (2, 1, 1, 1, 8, 8, 1, 3000, 500, 16, "f32"),     # four entries per thread, maximum over the heads
    (2, 2, 3, 2, 4, 4, 4, 700, 64, 4, "ties"),       # a list per head, scan rows repeated
    (1, 1, 1, 1, 4, 1, 1, 300, 300, 8, "bf16"),      # everything selected
    (1, 1, 1, 1, 2, 2, 1, 900, 1, 8, "f32"),         # a single entry equals its own predecessor: empty row
    (1, 1, 1, 1, 2, 1, 1, 6000, 512, 8, "bf16"),     # longer than the latency kernel takes
])
def test_finalize_indices_against_its_definition(select_fast, B, bs, bdst, stride, HEAD, score_heads, hg, n, K, chunk,
                                                 kind):
    from hip_attn import _native as N

    rng = np.random.default_rng(n * 17 + K)
    bq = 64
    scores = _scores(rng, (B, bs, score_heads, n), kind)
    # refined left edges: ascending, unaligned, with runs that fall into the same block
    left = np.sort(rng.integers(0, n * chunk // 2, size=(B, bs, HEAD, n)).astype(np.int32), axis=-1)
    pos = (np.arange(bdst * bq, dtype=np.int64)[None, :] + rng.integers(n * chunk // 8, n * chunk // 3, size=(B, 1)))
    pos = np.ascontiguousarray(pos)
    dev = torch.device("cuda")
    BK = min(K, n)
    idx = torch.full((B * HEAD, bdst, BK), -7, dtype=torch.int64, device=dev)
    ks = torch.full((B * HEAD, bdst), -7, dtype=torch.int64, device=dev)
    kse = torch.full((B * HEAD, bdst, 2), -7, dtype=torch.int32, device=dev)
    N.finalize_indices(torch.from_numpy(scores).to(dev), torch.from_numpy(left).to(dev), torch.from_numpy(pos).to(dev),
                       B, bs, bdst, stride, HEAD, score_heads, hg, n, K, chunk, bq, idx, ks, kse, dev)
    torch.cuda.synchronize()
    nheads, nsh = HEAD // hg, score_heads // hg
    want = np.full((B * HEAD, bdst, BK), INT64_MAX, dtype=np.int64)
    want_ks = np.zeros((B * HEAD, bdst), dtype=np.int64)
    for b in range(B):
        for qb in range(bdst):
            i = (qb + stride * bs - bdst) // stride
            for h in range(HEAD):
                g = h // nheads
                key = scores[b, i, g * nsh:(g + 1) * nsh].max(axis=0)
                sel = _top_positions(key, BK)
                v = left[b, i, h, sel].astype(np.int64) // chunk * chunk
                keep = v != np.roll(v, 1)
                u = v[keep]
                want[b * HEAD + h, qb, :u.size] = u
                want_ks[b * HEAD + h, qb] = int((u < pos[b, qb * bq] + bq).sum())
    assert np.array_equal(idx.cpu().numpy(), want)
    assert np.array_equal(ks.cpu().numpy(), want_ks)
    got_kse = kse.cpu().numpy()
    assert np.array_equal(got_kse[..., 0], np.zeros_like(want_ks))
    assert np.array_equal(got_kse[..., 1], want_ks)
