"""GPU parity on cut-down forms of the benchmark workloads, at the sizes that pick the kernel variants the benchmark
times.

A prefill with 16384 and more scan programs takes the wide scan kernels (two token blocks per wave, prescaled keys,
a wave walking eight chunk groups when a program has 64 query rows) and the tile attention kernel with the four heads
of a GQA group in one workgroup; the small parity cases never reach those.  The oracle cannot run such a call whole in
seconds, but the result of a query block depends on that block's queries only, so the oracle runs on the last query
blocks and is compared with the same blocks of the full-size GPU call.
"""
import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, to_paged
from gpu_utils import assert_context_close, assert_metadata_equal, from_torch, run_product, to_torch

pytestmark = pytest.mark.gpu


def _case(name):
    print(f"[case] {name}", flush=True)


def _tail(X, rows):
    """The last ``rows`` queries of a dense prefill as an oracle problem of their own."""
    return O.OInputs(X.dtype, np.ascontiguousarray(X.q[:, -rows:]), np.ascontiguousarray(X.pos[:, -rows:]), k=X.k, v=X.v)


def _assert_tail_equal(meta, ometa, ctx, octx, blocks, bq, dtype):
    assert np.array_equal(meta.indices[:, -blocks:].cpu().numpy(), ometa.indices), "indices differ"
    assert np.array_equal(meta.ks[:, -blocks:].cpu().numpy(), ometa.ks), "ks differ"
    assert np.array_equal(meta.ks_start_end[:, -blocks:].cpu().numpy(), ometa.ks_start_end)
    assert_context_close(ctx[:, -blocks * bq:], octx, dtype)


WIDE_BLOCKS = 6


@pytest.fixture(scope="module")
def wide_case():
    """Inputs of the wide prefill and the oracle's results on its last six and first two query blocks."""
    X = make_inputs(81, B=1, TQ=16384, TK=65536, H=16, HKV=4, D=128, dtype="bf16")
    X.v = X.k.copy()
    A = O.OArgs(sliding_window_size=1024)
    print("  oracle on the last query blocks ...", flush=True)
    tail = O.hip_attention_12(_tail(X, WIDE_BLOCKS * 64), A)
    print("  oracle on the first query blocks ...", flush=True)
    Xh = O.OInputs("bf16", np.ascontiguousarray(X.q[:, :128]), np.ascontiguousarray(X.pos[:, :128]), k=X.k, v=X.v)
    head = O.hip_attention_12(Xh, A)
    print("  oracle done", flush=True)
    return X, A, tail, head


@pytest.mark.parametrize("statistics", [False, True])
def test_wide_prefill_head_dim_128_against_the_oracle_on_its_last_query_blocks(wide_case, statistics):
    """Default stages, 16 query heads over 4 kv heads, head dim 128, 16384 queries against 65536 keys:
    65536 scan programs in stage 0 and 262144 in stages 1 and 2."""
    _case(f"wide prefill D=128, statistics={statistics}")
    X, A, (octx, ometa), (octx_h, ometa_h) = wide_case
    ctx, meta = run_product(X, A, require_cache_statistics=statistics)
    assert meta.indices.shape == (16, 256, 256)
    _assert_tail_equal(meta, ometa, ctx, octx, WIDE_BLOCKS, 64, "bf16")
    # the first query blocks see the shortest prefixes: their candidate lists end inside a chunk group
    assert np.array_equal(meta.indices[:, :2].cpu().numpy(), ometa_h.indices), "indices of the first blocks differ"
    assert np.array_equal(meta.ks[:, :2].cpu().numpy(), ometa_h.ks)
    assert_context_close(ctx[:, :128], octx_h, "bf16")
    if statistics:
        # every query block sets flags: what the oracle's blocks touched must be flagged by the full call
        for got, want in ((meta.mask_cache_statistics.access_counter, ometa.mask_access),
                          (meta.sa_cache_statistics.access_counter, ometa.sa_access),
                          (meta.mask_cache_statistics.access_counter, ometa_h.mask_access)):
            got = got.cpu().numpy()
            assert got.shape == want.shape
            assert not ((want != 0) & (got == 0)).any(), "a row the oracle loaded is not flagged"


def _plant_needles(k_bits, starts, u, level):
    """Overwrite 8-token blocks: their component along the unit vector ``u`` becomes ``level`` (all kv heads)."""
    k = O.bf16_bits_to_f32(k_bits)
    for st in starts:
        blk = k[0, st:st + 8]
        blk = blk - (blk @ u)[..., None] * u + level * u
        k[0, st:st + 8] = blk
    return O.f32_to_bf16_bits(k)


def _recall(indices, starts):
    """Fraction of planted blocks among the selected blocks, per index row: [rows, blocks] -> mean."""
    idx = np.asarray(indices)
    found = (idx[:, :, None] == np.asarray(starts)[None, None, :]).any(axis=1)
    return found.mean(), found


def test_needle_blocks_prefill_and_decode_recall_equals_the_oracles():
    """The long-context workload in miniature: 64k keys of N(0,1) with 16 planted 8-token blocks that point along a
    direction the queries share.  Selected indices must equal the oracle's bit for bit, hence recall as well; recall
    itself is reported, not required to be 1 (a search samples midpoints only)."""
    _case("needle recall, 64k keys")
    TK, H, HKV, D, TQ = 65536, 16, 4, 128, 256
    rng = np.random.default_rng(1234)
    u = rng.standard_normal(D).astype(np.float32)
    u /= np.linalg.norm(u)
    starts = np.sort(rng.permutation((TK - 4096) // 8)[:16] * 8 + 2048)
    X = make_inputs(82, B=1, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16")
    X.k = _plant_needles(X.k, starts, u, 12.0)
    X.v = X.k.copy()
    X.q = O.f32_to_bf16_bits(O.bf16_bits_to_f32(X.q) + 12.0 * u)
    A = O.OArgs(sliding_window_size=1024)
    # prefill: the last 256 queries of the context
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    r_gpu, f_gpu = _recall(meta.indices.cpu().numpy().reshape(-1, 1, meta.indices.shape[-1])[:, 0], starts)
    r_cpu, f_cpu = _recall(ometa.indices.reshape(-1, 1, ometa.indices.shape[-1])[:, 0], starts)
    assert r_gpu == r_cpu and np.array_equal(f_gpu, f_cpu)
    print(f"  prefill recall {r_gpu:.3f}", flush=True)
    assert r_gpu > 0.5, "planted blocks should dominate the selection"
    # decode: one query at the end of the context
    Xd = O.OInputs("bf16", np.ascontiguousarray(X.q[:, -1:]), np.array([[TK - 1]], dtype=np.int64), k=X.k, v=X.v)
    octx, ometa = O.hip_attention_12(Xd, A)
    ctx, meta = run_product(Xd, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    r_gpu, f_gpu = _recall(meta.indices[:, 0].cpu().numpy(), starts)
    r_cpu, f_cpu = _recall(ometa.indices[:, 0], starts)
    assert r_gpu == r_cpu and np.array_equal(f_gpu, f_cpu)
    print(f"  decode recall {r_gpu:.3f}", flush=True)
    assert r_gpu > 0.5


@pytest.mark.parametrize("page_size", [2, 4, 8, 32])
def test_paged_gather_equals_dense_at_every_page_size(page_size):
    """Paged K/V through a shuffled block table must give what the dense tensors give, bit for bit, at the page
    sizes the reference allows (attention_metadata.py:239; 1 and 16 are covered by the decode cases)."""
    _case(f"paged == dense, page={page_size}")
    # prefill with a ragged last block, and a decode step, on the same keys
    X = make_inputs(83, B=2, TQ=136, TK=4096, H=8, HKV=2, D=128, dtype="bf16")
    A = O.OArgs(sliding_window_size=512, second_stage_k=1024, extend_context_length=4096)
    octx, ometa = O.hip_attention_12(X, A)
    ctx_d, meta_d = run_product(X, A)
    XP = to_paged(X, page_size, seed=page_size)
    ctx_p, meta_p = run_product(XP, A)
    assert_metadata_equal(meta_p, ometa)
    assert torch.equal(meta_p.indices, meta_d.indices) and torch.equal(meta_p.ks, meta_d.ks)
    assert torch.equal(ctx_p.view(torch.int16), ctx_d.view(torch.int16)), "paged context differs from dense"
    assert_context_close(ctx_p, octx, "bf16")
    lens = np.array([4096, 2999])
    Xd = make_inputs(84, B=2, TQ=1, TK=4096, H=8, HKV=2, D=128, dtype="bf16", pos=(lens - 1)[:, None])
    octx, ometa = O.hip_attention_12(Xd, A)
    XPd = to_paged(Xd, page_size, seed=page_size + 1, seq_lens=lens)
    ctx_p, meta_p = run_product(XPd, A)
    assert_metadata_equal(meta_p, ometa)
    assert_context_close(ctx_p, octx, "bf16")
