"""GPU parity: the HIP path against the CPU oracle on identical seeded inputs.

Selected block indices, ks and ks_start_end must match bit for bit; attention outputs within
2e-2 abs / 1e-2 rel (bf16) or 1e-4 (f32).  Everything goes through the C ABI of libhipattn.so.
"""
import copy

import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, tiny_args, to_paged
from gpu_utils import assert_context_close, assert_metadata_equal, run_product, to_torch

pytestmark = pytest.mark.gpu


def _case(name):
    print(f"[case] {name}", flush=True)


def test_config1_tiny_fp32_prefill_full_size():
    """BASELINE config 1: B=1, 512 queries, 4096 keys, 4:1 GQA, D=64, f32, sink 16, window 256."""
    _case("config1 f32")
    X = make_inputs(0, B=1, TQ=512, TK=4096, H=4, HKV=1, D=64, dtype="f32")
    X.v = X.k.copy()
    A = tiny_args()
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert meta.indices.shape == (4, 16, 256)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "f32")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("paged", [False, True])
def test_prefill_ragged_gqa(dtype, paged):
    _case(f"prefill ragged {dtype} paged={paged}")
    # ragged last query block (200 = 6*32 + 8), 2 kv heads, strided query mean
    X = make_inputs(1, B=2, TQ=200, TK=2048, H=8, HKV=2, D=64, dtype=dtype)
    A = tiny_args(sliding_window_size=128, second_stage_k=128)
    if paged:
        X = to_paged(X, 16, seed=3)
        A.extend_context_length = 2048
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)


def test_default_stages_bf16_hid128():
    _case("default stages bf16 D=128")
    # the operator's default hierarchy (256/32/8 chunks, 64-row blocks) on a 16k context, cut-down config 2
    X = make_inputs(2, B=1, TQ=256, TK=16384, H=8, HKV=2, D=128, dtype="bf16")
    A = O.OArgs(sliding_window_size=1024)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert meta.indices.shape == (8, 4, 256)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")


@pytest.mark.parametrize("page_size", [1, 16])
def test_batched_paged_decode(page_size):
    _case(f"paged decode page={page_size}")
    # config 3 in miniature: B sequences of different lengths, q_len 1, shuffled block table
    lens = np.array([3000, 1777, 4096, 2500])
    X = make_inputs(4, B=4, TQ=1, TK=4096, H=8, HKV=2, D=128, dtype="bf16", pos=(lens - 1)[:, None])
    X = to_paged(X, page_size, seed=5, seq_lens=lens)
    A = O.OArgs(sliding_window_size=512, extend_context_length=4096)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    # cached mask reuse on the next step: same indices, decode kernel only
    ctx2, meta2 = run_product(X, A, cached=meta)
    assert torch.equal(meta2.indices, meta.indices)
    assert_context_close(ctx2, octx, "bf16")
    # the query-block kernel on the same decode problem (it attends every selected block once, while the decode
    # path repeats the reference's double visit of the blocks at the seams of its programs: 6 programs of 43 index
    # entries walked in tiles of 2 here)
    assert O.decode_seams(A.second_stage_k, A.sink_token_size, 512, 8, 256) == (43, 1)
    A2 = copy.deepcopy(A); A2.disable_flashdecode = True
    ctx3, _ = run_product(X, A2)
    octx3, _ = O.hip_attention_12(X, A2)
    assert_context_close(ctx3, octx3, "bf16")


@pytest.mark.parametrize("force", ["0", "1"])
def test_prescaled_keys_give_identical_masks(force, monkeypatch):
    _case(f"prescale forced {force}")
    monkeypatch.setenv("HIP_ATTN_PRESCALE_K", force)
    X = make_inputs(9, B=1, TQ=300, TK=8192, H=8, HKV=2, D=128, dtype="bf16")
    A = O.OArgs(sliding_window_size=512)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    XP = to_paged(X, 8, seed=11)
    A.extend_context_length = 8192
    ctx, meta = run_product(XP, A)
    assert_metadata_equal(meta, ometa)


def test_stage_cache_replay_reproduces_output():
    _case("stage cache replay")
    from hip_attn import HiPAttentionOutputMetadata12

    X = make_inputs(6, B=1, TQ=96, TK=4096, H=4, HKV=1, D=64, dtype="f32")
    A = tiny_args()
    ctx, meta = run_product(X, A)
    assert len(meta.stage_caches) == 3
    assert meta.stage_caches[1].indices_left.shape == (1, 3, 4, 128)
    for i in range(3):
        part = HiPAttentionOutputMetadata12(None, None, None, None, None, None, list(meta.stage_caches[: i + 1]))
        ctx_i, meta_i = run_product(X, A, cached=part)
        assert torch.equal(meta_i.indices, meta.indices) and torch.equal(meta_i.ks, meta.ks)
        assert ((ctx - ctx_i) ** 2).sum().item() < 1e-8
        assert len(part.stage_caches) == 3
    # stage caches hold the reference layout and match the oracle's
    _, ometa = O.hip_attention_12(X, A)
    for sc, osc in zip(meta.stage_caches[1:], ometa.stage_caches[1:]):
        assert np.array_equal(sc.indices_left.cpu().numpy(), osc.indices_left)
        assert np.array_equal(sc.indices_right.cpu().numpy(), osc.indices_right)
        assert np.array_equal(sc.out_scores.cpu().numpy(), osc.out_scores)


def test_restart_at_a_stage_with_another_block_size_is_refused():
    """The reference runs a restarted stage with the first stage's query block size and stride, so where they differ
    its restart is not its fresh run; that state raises here instead of returning something else."""
    _case("stage cache restart, block size changes at the restarted stage")
    from hip_attn import HiPAttentionOutputMetadata12

    X = make_inputs(6, B=1, TQ=128, TK=2048, H=2, HKV=1, D=64, dtype="f32")
    A = tiny_args(stages=[O.OStage(64, 2, 64, None, 1), O.OStage(32, 2, 16, 1024, 1), O.OStage(32, 1, 2, 1024, 1)])
    ctx, meta = run_product(X, A)
    part = HiPAttentionOutputMetadata12(None, None, None, None, None, None, list(meta.stage_caches[:2]))
    with pytest.raises(NotImplementedError):
        run_product(X, A, cached=part)
    # stage 2 also runs with blocks of 32 against the first stage's 64: a restart there is refused as well
    part = HiPAttentionOutputMetadata12(None, None, None, None, None, None, list(meta.stage_caches[:3]))
    with pytest.raises(NotImplementedError):
        run_product(X, A, cached=part)


def test_many_query_blocks_use_the_throughput_selection_kernel():
    """More than 64 scan rows: the selection runs in the 256-thread kernel (launches of up to 64 workgroups take the
    1024-thread one, which every small case above exercises)."""
    _case("prefill with 70 query blocks")
    X = make_inputs(17, B=1, TQ=2240, TK=4096, H=2, HKV=1, D=64, dtype="bf16")
    A = tiny_args()
    octx, ometa = O.hip_attention_12(X, A)
    assert ometa.indices.shape[1] == 70
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")


@pytest.mark.parametrize("case", ["chunks 48/12/4", "early terminate 2", "chunks 40/8", "early terminate 4, f32"])
def test_uneven_chunk_sizes_and_early_termination(case):
    """Chunk sizes that are no powers of two make searches of uneven length (ranges of 3, 5, 6 tokens ...), and
    stage_early_terminate cuts the last rounds off: both change which samples of a search repeat, which the scan
    kernel on the matrix cores serves from the round before instead of loading the row again."""
    _case(f"scan {case}")
    dtype = "f32" if "f32" in case else "bf16"
    X = make_inputs(61, B=1, TQ=100, TK=3000, H=4, HKV=2, D=64, dtype=dtype)
    if case == "chunks 48/12/4":
        A = tiny_args(stages=[O.OStage(32, 2, 48, None, 1), O.OStage(32, 2, 12, 1536, 1), O.OStage(32, 1, 4, 768, 1)])
    elif case == "chunks 40/8":
        A = tiny_args(stages=[O.OStage(32, 2, 40, None, 1), O.OStage(32, 1, 8, 1000, 1)], second_stage_k=600)
    else:
        A = tiny_args(stage_early_terminate=4 if "4" in case else 2)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)


def test_wide_scan_with_64_query_rows_walks_chunk_groups_in_a_loop():
    """16384 and more scan programs with 64 query rows: a wave of the scan kernel keeps its query fragments and walks
    eight chunk groups; 2050 chunks make 33 groups of 64, so the last wave of a row walks one group that holds two
    chunks.  (The oracle needs about 20 s of CPU time for this shape.)"""
    _case("wide scan, 64 rows, 33 chunk groups")
    TK = 16 + 128 + 2050 * 4
    X = make_inputs(71, B=1, TQ=2048, TK=TK, H=16, HKV=4, D=32, dtype="bf16")
    A = tiny_args(stages=[O.OStage(64, 1, 4, None, 1)], sliding_window_size=128, second_stage_k=256,
                  block_sparse_block_size_q=64)
    octx, ometa = O.hip_attention_12(X, A)
    print("  oracle done", flush=True)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")


def test_head_reduce_off_matches_oracle(monkeypatch):
    _case("head reduce off")
    monkeypatch.setenv("HIP_HEAD_REDUCE", "0")
    X = make_inputs(7, B=1, TQ=64, TK=2048, H=4, HKV=2, D=64, dtype="bf16")
    A = tiny_args(sliding_window_size=128, second_stage_k=128)
    A.head_reduce = False
    A.disable_flashdecode = True
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    per_head = meta.indices.view(1, 4, *meta.indices.shape[1:])
    assert not torch.equal(per_head[:, 0], per_head[:, 1])  # heads really select differently here
    assert_context_close(ctx, octx, "bf16")


def test_short_context_and_mask_only():
    _case("short context")
    # fewer keys than sink + window: no candidate chunks at all -> streaming attention
    X = make_inputs(8, B=1, TQ=40, TK=200, H=2, HKV=1, D=32, dtype="f32")
    A = tiny_args()
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert meta.indices.shape[-1] == 0 and (meta.ks == 0).all()
    assert_context_close(ctx, octx, "f32")
    A.mask_only = True
    assert run_product(X, A) == (None, None)


def test_operator_with_logit_softcap():
    _case("operator softcap")
    X = make_inputs(44, B=1, TQ=128, TK=2048, H=4, HKV=2, D=64, dtype="bf16", scale=1.5)
    A = tiny_args(logit_softcap=4.0)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)  # the cap never touches mask estimation
    assert_context_close(ctx, octx, "bf16")
    plain, _ = O.hip_attention_12(X, tiny_args())
    assert np.abs(O.bf16_bits_to_f32(plain) - O.bf16_bits_to_f32(octx)).max() > 0.05


def test_head_dim_256_with_softcap_like_gemma2():
    _case("operator D=256 softcap")
    X = make_inputs(45, B=1, TQ=160, TK=2048, H=4, HKV=2, D=256, dtype="bf16", scale=0.7)
    A = tiny_args(logit_softcap=50.0, block_size_k=32)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")


DENSE_CASES = {
    # name: (B, TQ, TK, H, HKV, D, stages, kwargs)
    "chunks 64/16/2, 16 and 32 rows, G=4": (1, 200, 4096, 8, 2, 64,
                                            [O.OStage(32, 2, 64, None, 1), O.OStage(32, 2, 16, 2048, 1), O.OStage(32, 1, 2, 1024, 1)], {}),
    "chunks 256/32/8, 64 rows, D=128, G=4": (1, 300, 12288, 8, 2, 128,
                                             [O.OStage(64, 4, 256, None, 1), O.OStage(64, 4, 32, 8192, 1), O.OStage(64, 1, 8, 2048, 1)],
                                             dict(sliding_window_size=512, sink_token_size=64, second_stage_k=1024)),
    "chunks 64/8/4, G=2, early terminate 2": (2, 100, 3000, 4, 2, 64,
                                              [O.OStage(32, 1, 64, None, 1), O.OStage(32, 1, 8, 1024, 1), O.OStage(32, 1, 4, 512, 1)],
                                              dict(stage_early_terminate=2, second_stage_k=256)),
    "chunks 128/16/4 with 16 chunks per program": (1, 64, 2500, 4, 1, 128,
                                                   [O.OStage(64, 1, 128, None, 1), O.OStage(64, 2, 16, 1024, 1), O.OStage(32, 1, 4, 256, 1)],
                                                   dict(block_size_k=16, second_stage_k=128, sliding_window_size=256)),
}


@pytest.mark.parametrize("paged", [0, 16, 4, 1])
@pytest.mark.parametrize("case", list(DENSE_CASES))
def test_small_chunk_stages_scored_densely(case, paged, monkeypatch):
    """Stages with chunks of 2 .. 16 tokens on prescaled keys can score every token of every chunk once per GQA group
    and replay the searches on the scores; forced here on small problems (the operator picks that kernel by itself
    only on wide launches).  Indices, ks and the access flags must equal the oracle's, which samples."""
    _case(f"dense scan: {case}, paged={paged}")
    monkeypatch.setenv("HIPATTN_MASK_DENSE", "2")
    monkeypatch.setenv("HIP_ATTN_PRESCALE_K", "1")
    B, TQ, TK, H, HKV, D, stages, kw = DENSE_CASES[case]
    X = make_inputs(500 + list(DENSE_CASES).index(case), B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16")
    A = tiny_args(stages=stages, **kw)
    if paged:  # page size; the pages of the token slots are looked up a pass of tiles ahead
        X = to_paged(X, paged, seed=7)
        A.extend_context_length = TK
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    # and the sampling kernels on the same input, for the access flags of a run that cannot be compared directly
    monkeypatch.setenv("HIPATTN_MASK_DENSE", "0")
    ctx2, meta2 = run_product(X, A)
    assert torch.equal(meta2.indices, meta.indices)
    assert torch.equal(meta2.mask_cache_statistics.access_counter, meta.mask_cache_statistics.access_counter)


@pytest.mark.parametrize("layout", ["dense", "page 16", "page 1"])
def test_single_token_scans_with_coalesced_row_fetch(layout, monkeypatch):
    """Decode launches of many waves fetch the sampled rows coalesced, straight into LDS, from keys as stored; forced
    here on a small batch (HIPATTN_MASK_DMA_INLINE=1).  Masks and access flags must equal the oracle's and those of
    the launches that load a half row per lane."""
    _case(f"coalesced single-token scans, {layout}")
    lens = np.array([3000, 1777, 4096, 2500])
    if layout == "dense":
        X = make_inputs(14, B=2, TQ=1, TK=4096, H=8, HKV=2, D=128, dtype="bf16", pos=np.array([[4095], [4095]]))
        A = O.OArgs(sliding_window_size=512)
    else:
        X = make_inputs(4, B=4, TQ=1, TK=4096, H=8, HKV=2, D=128, dtype="bf16", pos=(lens - 1)[:, None])
        X = to_paged(X, int(layout.split()[1]), seed=5, seq_lens=lens)
        A = O.OArgs(sliding_window_size=512, extend_context_length=4096)
    octx, ometa = O.hip_attention_12(X, A)
    monkeypatch.setenv("HIPATTN_MASK_DMA_INLINE", "1")
    ctx, meta = run_product(X, A, require_cache_statistics=True)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    monkeypatch.setenv("HIPATTN_MASK_DMA_INLINE", "0")
    ctx0, meta0 = run_product(X, A, require_cache_statistics=True)
    assert torch.equal(meta0.indices, meta.indices)
    assert torch.equal(meta0.mask_cache_statistics.access_counter, meta.mask_cache_statistics.access_counter)


@pytest.mark.parametrize("m16", ["0", "1"])
@pytest.mark.parametrize("paged", [0, 16])
def test_prefill_scans_with_coalesced_row_fetch_on_a_small_launch(paged, m16, monkeypatch):
    """The coalesced fetch of the wide prefill launches (prescaled keys; 32-bit row offsets on a dense tensor, 64-bit
    ones on a paged cache), forced on a launch of a few hundred programs (HIPATTN_MASK_DMA=2): ragged candidate
    lists, a wave walking past the end of its chunk groups, statistics flags."""
    _case(f"coalesced prefill scans on a small launch, paged={paged}, 16x16x32 products={m16}")
    # m16: the products of 16-row programs on v_mfma_f32_16x16x32_bf16 with its groups of eight elements in the order
    # of two 32x32x16 steps: the same bits
    monkeypatch.setenv("HIPATTN_MASK_M16", m16)
    monkeypatch.setenv("HIP_ATTN_PRESCALE_K", "1")
    monkeypatch.setenv("HIPATTN_MASK_DENSE", "0")
    X = make_inputs(15, B=2, TQ=300, TK=8192, H=8, HKV=2, D=128, dtype="bf16")
    A = O.OArgs(sliding_window_size=512)
    if paged:
        X = to_paged(X, paged, seed=13)
        A.extend_context_length = 8192
    octx, ometa = O.hip_attention_12(X, A)
    monkeypatch.setenv("HIPATTN_MASK_DMA", "2")
    ctx, meta = run_product(X, A, require_cache_statistics=True)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    monkeypatch.setenv("HIPATTN_MASK_DMA", "0")
    ctx0, meta0 = run_product(X, A, require_cache_statistics=True)
    assert torch.equal(meta0.indices, meta.indices)
    assert torch.equal(meta0.mask_cache_statistics.access_counter, meta.mask_cache_statistics.access_counter)


@pytest.mark.parametrize("scan", ["relative", "infllm", "streaming"])
@pytest.mark.parametrize("paged", [0, 16])
def test_coalesced_prefill_scans_on_keys_rotated_ahead(paged, scan, monkeypatch):
    """RoPE on load under the rules with fixed key positions: the keys are rotated and scaled ahead of the scan, one
    copy per sample side under ``relative``, and the coalesced fetch takes a right-hand sample from the second copy
    (forced on a small launch, both widths of the matrix instruction).  A score then belongs to (token, side): a lane
    may not take a repeated token's score from its partner of the other side.  Under ``streaming`` a key's position is
    the place of its chunk in the stage's list, which for the first stage of a dense tensor is known ahead too: that
    stage reads a copy rotated per token (a paged cache keeps the rotation in the kernel)."""
    from helpers import with_rope

    _case(f"coalesced prefill scans on keys rotated ahead, scan={scan}, paged={paged}")
    monkeypatch.setenv("HIP_ATTN_PRESCALE_K", "1")
    monkeypatch.setenv("HIPATTN_MASK_DENSE", "0")
    X = make_inputs(17, B=2, TQ=300, TK=8192, H=8, HKV=2, D=128, dtype="bf16", scale=0.5)
    kw = dict(sliding_window_size=512, using_extend=True, need_apply_rope=True, scan_extend_backend=scan,
              sa_extend_backend="streaming")
    if paged:
        X = to_paged(X, paged, seed=14)
        kw["extend_context_length"] = 8192
    X = with_rope(X, 16384)
    A = O.OArgs(**kw)
    octx, ometa = O.hip_attention_12(X, A)
    res = {}
    for m16 in ("0", "1"):
        monkeypatch.setenv("HIPATTN_MASK_M16", m16)
        monkeypatch.setenv("HIPATTN_MASK_DMA", "2")
        ctx, meta = run_product(X, A, require_cache_statistics=True)
        assert_metadata_equal(meta, ometa)
        assert_context_close(ctx, octx, "bf16")
        res[m16] = meta
    monkeypatch.setenv("HIPATTN_MASK_DMA", "0")
    ctx0, meta0 = run_product(X, A, require_cache_statistics=True)
    assert torch.equal(meta0.indices, res["0"].indices)
    assert torch.equal(meta0.mask_cache_statistics.access_counter, res["1"].mask_cache_statistics.access_counter)


def test_key_buffers_reported_as_spanning_32_gib_take_the_plain_scans(monkeypatch):
    """The flag that keeps launches off the coalesced variants (rows passed between lanes as 31-bit piece numbers)
    when a key buffer is too large for them: forced here on a small problem, prefill and decode."""
    _case("far rows flag")
    from hip_attn import operator as op

    monkeypatch.setenv("HIP_ATTN_PRESCALE_K", "1")
    monkeypatch.setenv("HIPATTN_MASK_DMA", "2")
    X = make_inputs(16, B=1, TQ=200, TK=8192, H=8, HKV=2, D=128, dtype="bf16")
    A = O.OArgs(sliding_window_size=512)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A, require_cache_statistics=True)
    monkeypatch.setattr(op, "_spans_32_gib", lambda t: True)
    ctx_far, meta_far = run_product(X, A, require_cache_statistics=True)
    assert_metadata_equal(meta_far, ometa)
    assert torch.equal(meta_far.indices, meta.indices)
    assert torch.equal(meta_far.mask_cache_statistics.access_counter, meta.mask_cache_statistics.access_counter)
    assert_context_close(ctx_far, octx, "bf16")
    Xd = make_inputs(17, B=2, TQ=1, TK=4096, H=8, HKV=2, D=128, dtype="bf16", pos=np.array([[4095], [4095]]))
    octx, ometa = O.hip_attention_12(Xd, A)
    ctx_far, meta_far = run_product(Xd, A)
    assert_metadata_equal(meta_far, ometa)
    assert_context_close(ctx_far, octx, "bf16")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_non_causal_operator_prefill_and_decode(dtype):
    """is_causal = False end to end: mask estimation is unchanged (the scan knows no such switch), attention drops its
    position tests."""
    print(f"[case] operator non-causal {dtype}", flush=True)
    X = make_inputs(71, B=2, TQ=200, TK=2048, H=4, HKV=2, D=64, dtype=dtype, scale=0.5)
    A = tiny_args(is_causal=False)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)
    cctx, _ = O.hip_attention_12(X, tiny_args())
    wid = (lambda a: O.bf16_bits_to_f32(a)) if dtype == "bf16" else (lambda a: a)
    assert np.abs(wid(cctx) - wid(octx)).max() > 1e-2
    lens = np.array([2048, 1500])
    XD = make_inputs(72, B=2, TQ=1, TK=2048, H=4, HKV=2, D=64, dtype=dtype, pos=(lens - 1)[:, None], scale=0.5)
    XP = to_paged(XD, 16, seed=4, seq_lens=lens)
    A = tiny_args(is_causal=False, extend_context_length=2048)
    octx, ometa = O.hip_attention_12(XP, A)
    ctx, meta = run_product(XP, A)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, dtype)


def test_caller_kept_prescaled_keys_change_nothing_but_the_time():
    """``HiPAttentionArgs.k_prescaled`` (an extension): mask estimation reads bf16(K * c_k) from a copy the caller keeps
    instead of scaling every sampled row; indices, flags and context must be what they are without it.  Decode on a
    dense tensor and on a paged cache, and a prefill."""
    from hip_attn import prescale_keys

    print("[case] caller-kept prescaled keys", flush=True)
    lens = np.array([4096, 3000])
    XD = make_inputs(81, B=2, TQ=1, TK=4096, H=8, HKV=2, D=128, dtype="bf16", pos=(lens - 1)[:, None])
    A = O.OArgs(sliding_window_size=512)
    octx, ometa = O.hip_attention_12(XD, A)
    for head_major in (True, False):
        khat = prescale_keys(to_torch(XD.k, "bf16"), head_major=head_major)
        ctx, meta = run_product(XD, A, k_prescaled=khat)
        assert_metadata_equal(meta, ometa)
        assert_context_close(ctx, octx, "bf16")
    XP = to_paged(XD, 16, seed=6, seq_lens=lens)
    A = O.OArgs(sliding_window_size=512, extend_context_length=4096)
    octx, ometa = O.hip_attention_12(XP, A)
    khat = prescale_keys(to_torch(XP.k_cache, "bf16"))
    ctx, meta = run_product(XP, A, k_prescaled=khat)
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    X = make_inputs(82, B=1, TQ=256, TK=4096, H=8, HKV=2, D=128, dtype="bf16")
    A = O.OArgs(sliding_window_size=512)
    octx, ometa = O.hip_attention_12(X, A)
    ctx, meta = run_product(X, A, k_prescaled=prescale_keys(to_torch(X.k, "bf16")))
    assert_metadata_equal(meta, ometa)
    assert_context_close(ctx, octx, "bf16")
    with pytest.raises(ValueError):
        run_product(X, A, k_prescaled=prescale_keys(to_torch(X.k, "bf16"))[:, :100])
