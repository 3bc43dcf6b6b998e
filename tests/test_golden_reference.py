"""The oracle against vectors produced by an execution of the reference's own v1.2 code.

``tests/golden/reference_*.npz`` hold inputs and the outputs of ``dual_stage_quadratic_hip_attention`` run from the
reference checkout under Triton's CPU interpreter (``tests/golden/make_reference_fixtures.py``).  The oracle must
reproduce the selected block indices, ``ks`` and ``ks_start_end`` exactly and the context within float32 round-off
(the interpreter's dot products are NumPy's, so only their accumulation order differs from the oracle's).
"""
import glob
import os

import numpy as np
import pytest

from oracle import hip12 as O

HERE = os.path.dirname(os.path.abspath(__file__))
_ALL = sorted(glob.glob(os.path.join(HERE, "golden", "reference_*.npz")))
FIXTURES = [f for f in _ALL if "_paged_api_" not in f]      # calls of dual_stage_quadratic_hip_attention
API_FIXTURES = [f for f in _ALL if "_paged_api_" in f]      # calls of forward_paged_hip


def load_case(path):
    d = np.load(path)
    bf16 = bool(int(d["bf16"]))
    dtype = "bf16" if bf16 else "f32"
    # q, k, v are stored as the upper 16 bits of their float32 patterns (the lower 16 are zero)
    conv = (lambda a: a) if bf16 else (
        lambda a: np.ascontiguousarray(a) if a.dtype == np.float32 else (a.astype(np.uint32) << 16).view(np.float32))
    stages = [O.OStage(int(a), int(b), int(c), None if e < 0 else int(e), int(f)) for a, b, c, e, f in d["stages"]]
    kw = dict(sink_token_size=int(d["sink"]), sliding_window_size=int(d["sw"]), second_stage_k=int(d["second_k"]),
              block_sparse_block_size_q=int(d["bsbq"]), stages=stages, block_size_k=int(d["block_size_k"]))
    pos = np.ascontiguousarray(d["pos"], dtype=np.int64)
    if "k_cache" in d.files:
        X = O.OInputs(dtype, conv(d["q"]), pos, k_cache=conv(d["k_cache"]), v_cache=conv(d["v_cache"]),
                      block_table=d["block_table"].astype(np.int64), cache_seq_lens=d["cache_seq_lens"].astype(np.int64))
        kw["extend_context_length"] = int(d["max_tsrc"])
    else:
        X = O.OInputs(dtype, conv(d["q"]), pos, k=conv(d["k"]), v=conv(d["k" if "v_is_k" in d.files else "v"]))
    if "rope_cos" in d.files:
        X.rope_cos, X.rope_sin = d["rope_cos"].astype(np.float32), d["rope_sin"].astype(np.float32)
        kw.update(using_extend=True, need_apply_rope=True, scan_extend_backend=str(d["scan_backend"]),
                  sa_extend_backend=str(d["sa_backend"]))
    if "model_context_length" in d.files:
        kw["model_context_length"] = int(d["model_context_length"])
    if "softcap" in d.files:
        kw["logit_softcap"] = float(d["softcap"])
    if "stage_early_terminate" in d.files:
        kw["stage_early_terminate"] = int(d["stage_early_terminate"])
    if "is_causal" in d.files:
        kw["is_causal"] = bool(int(d["is_causal"]))
    return d, X, O.OArgs(**kw), dtype


def _flags(d, name, suffix=""):
    if f"{name}{suffix}" not in d.files:
        return None
    shape = tuple(int(x) for x in d[f"{name}_shape{suffix}"])
    return np.unpackbits(d[f"{name}{suffix}"])[: int(np.prod(shape))].reshape(shape).astype(bool)


def test_fixtures_are_present():
    names = {os.path.basename(f) for f in _ALL}
    assert {"reference_f32_prefill_tiny.npz", "reference_f32_prefill_gqa_ragged.npz", "reference_f32_decode_paged.npz",
            "reference_f32_prefill_rope_relative.npz", "reference_f32_prefill_rope_streaming.npz",
            "reference_f32_decode_rope_infllm.npz", "reference_f32_prefill_stride_d64.npz",
            "reference_f32_prefill_rope_dynamic.npz", "reference_f32_decode_rope_dynamic.npz",
            "reference_f32_decode_default_stages.npz", "reference_f32_paged_api_prefill.npz",
            "reference_f32_smallest_benchmark_prefill.npz", "reference_f32_prefill_non_causal.npz",
            "reference_f32_decode_non_causal.npz", "reference_f32_prefill_rope_self_extend.npz",
            "reference_f32_paged_api_decode_rope.npz"} <= names


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(f)[10:-4] for f in FIXTURES])
def test_oracle_reproduces_the_reference_run(path):
    d, X, A, dtype = load_case(path)
    ctx, meta = O.hip_attention_12(X, A)
    assert np.array_equal(meta.indices, d["indices"]), f"{int((meta.indices != d['indices']).sum())} index entries differ"
    assert np.array_equal(meta.ks, d["ks"])
    assert np.array_equal(meta.ks_start_end, d["ks_start_end"])
    got = O.bf16_bits_to_f32(ctx) if dtype == "bf16" else ctx
    tol = 2e-2 if dtype == "bf16" else 5e-5
    assert np.abs(got - d["context"]).max() <= tol, np.abs(got - d["context"]).max()
    # which key rows the mask estimation and the attention touched
    for name, mine in (("mask_access", meta.mask_access), ("sa_access", meta.sa_access)):
        want = _flags(d, name)
        assert want is not None and want.shape == mine.shape
        assert np.array_equal(mine > 0, want), f"{name}: {int(((mine > 0) != want).sum())} flags differ"
    if "context_replay" in d.files:  # restart from the cached inputs of stage 1
        part = O.OMetadata(None, None, None, None, stage_caches=list(meta.stage_caches[:2]))
        ctx_r, meta_r = O.hip_attention_12(X, A, cached=part)
        assert np.array_equal(meta_r.indices, d["indices_replay"])
        assert np.abs(ctx_r - d["context_replay"]).max() <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(f)[10:-4] for f in FIXTURES])
def test_gpu_reproduces_the_reference_run(path):
    """The HIP path against the reference's own outputs, without the oracle in between."""
    from gpu_utils import assert_context_close, run_product

    print(f"[case] reference run {os.path.basename(path)}", flush=True)
    d, X, A, dtype = load_case(path)
    ctx, meta = run_product(X, A)
    assert np.array_equal(meta.indices.cpu().numpy(), d["indices"])
    assert np.array_equal(meta.ks.cpu().numpy(), d["ks"])
    assert np.array_equal(meta.ks_start_end.cpu().numpy(), d["ks_start_end"])
    want = O.f32_to_bf16_bits(d["context"]) if dtype == "bf16" else d["context"]
    assert_context_close(ctx, want, dtype)
    for name, st in (("mask_access", meta.mask_cache_statistics), ("sa_access", meta.sa_cache_statistics)):
        flags = _flags(d, name)
        got = st.access_counter.cpu().numpy() > 0
        assert got.shape == flags.shape and np.array_equal(got, flags), name


# ---------------------------------------------------------------- forward_paged_hip (paged_hip.py:35-320)

def _widen16(a):
    return (a.astype(np.uint32) << 16).view(np.float32)


def _api_oracle_inputs(d, layer_id):
    """The arguments ``_forward_paged_hip`` builds for this layer (paged_hip.py:356-452), as oracle inputs."""
    import json

    spec = json.loads(bytes(d["spec"]).decode())
    TQ = int(d["TQ"])
    kc, vc = _widen16(d["k_cache"]), _widen16(d["v_cache"])
    q = _widen16(d["q"])
    B, _, H, D = q.shape
    dense = layer_id in spec["dense_layers"]
    layer = spec["layers" if TQ == 1 else "prefill_layers"][0 if dense else 1]
    q = (q * np.float32(D ** -0.5)).astype(np.float32)
    X = O.OInputs("f32", q, d["positions"].astype(np.int64), k_cache=np.ascontiguousarray(kc[:, None]),
                  v_cache=np.ascontiguousarray(vc[:, None]),
                  block_table=d["req_to_tokens"][d["req_pool_indices"]].astype(np.int64),
                  cache_seq_lens=d["seq_lens"].astype(np.int64))
    kw = dict(sliding_window_size=layer.get("sliding_window_size", 1024), second_stage_k=layer.get("second_stage_k", 2048),
              sink_token_size=layer.get("sink_token_size", 256),
              extend_context_length=int(d["max_context_len"]), model_context_length=int(d["orig_context_len"]),
              disable_flashdecode=TQ != 1)
    if spec.get("using_extend", True):
        X.rope_cos, X.rope_sin = _widen16(d["rope_cos"]), _widen16(d["rope_sin"])
        kw.update(using_extend=True, need_apply_rope=True, scan_extend_backend="streaming" if dense else "relative",
                  sa_extend_backend="streaming")
    return X, O.OArgs(**kw)


def _sub(X, sl):
    Y = O.OInputs(X.dtype, np.ascontiguousarray(X.q[:, sl]), np.ascontiguousarray(X.pos[:, sl]), k_cache=X.k_cache,
                  v_cache=X.v_cache, block_table=X.block_table, cache_seq_lens=X.cache_seq_lens)
    Y.rope_cos, Y.rope_sin = X.rope_cos, X.rope_sin
    return Y


@pytest.mark.parametrize("path", API_FIXTURES, ids=[os.path.basename(f)[10:-4] for f in API_FIXTURES])
def test_oracle_reproduces_the_serving_entry_point(path):
    d = np.load(path)
    TQ = int(d["TQ"])
    for layer_id in d["layer_ids"]:
        X, A = _api_oracle_inputs(d, int(layer_id))
        B, _, H, D = X.q.shape
        want = d[f"o_{layer_id}"].reshape(B, TQ, H, D)
        if TQ == 1 or TQ < 128:
            ctx, meta = O.hip_attention_12(X, A)
        else:  # the last 64 queries are served by a second call whose window takes what the context length leaves
            ctx1, _ = O.hip_attention_12(_sub(X, slice(None, -64)), A)
            ctx2, meta = O.hip_attention_12(_sub(X, slice(-64, None)), O.OArgs(**{**A.__dict__, "sliding_window_size": 777}))
            ctx = np.concatenate([ctx1, ctx2], axis=1)
        assert np.array_equal(meta.indices, d[f"indices_{layer_id}"])
        assert np.array_equal(meta.ks, d[f"ks_{layer_id}"])
        assert np.abs(ctx - want).max() <= 5e-5, np.abs(ctx - want).max()
        for name, mine in (("mask_access", meta.mask_access), ("sa_access", meta.sa_access)):
            flags = _flags(d, name, f"_{layer_id}")  # of the last call
            assert flags.shape == mine.shape and np.array_equal(mine > 0, flags), name
        if TQ == 1:
            ctx2, _ = O.hip_attention_12(X, A, cached=meta)
            assert np.abs(ctx2 - d[f"o_cached_{layer_id}"].reshape(B, 1, H, D)).max() <= 5e-5


@pytest.mark.gpu
@pytest.mark.parametrize("path", API_FIXTURES, ids=[os.path.basename(f)[10:-4] for f in API_FIXTURES])
def test_gpu_reproduces_the_serving_entry_point(path):
    import torch

    from gpu_utils import assert_context_close
    from hip_attn import HiPAttentionConfig, forward_paged_hip

    print(f"[case] reference serving call {os.path.basename(path)}", flush=True)
    d = np.load(path)
    TQ = int(d["TQ"])
    dev = "cuda"
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    q = t(_widen16(d["q"]))
    B, _, H, D = q.shape
    cfg = HiPAttentionConfig(json_or_path=bytes(d["spec"]).decode())
    rope = "rope_cos" in d.files
    kw = dict(sm_scale=D ** -0.5, batch_size=B, k_cache=t(_widen16(d["k_cache"])), v_cache=t(_widen16(d["v_cache"])),
              offload_cache=None, positions=t(d["positions"].reshape(-1)), seq_lens=t(d["seq_lens"]),
              req_to_tokens=t(d["req_to_tokens"]), req_pool_indices=t(d["req_pool_indices"]),
              rope_cos=t(_widen16(d["rope_cos"])) if rope else None, rope_sin=t(_widen16(d["rope_sin"])) if rope else None,
              logit_cap=0.0, orig_context_len=int(d["orig_context_len"]), max_context_len=int(d["max_context_len"]),
              is_prefill=TQ != 1, hip_config=cfg, is_decode=TQ == 1)
    for layer_id in d["layer_ids"]:
        o, meta = forward_paged_hip(q.reshape(B * TQ, H, D), layer_id=int(layer_id), **kw)
        assert np.array_equal(meta.indices.cpu().numpy(), d[f"indices_{layer_id}"])
        assert np.array_equal(meta.ks.cpu().numpy(), d[f"ks_{layer_id}"])
        assert_context_close(o.reshape(B, TQ, H, D), d[f"o_{layer_id}"].reshape(B, TQ, H, D), "f32")
        for name, st in (("mask_access", meta.mask_cache_statistics), ("sa_access", meta.sa_cache_statistics)):
            flags = _flags(d, name, f"_{layer_id}")
            got = st.access_counter.cpu().numpy() > 0
            assert got.shape == flags.shape and np.array_equal(got, flags), name
        if TQ == 1:
            o2, _ = forward_paged_hip(q.reshape(B * TQ, H, D), layer_id=int(layer_id), cached_metadata=meta, **kw)
            assert_context_close(o2.reshape(B, TQ, H, D), d[f"o_cached_{layer_id}"].reshape(B, TQ, H, D), "f32")


def test_metadata_pool_layout_equals_the_reference_pool():
    """Buffer names, shapes, storage and view dtypes and batch formats of ``HiPMetadataCachePool`` as the reference's
    class allocates them for the same configuration (hip_memory_pool.py:55-222)."""
    import json

    import torch

    from hip_attn import HiPAttentionConfig, HiPMetadataCachePool

    with open(os.path.join(HERE, "golden", "reference_metadata_pool_layout.json")) as f:
        ref = json.load(f)
    pool = HiPMetadataCachePool(max_total_num_tokens=1 << 20, query_head_num=ref["heads"], layer_num=ref["layers"],
                                context_length=ref["context_length"], device="cpu",
                                hip_config=HiPAttentionConfig(json_or_path=ref["spec"]))
    assert len(pool.cache) == len(ref["layout"])
    for mine, theirs in zip(pool.cache, ref["layout"]):
        assert set(mine) == set(theirs)
        for name, want in theirs.items():
            b = mine[name]
            got = dict(shape=list(b.buffer.shape), store=str(b.buffer.dtype), dtype=str(b.dtype), format=b.batch_format)
            assert got == want, name
    assert pool.allocated_gpu_bytes == ref["allocated_bytes"]
