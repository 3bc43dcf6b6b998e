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
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "reference_*.npz")))


def load_case(path):
    d = np.load(path)
    bf16 = bool(int(d["bf16"]))
    dtype = "bf16" if bf16 else "f32"
    # q, k, v are stored as the upper 16 bits of their float32 patterns (the lower 16 are zero)
    conv = (lambda a: a) if bf16 else (lambda a: (a.astype(np.uint32) << 16).view(np.float32))
    stages = [O.OStage(int(a), int(b), int(c), None if e < 0 else int(e), int(f)) for a, b, c, e, f in d["stages"]]
    kw = dict(sink_token_size=int(d["sink"]), sliding_window_size=int(d["sw"]), second_stage_k=int(d["second_k"]),
              block_sparse_block_size_q=int(d["bsbq"]), stages=stages, block_size_k=int(d["block_size_k"]))
    pos = np.ascontiguousarray(d["pos"], dtype=np.int64)
    if "k_cache" in d.files:
        X = O.OInputs(dtype, conv(d["q"]), pos, k_cache=conv(d["k_cache"]), v_cache=conv(d["v_cache"]),
                      block_table=d["block_table"].astype(np.int64), cache_seq_lens=d["cache_seq_lens"].astype(np.int64))
        kw["extend_context_length"] = int(d["max_tsrc"])
    else:
        X = O.OInputs(dtype, conv(d["q"]), pos, k=conv(d["k"]), v=conv(d["v"]))
    if "rope_cos" in d.files:
        X.rope_cos, X.rope_sin = d["rope_cos"].astype(np.float32), d["rope_sin"].astype(np.float32)
        kw.update(using_extend=True, need_apply_rope=True, scan_extend_backend=str(d["scan_backend"]),
                  sa_extend_backend=str(d["sa_backend"]))
    if "softcap" in d.files:
        kw["logit_softcap"] = float(d["softcap"])
    return d, X, O.OArgs(**kw), dtype


def test_fixtures_are_present():
    names = {os.path.basename(f) for f in FIXTURES}
    assert {"reference_f32_prefill_tiny.npz", "reference_f32_prefill_gqa_ragged.npz", "reference_f32_decode_paged.npz",
            "reference_f32_prefill_rope_relative.npz", "reference_f32_prefill_rope_streaming.npz",
            "reference_f32_decode_rope_infllm.npz", "reference_f32_prefill_stride_d64.npz",
            "reference_f32_decode_default_stages.npz"} <= names


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
